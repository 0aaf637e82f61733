"""hb_fused_step_noalloc, the entry point whose caution counters live in the library's own device array, against
hb_fused_step on identical inputs: every buffer bit for bit, on two calls in a row, the second on a smaller set of
tensors (the array keeps the first call's counts, so a missed clear would show).  Both run through the C ABI."""

import ctypes

import numpy as np
import pytest
import torch

from heavyball_amd import _lib
from heavyball_amd.slab import chunk_table, layout

pytestmark = pytest.mark.gpu

CASES = {
    # (param_fmt, grad_fmt, state_fmt, algo, flags): the formats of the 8B-shaped configuration, and plain fp32
    "adamw_mars_caution_ecc_paramecc": (_lib.FMT_ECC_BF16_8, _lib.FMT_BF16, _lib.FMT_ECC_BF16_8, _lib.ALGO_ADAM,
                                        _lib.FLAG_MARS | _lib.FLAG_CAUTION),  # fmt: skip
    "laprop_caution_fp32": (_lib.FMT_F32, _lib.FMT_F32, _lib.FMT_F32, _lib.ALGO_LAPROP, _lib.FLAG_CAUTION | _lib.FLAG_CAUTIOUS_WD),
}
PRIM = {_lib.FMT_F32: torch.float32, _lib.FMT_BF16: torch.bfloat16, _lib.FMT_ECC_BF16_8: torch.bfloat16}


class Roles:
    """The flat role buffers of one slab, filled from a seed."""

    def __init__(self, numels, pf, gf, sf, seed, dev):
        self.numels = list(numels)
        self.offsets, self.total = layout(self.numels)
        g = torch.Generator().manual_seed(seed)

        def role(fmt, scale):
            prim = (torch.randn(self.total, generator=g) * scale).to(PRIM[fmt]).to(dev)
            corr = torch.randint(-127, 128, (self.total,), generator=g, dtype=torch.int8).to(dev) if fmt == _lib.FMT_ECC_BF16_8 else None
            return prim, corr

        self.param, self.param_corr = role(pf, 0.02)
        self.grad, _ = role(gf, 1e-3)
        self.m, self.m_corr = role(sf, 1e-3)
        self.v, self.v_corr = role(sf, 1e-3)
        self.v = self.v.abs()
        self.og, self.og_corr = role(sf, 1e-3)
        self.off_dev = torch.from_numpy(self.offsets.copy()).to(dev)
        self.numel_dev = torch.tensor(self.numels, dtype=torch.int64, device=dev)
        # hb_fused_step's caller-owned scratch
        self.counts = torch.full((len(self.numels) * _lib.CAUTION_SLOTS,), 12345, dtype=torch.int32, device=dev)

    def buffers(self):
        return {k: getattr(self, k) for k in ("param", "param_corr", "m", "m_corr", "v", "v_corr", "og", "og_corr") if getattr(self, k) is not None}

    def desc(self, active, pf, gf, sf, algo, flags, step, with_counts):
        tab = chunk_table(self.numels, active)
        self.chunks = torch.from_numpy(tab).to(self.param.device)
        d = _lib.HbStepDesc()
        ptr = lambda t: None if t is None else t.data_ptr()  # noqa: E731
        d.param, d.param_corr = ptr(self.param), ptr(self.param_corr)
        d.grad, d.grad_ptrs = ptr(self.grad), None
        d.exp_avg, d.exp_avg_corr = ptr(self.m), ptr(self.m_corr)
        d.exp_avg_sq, d.exp_avg_sq_corr = ptr(self.v), ptr(self.v_corr)
        if flags & _lib.FLAG_MARS:
            d.old_grad, d.old_grad_corr = ptr(self.og), ptr(self.og_corr)
        d.offsets, d.numel, d.chunks = self.off_dev.data_ptr(), self.numel_dev.data_ptr(), self.chunks.data_ptr()
        d.caution_count = self.counts.data_ptr() if with_counts else None
        d.n_chunks, d.n_tensors = int(tab.shape[0]), len(self.numels)
        d.algo, d.flags = algo, flags
        d.param_fmt, d.grad_fmt, d.state_fmt = pf, gf, sf
        f = np.float32
        d.a1, d.a2 = float(f(0.1)), float(f(0.01))
        d.one_minus_a1, d.one_minus_a2 = float(f(1) - f(0.1)), float(f(1) - f(0.01))
        d.mars_a = float(f(-0.0022556))
        d.one_minus_mars_a = float(f(1) - f(d.mars_a))
        d.neg_lr, d.one_minus_decay_lr, d.eps = float(f(-0.0025)), float(f(1) - f(0.01) * f(0.0025)), float(f(1e-8))
        d.rng_mode, d.step, d.seed = _lib.RNG_PHILOX, step, 99
        return d


@pytest.mark.parametrize("case", sorted(CASES))
def test_noalloc_entry_matches_fused_step_on_two_calls(case):
    pf, gf, sf, algo, flags = CASES[case]
    dev = torch.device("cuda:0")
    L = _lib.lib()
    stream = torch.cuda.current_stream(dev).cuda_stream
    # ragged sizes: whole chunks, a partial last chunk, a partial last octet, a tensor shorter than one chunk
    numels = [3 * 4096, 4096 + 1000, 70001, 333, 2 * 4096 + 5, 12288]
    print(f"case {case}: first call on {len(numels)} tensors, second on 3 of them", flush=True)
    ref, new = (Roles(numels, pf, gf, sf, 5, dev) for _ in range(2))
    for step, active in ((1, tuple(range(len(numels)))), (2, (1, 3, 4))):
        d_ref = ref.desc(active, pf, gf, sf, algo, flags, step, with_counts=True)
        d_new = new.desc(active, pf, gf, sf, algo, flags, step, with_counts=False)
        _lib.check(L.hb_fused_step(ctypes.byref(d_ref), stream), "hb_fused_step")
        _lib.check(L.hb_fused_step_noalloc(ctypes.byref(d_new), stream), "hb_fused_step_noalloc")
        torch.cuda.synchronize()
        masked = ref.counts.cpu().view(-1, _lib.CAUTION_SLOTS).sum(1)
        assert all(int(masked[i]) > 0 for i in active), "the case must exercise the counters"
        for name, want in ref.buffers().items():
            got = new.buffers()[name]
            same = torch.equal(got.view(torch.uint8), want.view(torch.uint8))
            assert same, f"{case} call {step}: {name} differs from hb_fused_step"


def test_noalloc_entry_rejects_more_tensors_than_its_scratch_holds():
    pf, gf, sf, algo, flags = CASES["laprop_caution_fp32"]
    dev = torch.device("cuda:0")
    L = _lib.lib()
    r = Roles([4096], pf, gf, sf, 1, dev)
    d = r.desc((0,), pf, gf, sf, algo, flags, 1, with_counts=False)
    before = r.param.clone()
    d.n_tensors = _lib.NOALLOC_MAX_TENSORS + 1
    assert L.hb_fused_step_noalloc(ctypes.byref(d), torch.cuda.current_stream(dev).cuda_stream) == -1
    assert b"at most 8192" in L.hb_last_error()
    torch.cuda.synchronize()
    assert torch.equal(r.param, before)  # nothing was launched
