"""GPU parity of the Muon path through the C ABI: Nesterov-EMA momentum (bit-exact fp32) and the Newton-Schulz
orthogonalisation (<= 2e-2 relative Frobenius against the CPU oracle, the tolerance of bf16 products whose fp32
accumulation order differs between backends), plus the golden vectors recorded from the reference."""

import ctypes
import os

import pytest
import torch

from heavyball_amd import _lib
from oracle import muon
from oracle.rounding import HalfRounding, PhiloxRounding

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
DEV = "cuda:0"
NS_TOL = 2e-2


def rel_fro(a, b):
    return ((a.double().cpu() - b.double().cpu()).norm() / b.double().cpu().norm()).item()


def ns_coeff_array(coeffs):
    from heavyball_amd.muon import ns_coefficients

    return ns_coefficients(coeffs)


def run_ns5(G, legacy=False, rng_mode=_lib.RNG_HALF, seed=0, step=0, base=0, scale=None):
    L = _lib.lib()
    rows, cols = G.shape
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_workspace_bytes(rows, cols, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    g = G.to(DEV, torch.float32).contiguous()  # a bf16 input travels as fp32 values under HB_NS_BF16_UPDATE
    out = torch.empty_like(g)
    coeffs = muon.LEGACY_COEFFS if legacy else muon.NS_COEFFS
    arr = (ctypes.c_float * 15)(*ns_coeff_array(coeffs))
    if scale is None:
        scale = max(1, rows / cols) ** 0.5
    flags = int(legacy) | {torch.bfloat16: _lib.NS_BF16_UPDATE, torch.float16: _lib.NS_F16_UPDATE}.get(G.dtype, 0)
    _lib.check(L.hb_ns5(g.data_ptr(), out.data_ptr(), rows, cols, arr, flags, 1e-7, scale, rng_mode, seed, step, base, ws.data_ptr(),
                        nbytes.value, None))
    torch.cuda.synchronize()
    return out.cpu()


def run_ns5_batched(Gs, rng_mode=_lib.RNG_PHILOX, seed=5, step=3, bases=None):
    L = _lib.lib()
    n = len(Gs)
    rows = (ctypes.c_int64 * n)(*[g.shape[0] for g in Gs])
    cols = (ctypes.c_int64 * n)(*[g.shape[1] for g in Gs])
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows, cols, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    gs = [g.to(DEV).contiguous() for g in Gs]
    outs = [torch.empty_like(g) for g in gs]
    arr = (ctypes.c_float * 15)(*ns_coeff_array(muon.NS_COEFFS))
    gp = (ctypes.c_void_p * n)(*[g.data_ptr() for g in gs])
    op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    scale = (ctypes.c_float * n)(*[max(1, g.shape[0] / g.shape[1]) ** 0.5 for g in Gs])
    base = (ctypes.c_int64 * n)(*(bases or [0] * n))
    _lib.check(L.hb_ns5_batched(n, gp, op, rows, cols, arr, 0, 1e-7, scale, rng_mode, seed, step, base, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    return [o.cpu() for o in outs]


def test_ns5_batched_equals_one_by_one():
    """A grouped call gives, bit for bit, what one call per matrix gives: both tile classes in one batch, ragged shapes
    with padding, tall matrices, tiny ones, and a short, very wide one whose X X^T is computed in chunks of K."""
    # (200, 8500): split along K on the 128-wide tiles; (1024, 8448), (1100, 16400): split along K on the 256-wide tiles, the second
    # with ragged edges and chunks whose K-tile count is not a multiple of the ring depth
    shapes = [(2048, 2304), (1024, 1280), (300, 200), (130, 515), (2304, 2048), (64, 64), (1100, 1024), (200, 8500), (1024, 8448), (1100, 16400)]
    gen = torch.Generator().manual_seed(11)
    Gs = [torch.randn(s, generator=gen) * 1e-2 for s in shapes]
    bases = [4096 * 8 * k for k in range(len(shapes))]
    together = run_ns5_batched(Gs, bases=bases)
    for k, G in enumerate(Gs):
        print("case", tuple(G.shape), flush=True)
        alone = run_ns5(G, rng_mode=_lib.RNG_PHILOX, seed=5, step=3, base=bases[k])
        assert torch.equal(together[k].view(torch.int32), alone.view(torch.int32)), f"matrix {k} {tuple(G.shape)}"
        assert rel_fro(alone, muon.orthogonal(G.clone(), PhiloxRounding(5, step=3, base=[bases[k]]), 0)) < NS_TOL


def test_ns5_mixed_schedules_in_one_call_equal_one_call_per_matrix():
    """hb_ns5_batched_mixed: a coefficient table and a flag word per matrix.  Under the legacy mode the square matrices take
    the legacy table and its two input roundings, the others the default one (heavyball/utils.py:790-795); one grouped call
    over all of them gives, bit for bit, what a call per matrix gives, in both tile classes and with a K-split product."""
    shapes = [(1024, 1024), (1024, 1280), (300, 300), (130, 515), (2304, 2048), (64, 64), (200, 8500), (1280, 1280)]
    gen = torch.Generator().manual_seed(12)
    Gs = [torch.randn(s, generator=gen) * 1e-2 for s in shapes]
    legacy = [r == c for r, c in shapes]
    assert any(legacy) and not all(legacy)
    bases = [4096 * 8 * k for k in range(len(shapes))]
    L = _lib.lib()
    n = len(Gs)
    rows = (ctypes.c_int64 * n)(*[g.shape[0] for g in Gs])
    cols = (ctypes.c_int64 * n)(*[g.shape[1] for g in Gs])
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows, cols, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    gs = [g.to(DEV).contiguous() for g in Gs]
    outs = [torch.empty_like(g) for g in gs]
    tabs = {False: ns_coeff_array(muon.NS_COEFFS), True: ns_coeff_array(muon.LEGACY_COEFFS)}
    arr = (ctypes.c_float * (15 * n))(*[x for lg in legacy for x in tabs[lg]])
    flags = (ctypes.c_int32 * n)(*[int(lg) for lg in legacy])
    gp = (ctypes.c_void_p * n)(*[g.data_ptr() for g in gs])
    op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    scale = (ctypes.c_float * n)(*[max(1, g.shape[0] / g.shape[1]) ** 0.5 for g in Gs])
    base = (ctypes.c_int64 * n)(*bases)
    _lib.check(L.hb_ns5_batched_mixed(n, gp, op, rows, cols, arr, flags, 1e-7, scale, _lib.RNG_PHILOX, 5, 3, base, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    for k, G in enumerate(Gs):
        print("case", tuple(G.shape), "legacy" if legacy[k] else "default", flush=True)
        alone = run_ns5(G, legacy=legacy[k], rng_mode=_lib.RNG_PHILOX, seed=5, step=3, base=bases[k])
        assert torch.equal(outs[k].cpu().view(torch.int32), alone.view(torch.int32)), f"matrix {k} {tuple(G.shape)}"
    # HB_NS_BF16_UPDATE per matrix too (a bucket whose gradients have both dtypes): matrices 1, 2 and 6 are bf16 values
    for k in (1, 2, 6):
        flags[k] |= _lib.NS_BF16_UPDATE
        gs[k].copy_(gs[k].bfloat16().float())
    _lib.check(L.hb_ns5_batched_mixed(n, gp, op, rows, cols, arr, flags, 1e-7, scale, _lib.RNG_PHILOX, 5, 3, base, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    for k in (1, 2, 6, 0, 7):
        G = gs[k].cpu().bfloat16() if k in (1, 2, 6) else Gs[k]
        alone = run_ns5(G, legacy=legacy[k], rng_mode=_lib.RNG_PHILOX, seed=5, step=3, base=bases[k])
        assert torch.equal(outs[k].cpu().view(torch.int32), alone.view(torch.int32)), f"mixed update dtypes: matrix {k} {tuple(G.shape)}"
    # ... and HB_NS_F16_UPDATE: matrices 0 and 3 become float16 values beside the bf16 and fp32 ones
    for k in (0, 3):
        flags[k] |= _lib.NS_F16_UPDATE
        gs[k].copy_(gs[k].half().float())
    _lib.check(L.hb_ns5_batched_mixed(n, gp, op, rows, cols, arr, flags, 1e-7, scale, _lib.RNG_PHILOX, 5, 3, base, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    for k in (0, 3, 1, 7):
        G = gs[k].cpu().half() if k in (0, 3) else gs[k].cpu().bfloat16() if k == 1 else Gs[k]
        alone = run_ns5(G, legacy=legacy[k], rng_mode=_lib.RNG_PHILOX, seed=5, step=3, base=bases[k])
        assert torch.equal(outs[k].cpu().view(torch.int32), alone.view(torch.int32)), f"three update dtypes: matrix {k} {tuple(G.shape)}"
    call = lambda: L.hb_ns5_batched_mixed(n, gp, op, rows, cols, arr, flags, 1e-7, scale, _lib.RNG_PHILOX, 5, 3, base, ws.data_ptr(), nbytes.value, None)  # noqa: E731
    flags[7] |= 8  # an unknown flag bit is refused
    assert call() != 0
    flags[7] &= ~8
    assert call() == 0
    flags[0] |= _lib.NS_BF16_UPDATE  # so are both update formats at once
    assert call() != 0
    torch.cuda.synchronize()


def test_ns5_of_a_bucket_with_more_matrices_than_a_kernel_argument_holds():
    """Sixty matrices in one call (the descriptors of a launch live in a table in device memory, written by the call itself):
    bit for bit what a call per matrix gives, for the first, the last and a few in between."""
    gen = torch.Generator().manual_seed(13)
    shapes = [(96 + 8 * (k % 7), 64 + 32 * (k % 5)) for k in range(58)] + [(1024, 1100), (200, 8500)]
    Gs = [torch.randn(s, generator=gen) * 1e-2 for s in shapes]
    bases = [4096 * 8 * k for k in range(len(shapes))]
    together = run_ns5_batched(Gs, bases=bases)
    for k in (0, 1, 27, 28, 29, 56, 57, 58, 59):
        print("case", k, tuple(Gs[k].shape), flush=True)
        alone = run_ns5(Gs[k], rng_mode=_lib.RNG_PHILOX, seed=5, step=3, base=bases[k])
        assert torch.equal(together[k].view(torch.int32), alone.view(torch.int32)), f"matrix {k} {tuple(Gs[k].shape)}"


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_both_product_kernels_return_the_same_bits(mode):
    """The two product kernels (eight wavefronts on 128 x 128 tiles; four hand-scheduled wavefronts on 256 x 256 tiles whose
    fragment reads go through inline assembly with manual waits) add into an accumulator in the same order, so the same
    product must come out bit for bit the same from both: a register read ahead of its wait, which the compiler cannot
    diagnose, would show here.  To be re-run whenever the compiler or a tuning macro of the kernels changes.
    Mode 1 mirrors the tiles above the diagonal, whose size differs between the kernels: compared where both computed directly."""
    L = _lib.lib()
    M, N, K = ((1024, 1024, 2304), (1024, 1024, 1024), (1024, 2304, 1024))[mode]
    gen = torch.Generator().manual_seed(40 + mode)
    A = (torch.randn(M, K, generator=gen) * 0.05).bfloat16().to(DEV)
    B = A if mode == 0 else (torch.randn(N, K, generator=gen) * 0.05).bfloat16().to(DEV)
    ws = torch.empty(4096, dtype=torch.uint8, device=DEV)
    out = {}
    for tile in (128, 256):
        print("case mode", mode, "tile", tile, flush=True)
        C = torch.full((M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        C2 = torch.full((N, M) if mode == 2 else (M, N), 7.0, dtype=torch.bfloat16, device=DEV)
        _lib.check(L.hb_ns_product(tile, mode, A.data_ptr(), B.data_ptr(), C.data_ptr(), C2.data_ptr(), M, N, K, 2.5, -3.25, ws.data_ptr(), 4096, None))
        torch.cuda.synchronize()
        out[tile] = (C.cpu().view(torch.int16), C2.cpu().view(torch.int16))
    want = (A.float() @ B.float().T).cpu()
    got = out[128][0].view(torch.bfloat16).float()
    direct = (torch.arange(M)[:, None] // 128) <= (torch.arange(N)[None, :] // 128)
    if mode == 1:
        want = want + torch.eye(M) * -3.25
        assert torch.equal(out[128][0][direct], out[256][0][direct])
        assert ((got - want).abs()[direct] <= 2.0**-7 * want.abs()[direct] + 1e-3).all()
        return
    assert torch.equal(out[128][0], out[256][0]) and torch.equal(out[128][1], out[256][1])
    assert ((got - want).abs() <= 2.0**-7 * want.abs() + 1e-3).all()
    if mode == 2:
        assert torch.equal(out[128][1], out[128][0].T)
    else:
        assert torch.equal(out[128][0], out[128][0].T)  # S mirrors exactly


def test_ns5_mirrored_symmetric_products():
    """Only the upper triangle of tiles of X X^T and of Y S is computed and mirrored; the output has to be what the full
    products give within the Newton-Schulz tolerance on matrices with off-diagonal tiles in both tile classes."""
    gen = torch.Generator().manual_seed(12)
    for shape in [(640, 384), (2048, 2560)]:
        G = torch.randn(shape, generator=gen) * 1e-2
        got = run_ns5(G)
        want = muon.orthogonal(G.clone(), HalfRounding(), 0)
        assert rel_fro(got, want) < NS_TOL, shape
        # singular values of the result sit in the band the per-iteration schedule drives them to
        sv = torch.linalg.svdvals(got.double() / max(1, shape[0] / shape[1]) ** 0.5)
        assert sv.max() < 1.35 and sv.min() > 0.3, (shape, sv.min().item(), sv.max().item())


@pytest.mark.parametrize("name", ["sq", "wide", "tall", "sq64"])
def test_ns5_matches_reference_vectors(name):
    d = torch.load(os.path.join(GOLDEN, "ns5.pt"), weights_only=True)
    print("case", name, flush=True)
    G = d[f"{name}/G"]
    assert rel_fro(run_ns5(G, scale=1.0), d[f"{name}/ns5"]) < NS_TOL
    assert rel_fro(run_ns5(G), d[f"{name}/orthogonal_scaled"]) < NS_TOL
    if f"{name}/legacy" in d:
        assert rel_fro(run_ns5(G, legacy=True, scale=1.0), d[f"{name}/legacy"]) < NS_TOL


@pytest.mark.parametrize("name", ["sq", "wide", "tall", "sq64"])
def test_ns5_on_bf16_inputs_matches_reference_vectors(name):
    """HB_NS_BF16_UPDATE, alone and with the legacy schedule, against vectors the reference computed on bf16 tensors."""
    d = torch.load(os.path.join(GOLDEN, "ns5_bf16.pt"), weights_only=True)
    print("case", name, flush=True)
    G = d[f"{name}/G"]
    got = run_ns5(G, scale=1.0)
    assert torch.equal(got, got.bfloat16().float()) and rel_fro(got, d[f"{name}/ns5"].float()) < NS_TOL
    if f"{name}/legacy" in d:
        got = run_ns5(G, legacy=True, scale=1.0)
        assert torch.equal(got, got.bfloat16().float()) and rel_fro(got, d[f"{name}/legacy"].float()) < NS_TOL


@pytest.mark.parametrize("name", ["sq", "wide", "tall", "sq64"])
def test_ns5_on_fp16_inputs_matches_reference_vectors(name):
    """HB_NS_F16_UPDATE, alone and with the legacy schedule, against vectors the reference computed on float16 tensors."""
    d = torch.load(os.path.join(GOLDEN, "ns5_fp16.pt"), weights_only=True)
    print("case", name, flush=True)
    G = d[f"{name}/G"]
    got = run_ns5(G, scale=1.0)
    assert torch.equal(got, got.half().float()) and rel_fro(got, d[f"{name}/ns5"].float()) < NS_TOL
    got = run_ns5(G)
    assert torch.equal(got, got.half().float()) and rel_fro(got, d[f"{name}/orthogonal_scaled"].float()) < NS_TOL
    if f"{name}/legacy" in d:
        got = run_ns5(G, legacy=True, scale=1.0)
        assert torch.equal(got, got.half().float()) and rel_fro(got, d[f"{name}/legacy"].float()) < NS_TOL


def run_ns_steps(Gs, coeffs, rng_mode=_lib.RNG_HALF, seed=0, step=0, bases=None):
    """hb_ns_batched_steps on the matrices ``Gs`` (fp32, bf16 or fp16 tensors) under one schedule of len(coeffs) iterations."""
    L = _lib.lib()
    n, n_steps = len(Gs), len(coeffs)
    rows = (ctypes.c_int64 * n)(*[g.shape[0] for g in Gs])
    cols = (ctypes.c_int64 * n)(*[g.shape[1] for g in Gs])
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows, cols, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    gs = [g.to(DEV, torch.float32).contiguous() for g in Gs]
    outs = [torch.empty_like(g) for g in gs]
    arr = (ctypes.c_float * (3 * n_steps * n))(*(ns_coeff_array(coeffs) * n))
    flags = (ctypes.c_int32 * n)(*[{torch.bfloat16: _lib.NS_BF16_UPDATE, torch.float16: _lib.NS_F16_UPDATE}.get(g.dtype, 0) for g in Gs])
    gp = (ctypes.c_void_p * n)(*[g.data_ptr() for g in gs])
    op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    scale = (ctypes.c_float * n)(*[1.0] * n)
    base = (ctypes.c_int64 * n)(*(bases or [0] * n))
    _lib.check(L.hb_ns_batched_steps(n, gp, op, rows, cols, n_steps, arr, flags, 1e-7, scale, None, None, None, rng_mode, seed, step, base, ws.data_ptr(),
                                     nbytes.value, None),
               "hb_ns_batched_steps")  # fmt: skip
    torch.cuda.synchronize()
    return [o.cpu() for o in outs]


@pytest.mark.parametrize("cautious", [False, True])
def test_apply_to_param_equals_the_product_followed_by_the_update(cautious):
    """HB_NS_APPLY_TO_PARAM through the C ABI, on both product kernels (tall, wide and ragged matrices of the 128- and the 256-wide
    class, fp32 and float16 update buffers): the parameter ends where the plain call's update, put through
    p * (1 - decay lr) + u * (-lr) in fp32 (decay factor 1 where signs differ under HB_NS_CAUTIOUS_WD), puts it, bit for bit;
    the update buffer handed in is left alone."""
    L = _lib.lib()
    gen = torch.Generator().manual_seed(29)
    shapes = [(320, 192), (130, 515), (1100, 1024), (1024, 1280)]
    Gs = [torch.randn(s, generator=gen) * 1e-2 for s in shapes]
    Gs[1] = Gs[1].half().float()
    Ps = [torch.randn(s, generator=gen) * 0.05 for s in shapes]
    n = len(Gs)
    rows = (ctypes.c_int64 * n)(*[g.shape[0] for g in Gs])
    cols = (ctypes.c_int64 * n)(*[g.shape[1] for g in Gs])
    assert [L.hb_ns_tile(*s) for s in shapes] == [128, 128, 256, 256]
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows, cols, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    gs = [g.to(DEV).contiguous() for g in Gs]
    us = [torch.empty_like(g) for g in gs]
    ps = [p.to(DEV).contiguous() for p in Ps]
    arr = (ctypes.c_float * (15 * n))(*(ns_coeff_array(muon.NS_COEFFS) * n))
    base_flags = [0, _lib.NS_F16_UPDATE, 0, 0]
    scale = (ctypes.c_float * n)(*[max(1, g.shape[0] / g.shape[1]) ** 0.5 for g in Gs])
    base = (ctypes.c_int64 * n)(*[4096 * 300 * k for k in range(n)])
    gp = (ctypes.c_void_p * n)(*[g.data_ptr() for g in gs])
    om, neg_lr = 1 - 0.1 * 0.02, -0.02
    step = (ctypes.c_float * 2)(om, neg_lr)

    def call(outs, extra):
        flags = (ctypes.c_int32 * n)(*[f | extra for f in base_flags])
        op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
        _lib.check(L.hb_ns_batched_steps(n, gp, op, rows, cols, 5, arr, flags, 1e-7, scale, step, None, None, _lib.RNG_PHILOX, 5, 3, base,
                                         ws.data_ptr(), nbytes.value, None), "hb_ns_batched_steps")  # fmt: skip
        torch.cuda.synchronize()

    print("case", cautious, flush=True)
    call(us, 0)
    call(ps, _lib.NS_APPLY_TO_PARAM | (_lib.NS_CAUTIOUS_WD if cautious else 0))
    for k in range(n):
        p0, u = Ps[k].to(DEV), us[k]
        factor = torch.full_like(p0, om)
        if cautious:
            factor = torch.where((p0.view(torch.int32) ^ u.view(torch.int32)) < 0, torch.ones_like(p0), factor)
        want = p0 * factor + u * torch.tensor(neg_lr, dtype=torch.float32, device=DEV)
        assert torch.equal(ps[k].view(torch.int32), want.view(torch.int32)), shapes[k]
        assert torch.equal(gs[k].cpu(), Gs[k])


def test_polar_express_matches_reference_vectors_and_oracle():
    """hb_ns_batched_steps under msign's ten-step schedule: against the vectors the reference computed (fp32, bf16 and float16
    inputs, one call for all five), against the oracle on larger matrices of both tile classes, and with five steps of the default
    schedule bit for bit what hb_ns5_batched gives."""
    d = torch.load(os.path.join(GOLDEN, "msign.pt"), weights_only=True)
    names = ["sq", "sq64", "sq96", "sq64_bf16", "sq64_fp16"]
    outs = run_ns_steps([d[f"{k}/G"] for k in names], muon.POLAR_COEFFS)
    for k, got in zip(names, outs):
        print("case", k, flush=True)
        assert rel_fro(got, d[f"{k}/msign"].float()) < NS_TOL
    gen = torch.Generator().manual_seed(23)
    Gs = [torch.randn(s, generator=gen) * 1e-2 for s in [(320, 320), (1100, 1100), (130, 515)]]
    bases = [0, 4096 * 40, 4096 * 400]
    outs = run_ns_steps(Gs, muon.POLAR_COEFFS, rng_mode=_lib.RNG_PHILOX, seed=5, step=3, bases=bases)
    for k, (G, got) in enumerate(zip(Gs, outs)):
        print("case", tuple(G.shape), flush=True)
        r = PhiloxRounding(5, step=3, base=[bases[k]])
        want = muon.polar_express(G.clone(), r.noise16(6, 0, G.shape))
        assert rel_fro(got, want) < NS_TOL
        sv = torch.linalg.svdvals(got.double())
        assert sv.max() < 1.2 and sv.median() > 0.9  # ten steps bring the bulk of the spectrum to 1
    five = run_ns_steps(Gs, muon.NS_COEFFS, rng_mode=_lib.RNG_PHILOX, seed=5, step=3, bases=bases)
    for G, got, b in zip(Gs, five, bases):
        alone = run_ns5(G, rng_mode=_lib.RNG_PHILOX, seed=5, step=3, base=b, scale=1.0)
        assert torch.equal(got.view(torch.int32), alone.view(torch.int32))


@pytest.mark.parametrize("legacy", [False, True])
def test_ns5_fp16_input_and_output_roundings_are_the_oracles(legacy):
    """The float16 route through an identity schedule (a = 1, b = c = 0 makes an iteration return X): what comes back is the
    normalised input after its roundings (float16 norm and quotient, one stochastic round to bf16; the legacy schedule rounds the
    input first and divides in fp32) and the two roundings of the way out (the cast to float16, which flushes what bf16 still
    resolves below 2^-24, and the scaling there).  Tiny entries make the cast lossy, the scale is not a power of two."""
    from oracle import philox
    from oracle.ecc import stochastic_round
    gen = torch.Generator().manual_seed(3)
    G = torch.randn(96, 160, generator=gen) * 1e-2
    G[::3] *= 1e-5  # quotients below float16's normal range
    G = G.half()
    L = _lib.lib()
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_workspace_bytes(96, 160, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    g = G.to(DEV, torch.float32).contiguous()
    out = torch.empty_like(g)
    arr = (ctypes.c_float * 15)(*([1.0, 0.0, 0.0] * 5))
    flags = int(legacy) | _lib.NS_F16_UPDATE
    scale = 1.2345
    print("case", legacy, flush=True)
    _lib.check(L.hb_ns5(g.data_ptr(), out.data_ptr(), 96, 160, arr, flags, 1e-7, scale, _lib.RNG_PHILOX, 9, 4, 640, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    nrm = G.norm()  # a float16 value
    r = PhiloxRounding(9, step=4, base=[640])
    if legacy:
        x = stochastic_round(G.clone(), r.noise16(philox.STREAM_NS_INPUT, 0, G.shape))
        x = stochastic_round(x.float() / nrm.float().clamp(min=1e-7), r.noise16(philox.STREAM_NS_INPUT + 1, 0, G.shape))
    else:
        x = stochastic_round(G / nrm.clamp(min=1e-7), r.noise16(philox.STREAM_NS_INPUT, 0, G.shape))
    want = x.to(torch.float16)
    want *= scale
    got = out.cpu()
    assert torch.equal(got, got.half().float())
    want = want.float()
    assert (got != want).float().mean() < 2e-3  # the norm's summation order may move its float16 rounding once in a while: then all differ
    assert rel_fro(got, want) < 1e-2


@pytest.mark.parametrize("legacy", [False, True])
def test_ns5_bf16_input_rounding_is_the_oracles(legacy):
    """The normalised bf16 input the kernel feeds its first product, read back through a one-iteration identity schedule
    (a = 1, b = c = 0 makes an iteration return X): the default schedule rounds the bf16 quotient to nearest, the legacy one
    rounds the fp32 quotient stochastically with stream NS_INPUT + 1."""
    from oracle import philox
    from oracle.ecc import stochastic_round
    gen = torch.Generator().manual_seed(3)
    G = (torch.randn(96, 96, generator=gen) * 1e-2).bfloat16()
    L = _lib.lib()
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_workspace_bytes(96, 96, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    g = G.to(DEV, torch.float32).contiguous()
    out = torch.empty_like(g)
    arr = (ctypes.c_float * 15)(*([1.0, 0.0, 0.0] * 5))
    flags = int(legacy) | _lib.NS_BF16_UPDATE
    print("case", legacy, flush=True)
    _lib.check(L.hb_ns5(g.data_ptr(), out.data_ptr(), 96, 96, arr, flags, 1e-7, 1.0, _lib.RNG_PHILOX, 9, 4, 640, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    nrm = G.norm()  # a bf16 value
    if legacy:
        r = PhiloxRounding(9, step=4, base=[640])
        want = stochastic_round(G.float() / nrm.float().clamp(min=1e-7), r.noise16(philox.STREAM_NS_INPUT + 1, 0, G.shape)).float()
    else:
        want = (G / nrm.clamp(min=1e-7)).float()
    got = out.cpu()
    assert (got != want).float().mean() < 2e-3  # the norm's summation order may move its bf16 rounding once in a while: then all differ
    assert rel_fro(got, want) < 1e-2


@pytest.mark.parametrize("shape", [(256, 256), (128, 384), (384, 128), (300, 200), (130, 515), (512, 2048), (2304, 768), (256, 9000), (9000, 200), (768, 50257),
                                   (1024, 8448), (16400, 1100)])
@pytest.mark.parametrize("rounding", ["half", "philox"])
def test_ns5_matches_oracle(shape, rounding):
    print("case", shape, rounding, flush=True)
    gen = torch.Generator().manual_seed(shape[0] * 7 + shape[1])
    G = torch.randn(shape, generator=gen) * 1e-2
    if rounding == "half":
        r, mode = HalfRounding(), _lib.RNG_HALF
    else:
        r, mode = PhiloxRounding(31, step=4, base=[40]), _lib.RNG_PHILOX
    want = muon.orthogonal(G.clone(), r, 0)
    got = run_ns5(G, rng_mode=mode, seed=31, step=4, base=40)
    err = rel_fro(got, want)
    print("rel fro", err, flush=True)
    assert err < NS_TOL
    # invariant independent of any oracle: singular values of the orthogonalised update sit near its post-scale
    sv = torch.linalg.svdvals(got.double())
    scale = max(1, shape[0] / shape[1]) ** 0.5
    assert sv.max() < 1.35 * scale


def test_ns5_input_rounding_is_the_oracles():
    """With one Newton-Schulz coefficient set to make the iteration the identity (a=1, b=c=0) the output is the
    stochastically rounded, normalised input itself: bit-exact against the oracle's rounding with the shared stream."""
    L = _lib.lib()
    gen = torch.Generator().manual_seed(5)
    G = torch.randn(128, 256, generator=gen)
    rows, cols = G.shape
    nbytes = ctypes.c_int64()
    _lib.check(L.hb_ns5_workspace_bytes(rows, cols, ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=DEV)
    g = G.to(DEV)
    out = torch.empty_like(g)
    arr = (ctypes.c_float * 15)(*([1.0, 0.0, 0.0] * 5))
    _lib.check(L.hb_ns5(g.data_ptr(), out.data_ptr(), rows, cols, arr, 0, 1e-7, 1.0, _lib.RNG_PHILOX, 9, 2, 16, ws.data_ptr(), nbytes.value, None))
    torch.cuda.synchronize()
    from oracle.ecc import stochastic_round

    Gn = G / G.norm().clamp(min=1e-7)
    want = stochastic_round(Gn, PhiloxRounding(9, step=2, base=[16]).noise16(6, 0, G.shape)).float()
    got = out.cpu()
    # the norm is a reduction (order differs from torch's), so allow the rare element whose quotient moved by an ulp
    # across a rounding boundary; everything else must be identical
    assert (got != want).float().mean() < 1e-3
    assert rel_fro(got, want) < 1e-3


# ---------------------------------------------------------------------------------------------------------------
# the Muon optimizer class end to end
# ---------------------------------------------------------------------------------------------------------------
def _muon_pair(shapes, kwargs, rounding="half", seed=21, mode="newtonschulz"):
    import heavyball_amd
    from tests import helpers as H

    host, params = H.make_params(shapes, DEV)
    opt = heavyball_amd.Muon(params, **kwargs)
    opt.rounding, opt.rng_seed = rounding, seed
    base = opt._buckets[0][0].slab.offsets_np.tolist()
    r = HalfRounding() if rounding == "half" else PhiloxRounding(seed, base=base)
    orc = muon.MuonOracle([h.clone() for h in host], rounding=r, mode=mode, **kwargs)
    return host, params, opt, orc


MUON_VARIANTS = [
    ("default", dict(betas=(0.95, 0.99), weight_decay=0.01, lr=0.02), torch.float32),
    ("ecc_momentum", dict(ecc="bf16+8", lr=0.02), torch.float32),
    ("bf16_grads_bf16_momentum", dict(storage_dtype="bfloat16", lr=0.02), torch.bfloat16),
    ("heavyball_ecc16_bf16_grads", dict(ecc="bf16+16", nesterov=False, heavyball_momentum=True, lr=0.02), torch.bfloat16),
    ("plain_ema_caution", dict(nesterov=False, caution=True, weight_decay=0.1, lr=0.02), torch.float32),
    # gradients of both dtypes in one bucket (dealt out in turn): the update buffer, and with it Newton-Schulz' normalisation, is per tensor
    ("mixed_grads", dict(lr=0.02, weight_decay=0.01), (torch.bfloat16, torch.float32)),
    ("mixed_grads_mars_ecc_caution", dict(lr=0.02, mars=True, ecc="bf16+8", caution=True), (torch.float32, torch.bfloat16)),
    # float16 gradients: the update buffer is float16, Newton-Schulz normalises there and hands a float16 update back
    ("fp16_grads", dict(lr=0.02, weight_decay=0.01), torch.float16),
    ("fp16_grads_mars_caution_bf16_momentum", dict(lr=0.02, mars=True, caution=True, storage_dtype="bfloat16"), torch.float16),
    ("three_grad_dtypes_ecc", dict(lr=0.02, ecc="bf16+16", weight_decay=0.01), (torch.float16, torch.bfloat16, torch.float32)),
]


@pytest.mark.parametrize("rounding", ["half", "philox"])
@pytest.mark.parametrize("variant", MUON_VARIANTS, ids=[v[0] for v in MUON_VARIANTS])
def test_muon_optimizer_matches_oracle(variant, rounding):
    """The momentum (any of its four forms; fp32, bf16 or an ECC pair) is elementwise: bit-exact, stochastic rounding
    included.  Vectors take the momentum direction unchanged: bit-exact.  Matrices go through Newton-Schulz: the step
    taken agrees to the NS tolerance."""
    from tests import helpers as H

    shapes = [(192, 320), (64,), (320, 128), (8, 6, 24), (130, 70)]
    _, kwargs, gdt = variant
    print("case", variant[0], rounding, flush=True)
    host, params, opt, orc = _muon_pair(shapes, kwargs, rounding)
    for p in params:
        p.grad_dtype = None
    for k in range(1, 4):
        gdts = [gdt[i % len(gdt)] for i in range(len(shapes))] if isinstance(gdt, tuple) else [gdt] * len(shapes)
        grads = [g.to(t) for g, t in zip(H.make_grads(shapes, k, torch.float32, 1e-2), gdts)]
        prev = [p.detach().cpu().clone() for p in params]
        prev_o = [p.clone() for p in orc.params]
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        orc.step([g.clone() for g in grads])
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            H.assert_bit_equal(opt.state[p][0][opt.KEY], orc.state[i][orc.KEY], f"step {k} momentum {i}")
            if kwargs.get("ecc"):
                H.assert_bit_equal(opt.state[p][0][opt.KEY + "::ecc"], orc.state[i][orc.KEY + "::ecc"], f"step {k} momentum correction {i}")
            if p.dim() < 2:
                H.assert_bit_equal(p.data, orc.params[i], f"step {k} vector {i}")
            else:
                got, want = p.detach().cpu() - prev[i], orc.params[i] - prev_o[i]
                # decay moves both sides identically up to the parameter drift; compare the steps
                assert rel_fro(got, want) < NS_TOL, (k, i, rel_fro(got, want))
        assert opt.param_groups[0]["step"] is None


@pytest.mark.parametrize("kwargs,gdt", [(dict(lr=0.02, weight_decay=0.1), torch.float32),
                                        (dict(lr=0.02, weight_decay=0.1, cautious_weight_decay=True, mars=True), torch.bfloat16),
                                        (dict(lr=0.02, ecc="bf16+8", nesterov=False), torch.float16)])
def test_step_inside_the_last_product_equals_the_separate_update(kwargs, gdt):
    """Where the chain allows it the last Newton-Schulz product applies p <- p (1 - decay lr) - lr u itself
    (HB_NS_APPLY_TO_PARAM) instead of writing u for hb_update_param to read back: the same arithmetic on the same values, so
    the parameters agree bit for bit with the two-launch route, over wide, tall, ragged and stacked matrices of both tile
    classes, with vectors (which keep the separate update) in the same bucket."""
    import heavyball_amd
    from tests import helpers as H

    shapes = [(192, 320), (64,), (320, 128), (8, 6, 24), (130, 70), (1100, 1024), (1, 5), (7,)]
    print("case", kwargs, gdt, flush=True)
    host, pa = H.make_params(shapes, DEV)
    _, pb = H.make_params(shapes, DEV)
    oa, ob = heavyball_amd.Muon(pa, **kwargs), heavyball_amd.Muon(pb, **kwargs)
    ob.fuse_update_into_newton_schulz = False
    for o in (oa, ob):
        o.rounding, o.rng_seed = "philox", 77
    for p in pa + pb:
        p.grad_dtype = None
    for k in range(1, 4):
        grads = H.make_grads(shapes, k, gdt, 1e-2)
        for p, q, g in zip(pa, pb, grads):
            p.grad, q.grad = g.to(DEV), g.to(DEV).clone()
        oa.step()
        ob.step()
        torch.cuda.synchronize()
        for i, (p, q) in enumerate(zip(pa, pb)):
            assert torch.equal(p.detach().view(torch.int32), q.detach().view(torch.int32)), (k, i, shapes[i])
    assert all(not torch.equal(p.detach().cpu(), h) for p, h in zip(pa, host))  # and they did move


def test_momentum_leaves_the_sums_of_squares_of_its_update():
    """hb_momentum_sumsq: the doubles it writes per chunk add up, tensor by tensor, to the sum of squares of the update it wrote
    (ragged sizes: a chunk's tail past the tensor's end contributes zeros), for fp32 and for bf16 gradients, whose update is
    rounded before it is squared.  Read off a Muon step whose last product applies the parameter step itself, so the update
    buffer still holds what the momentum kernel wrote."""
    import heavyball_amd
    from tests import helpers as H

    shapes = [(192, 320), (4097,), (130, 70), (1, 5), (8, 6, 24), (700, 900)]  # matrices of the 128-wide kernel: the step is fused
    L = _lib.lib()
    per_chunk, chunk = L.hb_momentum_sumsq_parts_per_chunk(), _lib.chunk_elems()
    for gdt in (torch.float32, torch.bfloat16):
        print("case", gdt, flush=True)
        _, params = H.make_params(shapes, DEV)
        opt = heavyball_amd.Muon(params, lr=0.02)
        for p, g in zip(params, H.make_grads(shapes, 1, gdt, 1e-2)):
            p.grad = g.to(DEV)
        opt.step()
        torch.cuda.synchronize()
        (b,) = opt._buckets[0]
        parts = opt._scratch64_pool[("sumsq", id(b), gdt)].cpu()
        first = 0
        for i, n in enumerate(b.slab.numels):
            count = -(-n // chunk)
            got = parts[first * per_chunk : (first + count) * per_chunk]
            first += count
            u = b.slab.view("_update", i).double().cpu()
            assert u.abs().max() > 0
            if gdt == torch.bfloat16:
                assert torch.equal(u, u.bfloat16().double())
            want = (u * u).sum()
            assert abs(got.sum() - want) <= 1e-12 * want, (i, float(got.sum()), float(want))
            assert (got >= 0).all()


def _random_muon_case(seed):
    import random

    rnd = random.Random(1000 + seed)
    kwargs = dict(lr=0.02, nesterov=rnd.random() < 0.6, heavyball_momentum=rnd.random() < 0.3, mars=rnd.random() < 0.4,
                  caution=rnd.random() < 0.4, betas=(rnd.choice([0.9, 0.95]), 0.99))  # fmt: skip
    if rnd.random() < 0.5:
        kwargs["weight_decay"] = rnd.choice([0.01, 0.1])
        kwargs["cautious_weight_decay"] = rnd.random() < 0.3
    storage = rnd.choice(["f32", "f32", "bf16", "bf16+8", "bf16+16", "fp16+8", "fp16+16"])
    if "+" in storage:
        kwargs["ecc"] = storage
    elif storage == "bf16":
        kwargs["storage_dtype"] = "bfloat16"
    if rnd.random() < 0.3:
        kwargs["param_ecc"] = rnd.choice(["bf16+8", "bf16+16"])
    gdt = rnd.choice([torch.float32, torch.float32, torch.bfloat16, torch.float16])
    dims = [1, 2, 7, 8, 33, 64, 127, 128, 129, 200, 256, 300]
    shapes = [(rnd.choice(dims), rnd.choice(dims)) for _ in range(rnd.randint(2, 4))] + [(rnd.choice([1, 9, 64, 4097]),)]
    if rnd.random() < 0.4:
        shapes.append((rnd.randint(2, 6), rnd.randint(2, 6), rnd.choice([8, 24, 31])))
    rnd.shuffle(shapes)
    rounding = rnd.choice(["half", "philox"])
    mode = "newtonschulz"
    if rnd.random() < 0.35:  # the legacy schedule or msign's, which square matrices take (heavyball/utils.py:790-797)
        mode = rnd.choice(["legacy_newtonschulz", "legacy_newtonschulz", "thinky_polar_express"])
        shapes += [(rnd.choice([8, 64, 130, 256]),) * 2, (3, 6, 18)]
    return kwargs, gdt, shapes, rounding, mode


@pytest.mark.parametrize("seed", range(300))
def test_random_muon_configurations_match_oracle(seed):
    """Seeded draws over Muon's momentum forms, MARS, caution, decay, storage of the momentum and of the parameter, gradient
    dtype, the Newton-Schulz schedule and shapes (vectors, thin and tiny matrices, stacks): momentum, MARS' old gradient and their corrections bit for
    bit, vectors bit for bit, matrices to the Newton-Schulz tolerance on the step taken."""
    from oracle.ecc import EccTensor
    from tests import helpers as H

    import heavyball_amd

    kwargs, gdt, shapes, rounding, mode = _random_muon_case(seed)
    print("case", seed, kwargs, gdt, shapes, rounding, mode, flush=True)
    host, params, opt, orc = _muon_pair(shapes, kwargs, rounding, mode=mode)
    if kwargs.get("param_ecc"):
        for b in opt._buckets[0]:
            for i, p in enumerate(b.params):
                j = [id(q) for q in params].index(id(p))
                opt._encode_param(b, i, host[j].to(DEV).contiguous(), opt.param_groups[0])

    def value(t, corr):
        t = t.detach().cpu()
        return EccTensor(t, corr.detach().cpu()).decode() if corr is not None else t.float()

    for k in range(1, 4):
        grads = H.make_grads(shapes, k, gdt, 1e-2)
        prev = [value(p.data, opt.state[p][0].get("param::ecc") if p in opt.state and 0 in opt.state[p] else None) for p in params]
        prev_o = [q.decode() if isinstance(q, EccTensor) else q.clone() for q in orc.params]
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        heavyball_amd.muon.zeroth_power_mode = mode
        try:
            opt.step()
        finally:
            heavyball_amd.muon.zeroth_power_mode = "newtonschulz"
        orc.step([g.clone() for g in grads])
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            st = opt.state[p][0]
            for key, val in orc.state[i].items():
                if isinstance(val, torch.Tensor) and key not in ("step", "param::ecc"):
                    H.assert_bit_equal(st[key], val, f"step {k} tensor {i} {key}")
            q = orc.params[i]
            if p.dim() < 2:
                H.assert_bit_equal(p.data, q.primary if isinstance(q, EccTensor) else q, f"step {k} vector {i}")
                if isinstance(q, EccTensor):
                    H.assert_bit_equal(st["param::ecc"], q.corr, f"step {k} vector {i} correction")
            else:
                got = value(p.data, st.get("param::ecc")) - prev[i]
                want = (q.decode() if isinstance(q, EccTensor) else q) - prev_o[i]
                # a parameter kept as an ECC pair moves in units of 2^-8/127 of a bf16 ulp: allow that resolution on top
                slack = 4 * (2.0**-8 / 127) * prev[i].abs().max().item() * prev[i].numel() ** 0.5 if kwargs.get("param_ecc") else 0.0
                assert (got - want).norm().item() <= NS_TOL * want.norm().item() + slack, (k, i, rel_fro(got, want))


def _matrix_step_close(d, k, i, p, st):
    """The step a matrix took against the fixture's, to the Newton-Schulz tolerance; ECC parameters are decoded first (the fixture
    holds no correction for the narrowed initial parameter, so their first step has no reference point)."""
    from oracle.ecc import EccTensor

    def full(t, key):
        return EccTensor(t, d[key]).decode() if key in d else t.float()

    if f"step{k}/state{i}/param::ecc" in d:
        if k == 1:
            return
        got = EccTensor(p.detach().cpu(), st["param::ecc"].cpu()).decode()
    else:
        got = p.detach().cpu()
    prev = full(d[f"step{k - 1}/p{i}"], f"step{k - 1}/state{i}/param::ecc") if k > 1 else d[f"init/p{i}"]
    want = full(d[f"step{k}/p{i}"], f"step{k}/state{i}/param::ecc")
    assert rel_fro(got - prev, want - prev) < NS_TOL, (k, i, rel_fro(got - prev, want - prev))


def test_muon_matches_reference_trajectories():
    import glob
    import json

    import heavyball_amd

    for path in sorted(glob.glob(os.path.join(GOLDEN, "traj_muon_*.pt"))):
        d = torch.load(path, weights_only=True)
        print("case", os.path.basename(path), flush=True)
        kwargs = json.loads(d["meta/kwargs"])
        if "betas" in kwargs:
            kwargs["betas"] = tuple(kwargs["betas"])
        n = len([k for k in d if k.startswith("init/p")])
        params = [torch.nn.Parameter(d[f"init/p{i}"].clone().to(DEV)) for i in range(n)]
        for p in params:
            p.grad_dtype = None  # bf16 gradients on fp32 parameters
        heavyball_amd.HBOptimizer.rounding = "half"  # param_ecc encodes the parameters at construction
        try:
            opt = heavyball_amd.Muon(params, **kwargs)
        finally:
            heavyball_amd.HBOptimizer.rounding = "philox"
        opt.rounding = "half"
        for k in range(1, d["meta/steps"] + 1):
            for i, p in enumerate(params):
                p.grad = d[f"step{k}/g{i}"].clone().to(DEV)
            heavyball_amd.muon.zeroth_power_mode = d.get("meta/zeroth_power_mode", "newtonschulz")
            try:
                opt.step()
            finally:
                heavyball_amd.muon.zeroth_power_mode = "newtonschulz"
            torch.cuda.synchronize()
            for i, p in enumerate(params):
                mom = d[f"step{k}/state{i}/{opt.KEY}"]
                got_mom = opt.state[p][0][opt.KEY].cpu()
                prefix = f"step{k}/state{i}/"
                want_state = {kk[len(prefix):]: d[kk] for kk in d if kk.startswith(prefix) and not kk.endswith("/step")}
                assert set(want_state) == {kk for kk in opt.state[p][0] if kk not in ("step", "is_initialized")}
                want, prev = d[f"step{k}/p{i}"], (d[f"step{k - 1}/p{i}"] if k > 1 else d[f"init/p{i}"])
                for kk, vv in want_state.items():  # ECC corrections and MARS' old gradient have to match too
                    if kk != opt.KEY and not (kk == "param::ecc" and want.dim() >= 2):
                        assert torch.equal(opt.state[p][0][kk].cpu(), vv), (k, i, kk)
                if "clip" in path:  # the clip norm is summed in another order: 2e-6 of the tensor's scale instead of equality
                    assert ((got_mom - mom).abs() <= 2e-6 * (mom.abs() + mom.abs().max())).all()
                    if want.dim() < 2:
                        assert torch.allclose(p.detach().cpu(), want, rtol=2e-6, atol=1e-9)
                        continue
                else:
                    assert torch.equal(got_mom, mom)
                if want.dim() < 2:
                    assert torch.equal(p.detach().cpu(), want)
                else:
                    _matrix_step_close(d, k, i, p, opt.state[p][0])
        sd = opt.state_dict()
        assert set(sd["state"][0][0].keys()) >= {opt.KEY, "is_initialized", "step"}
        want_init = set(d["final/is_initialized0"].tolist()) if "final/is_initialized0" in d else {0, 1, 2}
        assert sd["state"][0][0]["is_initialized"] == want_init


def test_muonadamw_matches_reference_trajectories_and_oracle():
    """heavyball.MuonAdamW: matrices through Muon, vectors through Adam, one step counter.  Against the fixtures written
    from the reference (matrix step within the Newton-Schulz tolerance, momentum exact, vectors to 8 fp32 ulps) and,
    for the vectors, bit for bit against the oracle."""
    import glob
    import json

    import heavyball_amd
    from tests import helpers as H

    paths = sorted(glob.glob(os.path.join(GOLDEN, "traj_muonadamw_*.pt")))
    assert paths
    for path in paths:
        d = torch.load(path, weights_only=True)
        print("case", os.path.basename(path), flush=True)
        kwargs = json.loads(d["meta/kwargs"])
        if "betas" in kwargs:
            kwargs["betas"] = tuple(kwargs["betas"])
        n = len([k for k in d if k.startswith("init/p")])
        params = [torch.nn.Parameter(d[f"init/p{i}"].clone().to(DEV)) for i in range(n)]
        for p in params:
            p.grad_dtype = None  # bf16 gradients on fp32 parameters
        heavyball_amd.HBOptimizer.rounding = "half"  # param_ecc encodes the parameters at construction
        try:
            opt = heavyball_amd.MuonAdamW(params, **kwargs)
        finally:
            heavyball_amd.HBOptimizer.rounding = "philox"
        opt.rounding = "half"
        orc = muon.MuonAdamWOracle([d[f"init/p{i}"].clone() for i in range(n)], rounding=HalfRounding(), **kwargs)
        for k in range(1, d["meta/steps"] + 1):
            for i, p in enumerate(params):
                p.grad = d[f"step{k}/g{i}"].clone().to(DEV)
            opt.step()
            orc.step([d[f"step{k}/g{i}"].clone() for i in range(n)])
            torch.cuda.synchronize()
            for i, p in enumerate(params):
                st = opt.state[p][0]
                prefix = f"step{k}/state{i}/"
                want_state = {kk[len(prefix):]: d[kk] for kk in d if kk.startswith(prefix) and not kk.endswith("/step")}
                assert set(want_state) == {kk for kk in st if kk not in ("step", "is_initialized")}
                want, prev = d[f"step{k}/p{i}"], (d[f"step{k - 1}/p{i}"] if k > 1 else d[f"init/p{i}"])
                fk = f"final/is_initialized{i}"
                if want.dim() < 2:
                    # clipping carries a reduction that is summed in another order: compare in the tensor's scale there
                    check = H.assert_close_in_scale if "clip" in path else H.assert_close_to_reference
                    check({"param": p.data, **st}, {"param": want, **want_state}, f"step {k} vector {i}")
                    if "clip" not in path:  # a clip norm is summed in another order than the oracle's
                        q = orc.params[i]
                        H.assert_bit_equal(p.data, q.primary if hasattr(q, "primary") else q, f"step {k} vector {i} vs oracle")
                    assert st["is_initialized"] == (set(d[fk].tolist()) if fk in d else {0})
                else:
                    for kk, vv in want_state.items():
                        if kk == "param::ecc":
                            continue
                        if "clip" in path and "updclip" not in path:  # gradient clipping ahead of the momentum
                            assert ((st[kk].cpu().float() - vv.float()).abs() <= 2e-6 * (vv.float().abs() + vv.float().abs().max())).all(), (k, i, kk)
                        else:
                            assert torch.equal(st[kk].cpu(), vv), (k, i, kk)
                    _matrix_step_close(d, k, i, p, st)
                    assert st["is_initialized"] == (set(d[fk].tolist()) if fk in d else {2, 3, 4})


def test_splitopt_delegates_and_round_trips_state():
    """heavyball.SplitOpt (heavyball/__init__.py:1721-1762): each spec gets its own optimizer; the result equals running the
    two optimizers by hand; state_dict is {"optimizers": [...]} and loads back."""
    import heavyball_amd

    gen = torch.Generator().manual_seed(3)
    mk = lambda: ([torch.nn.Parameter((torch.randn(64, 48, generator=torch.Generator().manual_seed(1)) * 0.02).to(DEV))],
                  [torch.nn.Parameter((torch.randn(48, generator=torch.Generator().manual_seed(2)) * 0.02).to(DEV))])  # noqa: E731
    m1, v1 = mk()
    m2, v2 = mk()
    split = heavyball_amd.SplitOpt([{"params": m1, "optimizer": heavyball_amd.Muon, "lr": 0.02},
                                    {"params": v1, "optimizer": heavyball_amd.AdamW, "lr": 1e-3},
                                    {"params": [], "optimizer": heavyball_amd.AdamW}])  # fmt: skip
    assert len(split.optimizers) == 2
    a, b = heavyball_amd.Muon(m2, lr=0.02), heavyball_amd.AdamW(v2, lr=1e-3)
    for o in (*split.optimizers, a, b):
        o.rounding = "half"
    for k in range(3):
        gm, gv = torch.randn(64, 48, generator=gen) * 1e-2, torch.randn(48, generator=gen) * 1e-2
        m1[0].grad, v1[0].grad, m2[0].grad, v2[0].grad = gm.to(DEV), gv.to(DEV), gm.to(DEV), gv.to(DEV)
        split.step()
        a.step()
        b.step()
    torch.cuda.synchronize()
    assert torch.equal(m1[0].data, m2[0].data) and torch.equal(v1[0].data, v2[0].data)
    sd = split.state_dict()
    assert list(sd.keys()) == ["optimizers"] and len(sd["optimizers"]) == 2
    split.load_state_dict(sd)
    split.zero_grad()
    with pytest.raises(ValueError):
        heavyball_amd.SplitOpt([{"params": [], "optimizer": heavyball_amd.AdamW}])
