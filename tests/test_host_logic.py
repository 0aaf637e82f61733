"""Host layer without a GPU: keyword handling, param-group contents, slab layout, step scalars, failure without a device.
(heavyball/chainable.py:197-220, :2387-2408; test/test_optimizer_cpu_smoke.py:87-98; test/test_ecc.py:551-560)"""

import json
import os
import warnings

import numpy as np
import pytest
import torch

import heavyball_amd
from heavyball_amd import _lib, optim, slab
from heavyball_amd.muon import NS_COEFFS, ns_coefficients

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def params():
    return [torch.nn.Parameter(torch.randn(8, 16)), torch.nn.Parameter(torch.randn(16))]


@pytest.mark.parametrize("cls", [heavyball_amd.AdamW, heavyball_amd.LaProp, heavyball_amd.Muon])
def test_keyword_errors(cls):
    with pytest.raises(TypeError, match="unknown keyword arguments"):
        cls(params(), not_a_real_kwarg=1)
    with pytest.raises(TypeError, match="Removed in HeavyBall 3.0"):
        cls(params(), stochastic_schedule=True)
    with warnings.catch_warnings(record=True) as w:
        warnings.simplefilter("always")
        opt = cls(params(), foreach=False)
    assert any(issubclass(x.category, FutureWarning) and "multi_tensor" in str(x.message) for x in w)
    assert opt.param_groups[0]["multi_tensor"] is False and "foreach" not in opt.param_groups[0]


@pytest.mark.parametrize("name,cls,kw", [("AdamW", heavyball_amd.AdamW, {}), ("LaProp_ecc", heavyball_amd.LaProp, {"ecc": "bf16+8"}),
                                         ("AdamW_mars", heavyball_amd.AdamW, {"mars": True}), ("Muon", heavyball_amd.Muon, {}),
                                         ("ADOPT", heavyball_amd.ADOPT, {}), ("AdEMAMix", heavyball_amd.AdEMAMix, {}),
                                         ("NAdam", heavyball_amd.NAdam, {})])  # fmt: skip
def test_param_group_keys_match_reference(name, cls, kw):
    """Everything the reference keeps in a param group before the first step, and nothing it removes
    (compile_step, promote, gradient_clipping, update_clipping, palm, orig_shapes)."""
    layout = json.load(open(os.path.join(GOLDEN, "layout.json")))[name]
    opt = cls(params(), **kw)
    after_step = {"base_lr", "is_preconditioning", "param_count", "prev_lr", "step"}
    want = set(layout["param_group_keys"]) - after_step
    assert set(opt.param_groups[0].keys()) == want
    for k, v in layout["param_group_values"].items():
        if k in after_step:
            continue
        got = opt.param_groups[0][k]
        assert (repr(got) == v) if isinstance(v, str) and not isinstance(got, str) else (got == v), (k, got, v)


def test_instance_attrs_are_not_group_keys():
    opt = heavyball_amd.AdamW(params(), compile_step=False, promote=True, consume_grad=False)
    assert opt.promote is True and opt.consume_grad is False
    for k in ("compile_step", "promote", "consume_grad", "gradient_clipping", "update_clipping", "palm"):
        assert k not in opt.param_groups[0]


def test_unknown_ecc_mode_and_clipping_name():
    with pytest.raises(KeyError):
        heavyball_amd.AdamW(params(), ecc="bf16+4")
    with pytest.raises(ValueError, match="Unknown function"):
        heavyball_amd.AdamW(params(), gradient_clipping="not_a_clip")
    heavyball_amd.AdamW(params(), gradient_clipping="l2_clip_")  # accepted name


def test_step_without_gpu_fails_loudly():
    p = params()
    opt = heavyball_amd.LaProp(p)
    p[0].grad = torch.zeros_like(p[0])
    with pytest.raises(_lib.HbError):
        opt.step()
    g = opt.param_groups[0]
    assert g["step"] is None and g["lr"] == g["base_lr"]  # restored by the finally of the step (chainable.py:2567-2570)
    with pytest.raises(_lib.HbError):
        heavyball_amd.AdamW(params(), param_ecc="bf16+8")  # the initial ECC encode needs the device too


def test_slab_layout_and_chunk_table():
    numels = [5000, 0, 4096, 1, 12289]
    offsets, total = slab.layout(numels)
    assert offsets.tolist() == [0, 8192, 8192, 12288, 16384] and total == 16384 + 16384
    assert all(o % _lib.chunk_elems() == 0 for o in offsets)
    slab.check_no_overlap(offsets, numels)
    with pytest.raises(ValueError):
        slab.check_no_overlap(np.array([0, 4000]), [4096, 10])
    tab = slab.chunk_table(numels, [0, 2, 3, 4])
    assert tab.tolist() == [[0, 0], [0, 1], [2, 0], [3, 0], [4, 0], [4, 1], [4, 2], [4, 3]]
    assert slab.chunk_table(numels, []).shape == (0, 2)
    s = slab.Slab([torch.Size([3, 5]), torch.Size([7])], torch.device("cpu"))
    s.role("x", torch.float32)
    v = s.view("x", 1)
    v.fill_(2.0)
    assert s.roles["x"][4096:4103].tolist() == [2.0] * 7 and s.roles["x"][:15].sum() == 0
    with pytest.raises(TypeError):
        s.role("x", torch.bfloat16)


def test_parameters_are_rehomed_into_the_slab():
    p = params()
    before = [q.detach().clone() for q in p]
    opt = heavyball_amd.AdamW(p)
    b = opt._buckets[0][0]
    for i, q in enumerate(p):
        assert torch.equal(q.data, before[i])
        assert q.data.data_ptr() == b.slab.view("param", i).data_ptr()


def test_step_scalars_match_reference_bits():
    """The host's debiased betas / lerp weights / lr against the bit patterns recorded from the reference."""
    sc = json.load(open(os.path.join(GOLDEN, "scalars.json")))
    hx = lambda x: "%08x" % (torch.tensor(x, dtype=torch.float32).view(torch.int32).item() & 0xFFFFFFFF)  # noqa: E731
    for key, rows in sc.items():
        if not key.startswith("betas_"):
            continue
        _, b1, b2 = key.split("_")
        for s, row in enumerate(rows, start=1):
            step = torch.tensor(s, dtype=torch.int64)
            d1 = optim.beta_debias(optim.f32(float(b1)), step)
            a1, oma1 = optim.lerp_weights(d1)
            d2 = optim.beta_debias(optim.f32(float(b2)), step)
            a2, oma2 = optim.lerp_weights(d2)
            assert [hx(float(d1)), hx(a1), hx(oma1), hx(float(d2)), hx(a2), hx(oma2)] == row
            # the step's own fast path: same bits with the IEEE operations on numpy scalars
            assert optim.debiased_weights(optim.f32(float(b1)), step) == (a1, oma1)
            assert optim.debiased_weights(optim.f32(float(b2)), step) == (a2, oma2)
            # and the cached-plan step's, which takes the power on numpy scalars too
            assert optim.debiased_weights_np(float(b1), s) == (a1, oma1)
            assert optim.debiased_weights_np(float(b2), s) == (a2, oma2)
    for key, rows in sc.items():
        if not key.startswith("lr_"):
            continue
        _, base_lr, warm = key.split("_")
        for s, want in enumerate(rows, start=1):
            assert hx(float(optim.step_lr_np(float(base_lr), s, int(warm)))) == want, (key, s)


def test_debiased_weights_equal_the_tensor_pipeline():
    """``debiased_weights`` against ``lerp_weights(beta_debias(...))`` on 0-d tensors, bit for bit, over many betas and steps
    (including beta = 0, where the debiased beta is 0, and steps at which beta**step underflows)."""
    gen = torch.Generator().manual_seed(3)
    betas = [0.0, 0.5, 0.9, 0.95, 0.99, 0.999, 0.9999, 1e-3] + torch.rand(40, generator=gen).tolist()
    steps = list(range(1, 40)) + [100, 1000, 12345, 10**6, 10**9]
    for b in betas:
        beta = optim.f32(b)
        for s in steps:
            step = torch.tensor(s, dtype=torch.int64)
            assert optim.debiased_weights(beta, step) == optim.lerp_weights(optim.beta_debias(beta, step)), (b, s)
            assert optim.debiased_weights_np(b, s) == optim.lerp_weights(optim.beta_debias(beta, step)), (b, s)


def test_numpy_step_scalars_equal_the_tensor_pipeline():
    """The scalars of the cached-plan step (numpy float32 scalars) against the general path's 0-d tensor arithmetic, bit for bit:
    the learning rate with warm-up, ``1 - decay * lr`` and ``-lr``, over learning rates, warm-ups, decays and steps - including
    steps beyond 2**24, where the step itself is rounded on its way to fp32."""
    import numpy as np

    gen = torch.Generator().manual_seed(5)
    lrs = [1e-3, 0.0025, 3e-3, 1.0, 0.1] + (torch.rand(20, generator=gen) * 1e-2).tolist()
    steps = list(range(1, 60)) + [1000, 99999, 2**24 + 1, 2**24 + 3, 10**9 + 7]
    for base_lr in lrs:
        for warm in (0, 3, 10, 2000):
            for s in steps:
                step = torch.tensor(s, dtype=torch.int64)
                want = optim.f32(base_lr * step / step.clamp(min=warm + 1))
                got = optim.step_lr_np(base_lr, s, warm)
                assert float(got) == float(want), (base_lr, warm, s)
                for decay in (0.0, 0.01, 0.1, 1e-4):
                    assert float(np.float32(1) - np.float32(decay) * got) == float(1 - optim.f32(decay) * want)
                assert float(-got) == float(-want)


def test_ns_coefficients_follow_cpu_scalar_rounding():
    c = ns_coefficients(NS_COEFFS)
    assert len(c) == 15
    assert c[0] == 4.09375 and c[1] == -6.90625  # a, b rounded to bf16 (in-place bf16 add casts its scalar)
    assert abs(c[2] - 2.9270) < 1e-6 and c[2] != float(torch.tensor(2.9270).bfloat16())  # c stays fp32


def test_corr_over_smax_newton_step_is_correctly_rounded_for_every_correction():
    """The kernels decode ``corr / smax`` (heavyball/utils.py:1298, an fp32 divide) as q0 = c * r, q = fma(fma(-q0, smax, c), r, q0)
    with r = fl32(1 / smax): exhaustively, for every int16 value and both smax (127, 32767), that equals the correctly
    rounded quotient.  numpy has no fma; the two fused steps are evaluated in float64, where products of fp32 values
    are exact and each sum carries one rounding to fp32 that cannot be a double rounding (the exact results have at most
    48 + 24 significant bits only in the first step, whose result c - q0 * smax is exactly representable)."""
    import numpy as np

    c = np.arange(-32768, 32768, dtype=np.int64)
    for smax in (127.0, 32767.0):
        cf = c.astype(np.float32)
        sm = np.float32(smax)
        r = np.float32(1.0) / sm
        want = cf / sm  # IEEE fp32 division
        q0 = cf * r
        rem = (cf.astype(np.float64) - q0.astype(np.float64) * np.float64(sm)).astype(np.float32)  # exact: |rem| < ulp(c), few bits
        assert np.array_equal(rem.astype(np.float64), cf.astype(np.float64) - q0.astype(np.float64) * np.float64(sm))
        exact = q0.astype(np.float64) + rem.astype(np.float64) * np.float64(r)  # 24 x 24-bit product plus a 24-bit value
        q = exact.astype(np.float32)
        # the float64 sum is itself rounded (to 53 bits) before the rounding to fp32: where it falls within one float64 ulp
        # of an fp32 rounding boundary the two-step result could differ from the fused one; no case comes that close
        mid = (q.astype(np.float64) + np.nextafter(q, np.where(exact > q, np.float32(np.inf), np.float32(-np.inf))).astype(np.float64)) / 2
        assert (np.abs(exact - mid) > 4 * np.spacing(np.abs(exact))).all()
        assert np.array_equal(q.view(np.uint32), want.view(np.uint32)), smax


def test_cpp_tensor_loop_checks_what_the_python_loop_checks():
    """csrc/hostloop.cpp on CPU tensors: the gradients' addresses when every tensor passes, and the reason code for each thing that
    sends a step back to the general path (a missing gradient, another dtype, a strided gradient, a misaligned one, a parameter
    whose data moved); ``drop_grads`` leaves every gradient None."""
    helper = optim.hostloop()
    assert helper is not None, "heavyball_amd/_hostloop.so has not been built (make -C heavyball_amd/csrc)"
    ps = [torch.nn.Parameter(torch.randn(8, 16)) for _ in range(5)]
    for p in ps:
        p.grad_dtype = None
    gs = [torch.randn(8, 16).bfloat16() for _ in ps]

    def arm():
        for p, g in zip(ps, gs):
            p.grad = g

    arm()
    home = torch.tensor([p.data_ptr() for p in ps], dtype=torch.int64)
    out = torch.zeros(len(ps), dtype=torch.int64)
    assert helper.collect(ps, home, out, torch.bfloat16) == 0
    assert out.tolist() == [g.data_ptr() for g in gs]
    assert helper.collect(ps, home, out, torch.float32) == 2
    ps[3].grad = None
    assert helper.collect(ps, home, out, torch.bfloat16) == 1
    arm()
    ps[1].grad = torch.randn(16, 8).bfloat16().t()  # same shape, column-major
    assert helper.collect(ps, home, out, torch.bfloat16) == 3
    arm()
    ps[2].grad = torch.randn(8 * 16 + 1).bfloat16()[1:].view(8, 16)  # two bytes off a 16-byte boundary
    assert ps[2].grad.data_ptr() % 16 and helper.collect(ps, home, out, torch.bfloat16) == 4
    arm()
    ps[4].data = ps[4].data.clone()
    assert helper.collect(ps, home, out, torch.bfloat16) == 5
    assert helper.collect(ps, home[:3], out, torch.bfloat16) == 6  # tables of another length
    helper.drop_grads(ps)
    assert all(p.grad is None for p in ps)
