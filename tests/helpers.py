"""Shared pieces of the parity tests: run the HIP optimizer and the CPU oracle on identical seeded inputs and compare
every parameter and state tensor bit for bit."""

import torch

from oracle import first_order as fo
from oracle.ecc import EccTensor
from oracle.rounding import HalfRounding, PhiloxRounding


def bits(t):
    t = t.detach().cpu()
    if t.dtype == torch.float32:
        return t.view(torch.int32)
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16)
    return t


def assert_bit_equal(got, want, what):
    got, want = got.detach().cpu(), want.detach().cpu()
    assert got.dtype == want.dtype, f"{what}: dtype {got.dtype} vs {want.dtype}"
    assert got.shape == want.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(want.shape)}"
    a, b = bits(got), bits(want)
    if not torch.equal(a, b):
        bad = (a != b).nonzero()
        first = tuple(bad[0].tolist())
        raise AssertionError(
            f"{what}: {bad.shape[0]} of {got.numel()} elements differ; first at {first}: got {got[first].item()!r} want {want[first].item()!r}"
        )


def ulp_distance(a, b):
    """Distance in units in the last place between two float tensors of the same dtype (sign-magnitude ordered)."""
    ia, ib = bits(a).to(torch.int64), bits(b).to(torch.int64)
    width = 32 if a.dtype == torch.float32 else 16
    sign = 1 << (width - 1)
    ia = torch.where(ia < 0, -(ia & (sign - 1)), ia)
    ib = torch.where(ib < 0, -(ib & (sign - 1)), ib)
    return (ia - ib).abs()


FP32_ULPS = 8  # 8 * 2^-23 = 9.5e-7: the 1e-6 relative bound on fp32 moments and parameters


def assert_close_to_reference(got: dict, want: dict, what: str):
    """Compare tensors of one parameter (its value under "param" plus its state entries) with what the reference itself
    produced.  The reference's CPU square root is within 1 ulp but not correctly rounded, so agreement is to the stated
    tolerance, not bit for bit: fp32 within FP32_ULPS ulps; plain bf16 within 1 bf16 ulp; an ECC pair (primary +
    "::ecc" correction) within one correction unit of the decoded value."""
    from oracle.ecc import EccTensor, log_ulp

    for key, w in want.items():
        if key.endswith("::ecc") or not isinstance(w, torch.Tensor) or key == "step":
            continue
        assert key in got, f"{what}: missing {key}"
        g = got[key].detach().cpu()
        w = w.detach().cpu()
        assert g.dtype == w.dtype and g.shape == w.shape, f"{what} {key}: {g.dtype}{tuple(g.shape)} vs {w.dtype}{tuple(w.shape)}"
        ck = "param::ecc" if key == "param" else key + "::ecc"
        if ck in want:
            gc, wc = got[ck].detach().cpu(), want[ck].detach().cpu()
            assert gc.dtype == wc.dtype, f"{what} {ck}: {gc.dtype} vs {wc.dtype}"
            gd, wd = EccTensor(g, gc).decode(), EccTensor(w, wc).decode()
            unit = torch.exp2(log_ulp(w).float() - 1) / EccTensor(w, wc).smax
            tol = unit * 1.001 + wd.abs() * (FP32_ULPS * 2.0**-23)
            bad = (gd - wd).abs() > tol
            assert not bad.any(), f"{what} {key} (ECC): {int(bad.sum())} of {w.numel()} decoded values off by more than one correction unit"
        elif w.dtype == torch.float32:
            d = ulp_distance(g, w)
            assert d.max() <= FP32_ULPS, f"{what} {key}: up to {int(d.max())} ulps from the reference ({int((d > 0).sum())} of {w.numel()} differ)"
        elif w.dtype in (torch.bfloat16, torch.float16):
            d = ulp_distance(g, w)
            assert d.max() <= 1, f"{what} {key}: up to {int(d.max())} {w.dtype} ulps from the reference"
        else:
            assert torch.equal(g, w), f"{what} {key}"


def assert_close_in_scale(got: dict, want: dict, what: str, rel: float = 2e-6):
    """Like assert_close_to_reference, for quantities that carry a norm computed by a reduction (gradient clipping): the
    reduction order moves the clip scale by an ulp, and a moment that nearly cancels then differs by many of ITS ulps
    while the error stays at ``rel`` of the tensor's magnitude.  |got - want| <= rel * (|want| + max|want|), plus one
    correction unit for an ECC pair and one ulp for a plain 16-bit tensor."""
    from oracle.ecc import EccTensor, log_ulp

    for key, w in want.items():
        if key.endswith("::ecc") or not isinstance(w, torch.Tensor) or key == "step":
            continue
        assert key in got, f"{what}: missing {key}"
        g, w = got[key].detach().cpu(), w.detach().cpu()
        assert g.dtype == w.dtype and g.shape == w.shape, f"{what} {key}"
        ck = "param::ecc" if key == "param" else key + "::ecc"
        extra = 0.0
        if ck in want:
            gc, wc = got[ck].detach().cpu(), want[ck].detach().cpu()
            extra = torch.exp2(log_ulp(w).float() - 1) / EccTensor(w, wc).smax * 1.001
            g, w = EccTensor(g, gc).decode(), EccTensor(w, wc).decode()
        elif w.dtype in (torch.bfloat16, torch.float16):
            extra = (w.float().abs() * (2.0**-7 if w.dtype == torch.bfloat16 else 2.0**-10)).clamp(min=1e-30)
            g, w = g.float(), w.float()
        tol = rel * (w.abs() + w.abs().max()) + extra
        bad = (g - w).abs() > tol
        assert not bad.any(), f"{what} {key}: {int(bad.sum())} of {w.numel()} outside {rel:g} of the tensor's scale, worst {float(((g - w).abs() / tol).max()):.2f}x"


def make_params(shapes, device, seed=0, scale=0.02):
    gen = torch.Generator().manual_seed(seed)
    host = [torch.randn(s, generator=gen) * scale for s in shapes]
    params = [torch.nn.Parameter(h.clone().to(device)) for h in host]
    for p in params:
        p.grad_dtype = None  # allow a gradient dtype other than the parameter's
    return host, params


def make_grads(shapes, k, dtype, scale):
    g = torch.Generator().manual_seed(1000 + k)
    return [(torch.randn(s, generator=g) * scale).to(dtype) for s in shapes]


def build_pair(cls, kind, shapes, kwargs, device, rounding="philox", seed=77):
    host, params = make_params(shapes, device)
    opt = cls(params, **kwargs)
    opt.rounding = rounding
    opt.rng_seed = seed
    if kwargs.get("param_ecc"):
        # the constructor already encoded the parameters with the default seed: redo it with the test's settings
        for b in opt._buckets[0]:
            for i, p in enumerate(b.params):
                j = [id(q) for q in params].index(id(p))
                opt._encode_param(b, i, host[j].to(device).contiguous(), opt.param_groups[0])
    base = opt._buckets[0][0].slab.offsets_np.tolist()
    r = HalfRounding() if rounding == "half" else PhiloxRounding(seed, base=base)
    orc = fo.FirstOrderOracle(kind, [h.clone() for h in host], rounding=r, **kwargs)
    return host, params, opt, orc


def compare(opt, orc, params, what=""):
    torch.cuda.synchronize()
    for i, p in enumerate(params):
        want = orc.params[i]
        want = want.primary if isinstance(want, EccTensor) else want
        assert_bit_equal(p.data, want, f"{what} param {i}")
        st = opt.state[p].get(0, {}) if p in opt.state else {}
        for key, val in orc.state[i].items():
            if key == "step":
                assert int(st["step"]) == int(val)
                continue
            assert key in st, f"{what} tensor {i}: missing state key {key}; have {sorted(k for k in st if isinstance(k, str))}"
            if not isinstance(val, torch.Tensor):  # plain counters such as ADOPT's "_warmup_1"
                assert st[key] == val, f"{what} tensor {i} {key}: {st[key]!r} vs {val!r}"
                continue
            assert_bit_equal(st[key], val, f"{what} tensor {i} {key}")


def run_steps(opt, orc, params, shapes, steps, grad_dtype, grad_scale, device, none_for=None, check_each=True, tag=""):
    for k in range(1, steps + 1):
        grads = make_grads(shapes, k, grad_dtype, grad_scale)
        if none_for is not None and k in none_for:
            for i in none_for[k]:
                grads[i] = None
        for p, g in zip(params, grads):
            p.grad = None if g is None else g.to(device)
        opt.step()
        orc.step([None if g is None else g.clone() for g in grads])
        assert all(p.grad is None for p in params)
        if check_each or k == steps:
            compare(opt, orc, params, f"{tag} step {k}")


def whole_from_blocks(d, prefix, key, shape, kwargs):
    """A per-view state entry of a fixture (``prefix + key`` for block 0, ``prefix + "block<k>/" + key`` for the others) put
    together in the parameter's own layout; the entry itself when the parameter is not cut."""
    from oracle.soap import dim_merger

    first = d[prefix + key]
    if not (kwargs.get("split") and kwargs.get("merge_dims", True)) or tuple(first.shape) == tuple(shape):
        return first
    n = 1
    for s_ in shape:
        n *= s_
    places = dim_merger(torch.arange(n).reshape(shape), kwargs.get("max_precond_dim", 2048), True)
    out = torch.empty(n, dtype=first.dtype)
    for k, idx in enumerate(places):
        out[idx.reshape(-1)] = d[prefix + (f"block{k}/" if k else "") + key].reshape(-1)
    return out.reshape(shape)
