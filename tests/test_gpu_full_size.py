"""The benchmark configurations at their full sizes.

First-order steps: the GPT-2-small-shaped set (123.65 M elements) is small enough for the CPU oracle, so it is compared
whole, bit for bit; of the Llama-3-8B-shaped set (8.03 G elements, flat slab offsets beyond 2^32) the step runs on all 291
tensors and a handful of whole tensors from both ends of the slab are compared with the oracle, which is given their slab
offsets (every tensor is independent of the others: the caution count is per tensor, the Philox counter is the element's
flat slab index).
Newton-Schulz on the seven matrices of one Llama-3-8B layer and SOAP's products and orthonormalisation on the [2048, 8192]
matrix, where the CPU oracle would take minutes, are checked through size-independent properties; the small-size tests
carry their comparison against the oracle, these show that the same code paths (grouped launches over thousands of tiles,
256-wide tiles, split-K) keep the invariants at scale."""

import ctypes

import pytest
import torch

import heavyball_amd
from heavyball_amd import _lib, muon
from heavyball_amd.soap import _Gemm, orthonormalize_
from oracle import first_order as fo
from oracle.rounding import PhiloxRounding

from tests import helpers as H

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")
C4_SHAPES = [(4096, 4096), (4096, 4096), (1024, 4096), (1024, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]


def _gpt2_small_shapes():
    shapes = []
    for _ in range(12):
        shapes += [(768,), (768,), (768, 2304), (2304,), (768, 768), (768,), (768,), (768,), (768, 3072), (3072,), (3072, 768), (768,)]
    return shapes + [(768,), (768,), (50257, 768)]


def _llama8b_shapes():
    shapes = []
    for _ in range(32):
        shapes += [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336), (4096,), (4096,)]
    return shapes + [(128256, 4096), (128256, 4096), (4096,)]


def test_c2_full_size_matches_oracle():
    """Benchmark configuration 2 whole: LaProp ecc=bf16+8 on the 147 GPT-2-small-shaped tensors, fp32 parameters, bf16
    gradients, shared Philox stream, two steps, every parameter and state bit-identical to the oracle."""
    shapes = _gpt2_small_shapes()
    assert sum(int(torch.Size(s).numel()) for s in shapes) == 123_653_376
    host, params, opt, orc = H.build_pair(heavyball_amd.LaProp, "laprop", shapes, dict(ecc="bf16+8"), DEV)
    H.run_steps(opt, orc, params, shapes, 2, torch.bfloat16, 1e-3, DEV, check_each=False, tag="C2 full size")


def test_c3_full_size_tensors_from_both_ends_match_oracle():
    """Benchmark configuration 3 whole on the GPU: AdamW mars + caution + ecc + param_ecc on the 291 Llama-3-8B-shaped
    tensors (112 GB of parameters and state), two steps.  Compared with the oracle, bit for bit: the first q and k
    projections and a norm weight (slab offsets from 0), the k projection and norm weights of the last layer and the final
    norm weight (slab offsets 6.9e9 ... 8.03e9 elements, i.e. beyond 32 bits), each with its construction-time param_ecc
    encoding, caution count and Philox streams."""
    free, _ = torch.cuda.mem_get_info(DEV)
    if free < 200 * 2**30:
        pytest.skip("needs 200 GiB of free device memory")
    shapes = _llama8b_shapes()
    assert sum(int(torch.Size(s).numel()) for s in shapes) == 8_030_261_248
    last = 9 * 31
    sel = [0, 1, 7, last + 1, last + 7, last + 8, len(shapes) - 1]
    assert [shapes[i] for i in sel] == [(4096, 4096), (1024, 4096), (4096,), (1024, 4096), (4096,), (4096,), (4096,)]
    kwargs = dict(mars=True, caution=True, ecc="bf16+8", param_ecc="bf16+8")
    torch.manual_seed(77)  # the optimizer takes its Philox seed from torch's at construction, where param_ecc encodes
    params, host = [], {}
    for i, sh in enumerate(shapes):
        p = torch.nn.Parameter(torch.randn(sh, device=DEV) * 0.02)
        p.grad_dtype = None
        if i in sel:
            host[i] = p.detach().cpu().clone()
        params.append(p)
    opt = heavyball_amd.AdamW(params, **kwargs)
    assert opt.rng_seed == 77 and opt.rounding == "philox"
    offsets = opt._buckets[0][0].slab.offsets_np
    assert int(offsets[sel[-1]]) > 2**32
    orc = fo.FirstOrderOracle("adam", [host[i] for i in sel], rounding=PhiloxRounding(77, base=[int(offsets[i]) for i in sel]), **kwargs)
    picked = [params[i] for i in sel]
    H.compare(opt, orc, picked, "C3 full size, after construction")
    for k in (1, 2):
        print("step", k, flush=True)
        hg = []
        for i, (p, sh) in enumerate(zip(params, shapes)):
            p.grad = (torch.randn(sh, device=DEV) * 1e-3).to(torch.bfloat16)
            if i in sel:
                hg.append(p.grad.cpu().clone())
        opt.step()
        orc.step(hg)
        H.compare(opt, orc, picked, f"C3 full size step {k}")
    del opt, params
    torch.cuda.empty_cache()


def _ns5_batched(grads, rng_mode=_lib.RNG_HALF):
    L = _lib.lib()
    n = len(grads)
    rows = (ctypes.c_int64 * n)(*[g.shape[0] for g in grads])
    cols = (ctypes.c_int64 * n)(*[g.shape[1] for g in grads])
    nb = ctypes.c_int64()
    _lib.check(L.hb_ns5_batched_workspace_bytes(n, rows, cols, ctypes.byref(nb)))
    ws = torch.empty(nb.value, dtype=torch.uint8, device=DEV)
    outs = [torch.empty_like(g) for g in grads]
    arr = (ctypes.c_float * 15)(*muon.ns_coefficients(muon.NS_COEFFS))
    gp = (ctypes.c_void_p * n)(*[g.data_ptr() for g in grads])
    op = (ctypes.c_void_p * n)(*[o.data_ptr() for o in outs])
    scale = (ctypes.c_float * n)(*([1.0] * n))
    base = (ctypes.c_int64 * n)(*([0] * n))
    _lib.check(L.hb_ns5_batched(n, gp, op, rows, cols, arr, 0, 1e-7, scale, rng_mode, 1, 1, base, ws.data_ptr(), nb.value, None))
    torch.cuda.synchronize()
    return outs


def test_newton_schulz_on_a_llama_layer():
    """(a) the singular values of every output lie in the band the five-step schedule maps the input's into;
    (b) the iteration normalises its input, so scaling the gradient by a power of two changes nothing, bit for bit;
    (c) a matrix gives the same bits in the batch of seven and on its own;
    (d) one matrix of each of the four shapes against the oracle."""
    torch.manual_seed(5)
    grads = [torch.randn(s, device=DEV) * 1e-2 for s in C4_SHAPES]
    outs = _ns5_batched(grads)
    for g, o in zip(grads, outs):
        print("case", tuple(g.shape), flush=True)
        assert torch.isfinite(o).all()
        small = o if o.shape[0] <= o.shape[1] else o.T
        ev = torch.linalg.eigvalsh((small @ small.T).double())  # squares of the singular values
        sv = ev.clamp(min=0).sqrt()
        assert sv.max() < 1.35, (tuple(g.shape), sv.max().item())
        if g.shape[0] != g.shape[1]:  # aspect >= 3.5: a well-conditioned input, every singular value is lifted
            assert sv.min() > 0.3, (tuple(g.shape), sv.min().item())
        else:  # a square Gaussian matrix has singular values down to ~0, which five steps cannot lift; the bulk is
            assert (sv > 0.6).double().mean() > 0.85, (tuple(g.shape), (sv > 0.6).double().mean().item())
    scaled = _ns5_batched([g * 4.0 for g in grads])
    for a, b in zip(outs, scaled):
        assert torch.equal(a, b)
    alone = _ns5_batched([grads[4]])[0]
    assert torch.equal(alone, outs[4])
    # (d) one matrix of each shape against the oracle (15 bf16 products each on the CPU): 2e-2 relative Frobenius
    from oracle import muon as omuon
    from oracle.rounding import HalfRounding

    for i in (0, 2, 4, 6):
        want = omuon.orthogonal(grads[i].cpu().clone(), HalfRounding(), 0)
        want = want / max(1, grads[i].shape[0] / grads[i].shape[1]) ** 0.5  # _ns5_batched above runs with a post-scale of 1
        err = ((outs[i].cpu().double() - want.double()).norm() / want.double().norm()).item()
        print(tuple(grads[i].shape), "vs oracle, rel fro", err, flush=True)
        assert err < 2e-2


@pytest.mark.parametrize("n", [2048, 4096])
def test_legacy_newton_schulz_matches_oracle_on_square_matrices(n):
    """The legacy schedule (one coefficient triple, the norm taken after the bf16 cast, a second stochastic round;
    heavyball/utils.py:637-657) applies to square matrices only.  At these sizes the products run on the 256-square
    tile class with mirrored symmetric tiles, which the small reference vectors (16 and 64 wide) never reach."""
    from oracle import muon as omuon
    from oracle.rounding import HalfRounding

    L = _lib.lib()
    print("case legacy", n, flush=True)
    torch.manual_seed(40 + n)
    g = torch.randn(n, n, device=DEV) * 1e-2
    nb = ctypes.c_int64()
    _lib.check(L.hb_ns5_workspace_bytes(n, n, ctypes.byref(nb)))
    ws = torch.empty(nb.value, dtype=torch.uint8, device=DEV)
    out = torch.empty_like(g)
    arr = (ctypes.c_float * 15)(*muon.ns_coefficients(muon.LEGACY_COEFFS))
    _lib.check(L.hb_ns5(g.data_ptr(), out.data_ptr(), n, n, arr, _lib.NS_LEGACY, 1e-7, 1.0, _lib.RNG_HALF, 1, 1, 0, ws.data_ptr(), nb.value, None))
    torch.cuda.synchronize()
    want = omuon.orthogonal(g.cpu().clone(), HalfRounding(), 0, mode="legacy_newtonschulz")
    err = ((out.cpu().double() - want.double()).norm() / want.double().norm()).item()
    print("legacy", n, "vs oracle, rel fro", err, flush=True)
    assert err < 2e-2
    # the legacy triple maps singular values into a band around 1 as well (wider than the default schedule's)
    sv = torch.linalg.eigvalsh((out @ out.T).double()).clamp(min=0).sqrt()
    assert sv.max() < 1.35 and (sv > 0.6).double().mean() > 0.85


def test_soap_products_and_orthonormalisation_at_full_size():
    """[2048, 8192]: an orthonormal basis from hb_orthonormalize_f32 on each side, rotate and rotate back (four GEMMs in
    all four operand orientations) returns the matrix; the factor product is symmetric and matches a float64 row."""
    torch.manual_seed(6)
    m, n = 2048, 8192
    G = torch.randn(m, n, device=DEV) * 1e-2
    Ql = torch.randn(m, m, device=DEV)
    Qr = torch.randn(n, n, device=DEV)
    assert orthonormalize_(Ql) and orthonormalize_(Qr)
    eye = torch.eye(n, device=DEV)
    assert (Qr.T @ Qr - eye).abs().max() < 5e-5
    gemm = _Gemm(DEV)
    t1, t2, t3, t4 = torch.empty_like(G), torch.empty_like(G), torch.empty_like(G), torch.empty_like(G)
    gemm(Ql, G, t1, ta=True)  # Ql^T G
    gemm(t1, Qr, t2)  # (.) Qr
    gemm(Ql, t2, t3)  # Ql (.)
    gemm(t3, Qr, t4, tb=True)  # (.) Qr^T
    torch.cuda.synchronize()
    assert ((t4 - G).norm() / G.norm()).item() < 2e-5
    assert abs((t2.norm() / G.norm()).item() - 1.0) < 1e-4  # rotations keep the Frobenius norm
    GG = torch.zeros(n, n, device=DEV)
    gemm(G, G, GG, ta=True, accumulate=True, alpha=1.0, beta=0.0)
    torch.cuda.synchronize()
    assert torch.equal(GG, GG.T)  # both triangles accumulate the same products in the same order
    want = G.double().T[:4] @ G.double()
    assert torch.allclose(GG[:4].double(), want, rtol=1e-5, atol=1e-6 * want.abs().max().item())  # sums of 2048 cancelling products
