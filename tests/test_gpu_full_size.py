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


@pytest.mark.timeout(600)
def test_muon_step_on_llama_sized_matrices_matches_oracle():
    """``Muon.step()`` end to end (momentum, grouped Newton-Schulz on the 256-wide tile class, ``update_param_``) on a [1024, 4096]
    and a [4096, 4096] matrix plus a vector, two steps against the oracle: the momentum bit for bit, the vector's parameter bit
    for bit, each matrix' step to the Newton-Schulz tolerance (2e-2 relative Frobenius)."""
    from oracle import muon as omuon
    from oracle.rounding import HalfRounding

    shapes = [(1024, 4096), (4096,), (4096, 4096)]
    host, params = H.make_params(shapes, DEV)
    kwargs = dict(betas=(0.95, 0.99), weight_decay=0.01, lr=0.02)
    opt = heavyball_amd.Muon(params, **kwargs)
    opt.rounding = "half"
    orc = omuon.MuonOracle([h.clone() for h in host], rounding=HalfRounding(), **kwargs)
    for k in (1, 2):
        print("case step", k, flush=True)
        grads = H.make_grads(shapes, k, torch.float32, 1e-2)
        prev = [p.detach().cpu().clone() for p in params]
        prev_o = [p.clone() for p in orc.params]
        for p, g in zip(params, grads):
            p.grad = g.to(DEV)
        opt.step()
        orc.step([g.clone() for g in grads])
        torch.cuda.synchronize()
        for i, p in enumerate(params):
            H.assert_bit_equal(opt.state[p][0][opt.KEY], orc.state[i][orc.KEY], f"step {k} momentum {i}")
            if p.dim() < 2:
                H.assert_bit_equal(p.data, orc.params[i], f"step {k} vector {i}")
                continue
            got, want = (p.detach().cpu() - prev[i]).double(), (orc.params[i] - prev_o[i]).double()
            err = ((got - want).norm() / want.norm()).item()
            print(tuple(p.shape), "step vs oracle, rel fro", err, flush=True)
            assert err < 2e-2, (k, i, err)


@pytest.mark.timeout(900)
def test_soap_with_both_factors_at_benchmark_shapes():
    """The SOAP benchmark configuration as stated (max_precond_dim = 8192: every side of [2048, 2048], [2048, 8192] and
    [8192, 2048] has a factor and a basis) through ``SOAP.step()``: initialisation, a step with a basis refresh and a plain step
    in the refreshed basis (precondition_frequency = 2).  A float64 eigh of an 8192-wide factor on the CPU would take minutes,
    so every step is checked through what it must satisfy, recomputed on the device in float64 from the optimizer's own state:

      * the bases after initialisation are orthonormal and diagonalise their factors, eigenvalues in descending order;
      * a step is Adam in the basis the step began with, rotated back: the parameters move by exactly that update, the second
        moment is the one Adam leaves, the factors are the lerp of the old ones with G G^T and G^T G;
      * a refreshed basis is orthonormal, it is the QR factor of (factor x old basis) with its columns sorted by the estimates
        diag(Q^T GG Q) - checked as: new_basis^T (GG Q)[sorted] is upper triangular, up to exchanges of neighbouring columns
        whose sort keys fp32 cannot tell apart - it diagonalises the factor no worse than the old one, and exp_avg is the
        momentum of the step rotated from the old basis into the new one."""
    from heavyball_amd.optim import beta_debias, f32

    shapes = [(2048, 2048), (2048, 8192), (8192, 2048)]
    free, _ = torch.cuda.mem_get_info(DEV)
    if free < 40 * 2**30:
        pytest.skip("needs 40 GiB of device memory")
    host, params = H.make_params(shapes, DEV)
    lr, wd, b1, b2, sb, eps = 3e-3, 0.01, 0.9, 0.95, 0.95, 1e-8
    opt = heavyball_amd.SOAP(params, lr=lr, betas=(b1, b2), shampoo_beta=sb, eps=eps, weight_decay=wd, precondition_frequency=2,
                             max_precond_dim=8192)  # fmt: skip
    KM, KV, KQ, KGG = "scale_by_soap_exp_avg_2", "scale_by_soap_exp_avg_sq_2", "scale_by_soap_Q_3", "scale_by_soap_GG_3"

    def rel(a, b):
        return ((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-300)).item()

    def orthonormal(q):
        qd = q.double()
        return (qd.T @ qd - torch.eye(qd.shape[0], dtype=torch.float64, device=DEV)).abs().max().item()

    fired = []
    for k in (1, 2, 3):
        print("case step", k, flush=True)
        grads = [g.to(DEV) for g in H.make_grads(shapes, k, torch.float32, 1e-2)]
        before = []
        for p in params:
            st = opt.state[p][0] if p in opt.state and KM in opt.state[p].get(0, {}) else None
            before.append(None if st is None else dict(p=p.detach().clone(), m=st[KM][0].clone(), v=st[KV][0].clone(),
                                                       Q=[q[0].clone() for q in st[KQ]], GG=[m[0].clone() for m in st[KGG]]))  # fmt: skip
        for p, g in zip(params, grads):
            p.grad = g
        opt.step()
        torch.cuda.synchronize()
        fired.append(bool(opt.param_groups[0]["is_preconditioning"]))
        for i, (p, g) in enumerate(zip(params, grads)):
            st = opt.state[p][0]
            G = g.double()
            if k == 1:
                assert torch.equal(p.detach().cpu(), host[i])  # the first step only initialises
                for li, (q, gg) in enumerate(zip(st[KQ], st[KGG])):
                    want = G @ G.T if li == 0 else G.T @ G  # beta = 0 at initialisation: the factor is the product itself
                    assert rel(gg[0], want) < 1e-5, (i, li)
                    assert orthonormal(q[0]) < 1e-4
                    lam = q[0].double().T @ gg[0].double() @ q[0].double()
                    top = lam.diagonal().max().item()
                    assert (lam - torch.diag(lam.diagonal())).abs().max().item() < 1e-4 * top, (i, li)
                    assert (lam.diagonal()[1:] - lam.diagonal()[:-1]).max().item() < 1e-4 * top, (i, li)
                continue
            b = before[i]
            Ql, Qr = b["Q"][0].double(), b["Q"][1].double()
            step = torch.tensor(k, dtype=torch.int64)
            d1, d2 = float(beta_debias(f32(b1), step - 1)), float(beta_debias(f32(b2), step - 1))  # heavyball/chainable.py:1270
            gp = Ql.T @ G @ Qr
            m_new = b["m"].double() * d1 + gp * (1 - d1)
            v_new = b["v"].double() * d2 + gp * gp * (1 - d2)
            precond = m_new / v_new.sqrt().clamp(min=eps)
            update = Ql @ precond @ Qr.T
            want_p = b["p"].double() * (1 - wd * lr) - lr * update
            moved, want_moved = p.detach().double() - b["p"].double(), want_p - b["p"].double()
            assert rel(moved, want_moved) < 2e-3, (k, i, rel(moved, want_moved))
            assert rel(st[KV][0], v_new) < 1e-4, (k, i)
            a = 1 - float(beta_debias(sb, step))  # heavyball/chainable.py:1244
            for li, gg in enumerate(st[KGG]):
                outer = G @ G.T if li == 0 else G.T @ G
                assert rel(gg[0], b["GG"][li].double() * (1 - a) + outer * a) < 1e-5, (k, i, li)
            if not fired[-1]:
                assert rel(st[KM][0], m_new) < 1e-4, (k, i)
                for li, q in enumerate(st[KQ]):
                    assert torch.equal(q[0], b["Q"][li])
                continue
            new_q = [q[0].double() for q in st[KQ]]
            for li, qn in enumerate(new_q):
                assert orthonormal(st[KQ][li][0]) < 1e-4, (k, i, li)
                old = b["Q"][li].double()
                tmp = st[KGG][li][0].double() @ old
                order = torch.argsort((old * tmp).sum(0), descending=True)
                # upper triangular if qn[:, order] is the QR factor of tmp[:, order].  Thousands of sort keys lie closer together
                # than fp32 products resolve, so the optimizer's order is this float64 order up to exchanges among neighbours:
                # the triangle is asked for outside a band of 64 columns, and inside the band only to the size of the
                # neighbouring diagonal entries
                r = qn[:, order].T @ tmp[:, order]
                scale = r.diagonal().abs().max().item()
                assert r.tril(-64).abs().max().item() < 1e-4 * scale, (k, i, li, r.tril(-64).abs().max().item() / scale)
                assert r.tril(-1).abs().max().item() < 2e-2 * scale, (k, i, li, r.tril(-1).abs().max().item() / scale)
                # and one step of power iteration cannot make the basis diagonalise its factor worse
                def off_mass(q):
                    lam = q.T @ st[KGG][li][0].double() @ q
                    return (lam - torch.diag(lam.diagonal())).norm().item()
                assert off_mass(qn) <= off_mass(old) * 1.001, (k, i, li)
            want_m = new_q[0].T @ (Ql @ m_new @ Qr.T) @ new_q[1]  # heavyball/utils.py:877-884
            assert rel(st[KM][0], want_m) < 2e-3, (k, i, rel(st[KM][0], want_m))
    assert fired == [False, True, False]
