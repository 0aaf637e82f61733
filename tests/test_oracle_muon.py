"""Muon oracle: golden vectors written from the reference (Newton-Schulz is untested in the reference itself), the
polar-factor invariant, transpose symmetry, and the golden Muon trajectories."""

import glob
import json
import os

import pytest

from oracle.ecc import EccTensor
import torch

from oracle import muon
from oracle.rounding import HalfRounding

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def rel_fro(a, b):
    return ((a.double() - b.double()).norm() / b.double().norm()).item()


@pytest.mark.parametrize("name", ["sq", "wide", "tall", "sq64"])
def test_newton_schulz_matches_reference_vectors(name):
    d = torch.load(os.path.join(GOLDEN, "ns5.pt"), weights_only=True)
    G = d[f"{name}/G"]
    half = torch.full(G.shape, 1 << 15, dtype=torch.int32)
    out = muon.newton_schulz5(G.clone(), half)
    assert rel_fro(out, d[f"{name}/ns5"]) < 1e-2  # same ATen op as the reference; its blocking may differ between CPU models
    if f"{name}/legacy" in d:
        out = muon.legacy_newton_schulz5(G.clone(), half, half)
        assert rel_fro(out, d[f"{name}/legacy"]) < 1e-2
    out = muon.orthogonal(G.clone(), HalfRounding(), 0)
    assert rel_fro(out, d[f"{name}/orthogonal_scaled"]) < 1e-2


@pytest.mark.parametrize("name", ["sq", "wide", "tall", "sq64"])
def test_newton_schulz_on_bf16_inputs_matches_reference_vectors(name):
    """A bf16 update buffer: the norm and the normalised input are bf16 values, the input's stochastic round is the identity; the
    legacy variant divides in fp32 and rounds that quotient stochastically (heavyball/utils.py:555-556, :641-645, :1174-1179)."""
    d = torch.load(os.path.join(GOLDEN, "ns5_bf16.pt"), weights_only=True)
    G = d[f"{name}/G"]
    assert G.dtype == torch.bfloat16
    half = torch.full(G.shape, 1 << 15, dtype=torch.int32)
    out = muon.newton_schulz5(G.clone(), half)
    assert out.dtype == torch.bfloat16 and rel_fro(out, d[f"{name}/ns5"]) < 1e-2
    if f"{name}/legacy" in d:
        out = muon.legacy_newton_schulz5(G.clone(), half, half)
        assert out.dtype == torch.bfloat16 and rel_fro(out, d[f"{name}/legacy"]) < 1e-2


@pytest.mark.parametrize("name", ["sq", "wide", "tall", "sq64"])
def test_newton_schulz_on_fp16_inputs_matches_reference_vectors(name):
    """A float16 update buffer: the norm and the quotient are float16 values, the quotient is rounded to bf16 like an fp32 one, the
    result goes back to float16 and is scaled there (heavyball/utils.py:555-556, :577, :808-809).  The matrices up to 32 wide
    are compared for equality (a bf16 product that small is summed in one order by any blocking, so the oracle's arithmetic is
    the reference's to the bit: a float16 rounding left out anywhere would show); the 64-wide one to the Newton-Schulz tolerance."""
    d = torch.load(os.path.join(GOLDEN, "ns5_fp16.pt"), weights_only=True)
    G = d[f"{name}/G"]
    assert G.dtype == torch.float16
    same = torch.equal if max(G.shape) <= 32 else (lambda a, b: rel_fro(a, b) < 1e-2)
    half = torch.full(G.shape, 1 << 15, dtype=torch.int32)
    out = muon.newton_schulz5(G.clone(), half)
    assert out.dtype == torch.float16 and same(out, d[f"{name}/ns5"])
    if f"{name}/legacy" in d:
        out = muon.legacy_newton_schulz5(G.clone(), half, half)
        assert out.dtype == torch.float16 and same(out, d[f"{name}/legacy"])
    out = muon.orthogonal(G.clone(), HalfRounding(), 0)
    assert out.dtype == torch.float16 and same(out, d[f"{name}/orthogonal_scaled"])


@pytest.mark.parametrize("name", ["sq", "sq64", "sq96", "sq64_bf16", "sq64_fp16"])
def test_polar_express_matches_reference_vectors(name):
    """msign(x, 10), what square matrices take under zeroth_power_mode = "thinky_polar_express" (heavyball/utils.py:605-631,
    :796-797), on fp32, bf16 and float16 inputs; and the schedule does what it is for: the singular values end near 1."""
    d = torch.load(os.path.join(GOLDEN, "msign.pt"), weights_only=True)
    G = d[f"{name}/G"]
    half = torch.full(G.shape, 1 << 15, dtype=torch.int32)
    out = muon.polar_express(G.clone(), half)
    assert out.dtype == G.dtype and rel_fro(out, d[f"{name}/msign"]) < 1e-2
    sv = torch.linalg.svdvals(out.double())
    assert sv.max() < 1.2 and sv.median() > 0.8
    assert len(muon.POLAR_COEFFS) == 10 and muon.POLAR_COEFFS[7] == muon.POLAR_COEFFS[9] == (1.875, -1.25, 0.375)


def test_polar_factor_invariant():
    """The per-iteration schedule drives every singular value towards 1: the result is close to U V^T of the SVD and
    its singular values lie in a band around 1 (a wrong coefficient, sign or a transposed operand leaves them far off)."""
    gen = torch.Generator().manual_seed(0)
    for shape in [(64, 64), (32, 96), (96, 32)]:
        # a well-conditioned input: prescribed singular values in [0.2, 1] (a square Gaussian matrix has one near 0,
        # which five iterations cannot lift)
        k = min(shape)
        u, _ = torch.linalg.qr(torch.randn(shape[0], k, generator=gen, dtype=torch.float64))
        v, _ = torch.linalg.qr(torch.randn(shape[1], k, generator=gen, dtype=torch.float64))
        sv_in = torch.linspace(0.2, 1.0, k, dtype=torch.float64)
        G = ((u * sv_in) @ v.T).float()
        out = muon.newton_schulz5(G, torch.full(shape, 1 << 15, dtype=torch.int32))
        sv = torch.linalg.svdvals(out.double())
        assert sv.max() < 1.3 and sv.min() > 0.6, (shape, sv.min().item(), sv.max().item())
        assert rel_fro(out, u @ v.T) < 0.2


def test_transpose_symmetry_and_scale():
    gen = torch.Generator().manual_seed(1)
    G = torch.randn(24, 72, generator=gen)
    half = torch.full(G.shape, 1 << 15, dtype=torch.int32)
    a = muon.newton_schulz5(G, half)
    b = muon.newton_schulz5(G.T.contiguous(), half.T.contiguous())
    assert torch.equal(a, b.T)
    wide = muon.orthogonal(G.clone(), HalfRounding(), 0)
    tall = muon.orthogonal(G.T.contiguous(), HalfRounding(), 0)
    assert torch.equal(wide, a)  # rows < cols: scale 1
    assert torch.allclose(tall, b * (72 / 24) ** 0.5)


def _assert_matrix_step(d, k, i, got, want):
    """The step a matrix took, lr * NS(..), to the Newton-Schulz tolerance; a parameter kept as an ECC pair is decoded first
    (its resolution, 2^-8 / smax of a bf16 ulp, is far below that tolerance)."""

    def full(t, key):
        return EccTensor(t, d[key]).decode() if key in d else t.float()

    prev = full(d[f"step{k - 1}/p{i}"], f"step{k - 1}/state{i}/param::ecc") if k > 1 else d[f"init/p{i}"]
    want = full(want, f"step{k}/state{i}/param::ecc")
    got = got.decode() if isinstance(got, EccTensor) else got
    if k == 1 and f"step1/state{i}/param::ecc" in d:
        return  # the fixture holds no correction for the narrowed initial parameter: the first step has no reference point
    assert rel_fro(got - prev, want - prev) < 2e-2, (k, i, rel_fro(got - prev, want - prev))


TRAJ = sorted(glob.glob(os.path.join(GOLDEN, "traj_muon_*.pt")))


@pytest.mark.parametrize("path", TRAJ, ids=[os.path.basename(p)[5:-3] for p in TRAJ])
def test_muon_trajectory_matches_reference(path):
    d = torch.load(path, weights_only=True)
    kwargs = json.loads(d["meta/kwargs"])
    if "betas" in kwargs:
        kwargs["betas"] = tuple(kwargs["betas"])
    n = len([k for k in d if k.startswith("init/p")])
    orc = muon.MuonOracle([d[f"init/p{i}"].clone() for i in range(n)], rounding=HalfRounding(),
                          mode=d.get("meta/zeroth_power_mode", "newtonschulz"), **kwargs)
    for k in range(1, d["meta/steps"] + 1):
        orc.step([d[f"step{k}/g{i}"].clone() for i in range(n)])
        for i in range(n):
            prefix = f"step{k}/state{i}/"
            want_state = {kk[len(prefix):]: d[kk] for kk in d if kk.startswith(prefix) and not kk.endswith("/step")}
            assert set(want_state) == set(orc.state[i]), (i, set(want_state), set(orc.state[i]))
            want, got = d[f"step{k}/p{i}"], orc.params[i]
            for kk, vv in want_state.items():
                if kk == "param::ecc" and want.dim() >= 2:
                    continue  # a matrix moves by lr * NS(..), compared below to the Newton-Schulz tolerance
                assert torch.equal(orc.state[i][kk], vv), (k, i, kk)  # elementwise fp32: exact
            if want.dim() < 2:
                assert torch.equal(got.primary if isinstance(got, EccTensor) else got, want)
            else:
                _assert_matrix_step(d, k, i, got, want)


TRAJ_MA = sorted(glob.glob(os.path.join(GOLDEN, "traj_muonadamw_*.pt")))


@pytest.mark.parametrize("path", TRAJ_MA, ids=[os.path.basename(p)[5:-3] for p in TRAJ_MA])
def test_muonadamw_trajectory_matches_reference(path):
    """Matrices: momentum exact, step within the Newton-Schulz tolerance.  Vectors (scale_by_adam + update_param_): the
    reference's CPU square root is not correctly rounded, so fp32 agrees to 8 ulps."""
    from tests import helpers as H

    d = torch.load(path, weights_only=True)
    kwargs = json.loads(d["meta/kwargs"])
    if "betas" in kwargs:
        kwargs["betas"] = tuple(kwargs["betas"])
    n = len([k for k in d if k.startswith("init/p")])
    orc = muon.MuonAdamWOracle([d[f"init/p{i}"].clone() for i in range(n)], rounding=HalfRounding(), **kwargs)
    for k in range(1, d["meta/steps"] + 1):
        orc.step([d[f"step{k}/g{i}"].clone() for i in range(n)])
        for i in range(n):
            prefix = f"step{k}/state{i}/"
            want_state = {kk[len(prefix):]: d[kk] for kk in d if kk.startswith(prefix) and not kk.endswith("/step")}
            assert set(want_state) == set(kk for kk in orc.state[i] if kk != "step"), (i, set(want_state), set(orc.state[i]))
            want, got = d[f"step{k}/p{i}"], orc.params[i]
            if want.dim() < 2:
                got_p = got.primary if isinstance(got, EccTensor) else got
                H.assert_close_to_reference({"param": got_p, **orc.state[i]}, {"param": want, **want_state}, f"step {k} vector {i}")
            else:
                for kk, vv in want_state.items():
                    if kk != "param::ecc":
                        assert torch.equal(orc.state[i][kk], vv), (k, i, kk)
                _assert_matrix_step(d, k, i, got, want)
