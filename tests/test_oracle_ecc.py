"""ECC codec / stochastic rounding oracle: golden vectors from the reference, the reference tests' invariants
(test/test_ecc.py:66-107, test/test_stochastic_utils_cpu.py:34-42, test/test_utils_cpu.py:262-286), an exhaustive
sweep over every bf16 bit pattern, and Philox known-answer vectors."""

import os

import numpy as np
import pytest
import torch

from oracle import ecc, philox
from oracle.rounding import HalfRounding, PhiloxRounding

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")


def test_philox_known_answers():
    """Random123 kat_vectors for philox4x32-10."""
    kat = [
        ((0, 0, 0, 0), (0, 0), (0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8)),
        ((0xFFFFFFFF,) * 4, (0xFFFFFFFF,) * 2, (0x408F276D, 0x41C83B0E, 0xA20BC7C6, 0x6D5451FD)),
        ((0x243F6A88, 0x85A308D3, 0x13198A2E, 0x03707344), (0xA4093822, 0x299F31D0), (0xD16CFE09, 0x94FDCCEB, 0x5001E420, 0x24126EA1)),
    ]  # fmt: skip
    for ctr, key, want in kat:
        got = tuple(int(x) for x in philox.philox4x32_10(*ctr, *key))
        assert got == want


def test_philox_layout():
    """four consecutive elements and the two streams of a pair share one call: stream 2p takes words 0 and 1, stream
    2p + 1 words 2 and 3; element j takes half-word j of its stream's two words."""
    seed, step = 0x1234_5678_9ABC_DEF0, 7
    idx = np.arange(4 * 5, 4 * 5 + 4)
    w = [int(x) for x in philox.philox4x32_10(5, 0, step, 1, seed & 0xFFFFFFFF, seed >> 32)]
    assert philox.bits16(seed, step, 2, idx).tolist() == [w[0] & 0xFFFF, w[0] >> 16, w[1] & 0xFFFF, w[1] >> 16]
    assert philox.bits16(seed, step, 3, idx).tolist() == [w[2] & 0xFFFF, w[2] >> 16, w[3] & 0xFFFF, w[3] >> 16]
    # another pair is another counter word, not another half of the same call
    w4 = [int(x) for x in philox.philox4x32_10(5, 0, step, 2, seed & 0xFFFFFFFF, seed >> 32)]
    assert philox.bits16(seed, step, 4, idx).tolist() == [w4[0] & 0xFFFF, w4[0] >> 16, w4[1] & 0xFFFF, w4[1] >> 16]
    # high counter word
    big = np.array([(1 << 34) + 3], dtype=np.uint64)
    w = philox.philox4x32_10(0, 1, step, 1, seed & 0xFFFFFFFF, seed >> 32)
    assert philox.bits16(seed, step, 3, big)[0] == (int(w[3]) >> 16)


@pytest.mark.parametrize("mode", list(ecc.MODES))
def test_codec_matches_reference_vectors(mode):
    d = torch.load(os.path.join(GOLDEN, "ecc.pt"), weights_only=True)
    x, u = d["x"], d["u"]
    pd, cd = ecc.MODES[mode]
    e = ecc.EccTensor(torch.zeros(x.shape, dtype=pd), torch.zeros(x.shape, dtype=cd))
    e.encode(x, u)
    assert torch.equal(e.primary.view(torch.int16), d[f"{mode}/primary"].view(torch.int16))
    assert torch.equal(e.corr, d[f"{mode}/corr"])
    assert torch.equal(e.decode().view(torch.int32), d[f"{mode}/decoded"].view(torch.int32))
    assert torch.equal(ecc.log_ulp(e.primary), d[f"{mode}/log_ulp"])


def test_stochastic_round_matches_reference_vectors():
    d = torch.load(os.path.join(GOLDEN, "ecc.pt"), weights_only=True)
    out = ecc.stochastic_round(d["x"], d["sr/noise"])
    assert torch.equal(out.view(torch.int16), d["sr/out"].view(torch.int16))


@pytest.mark.parametrize("mode", list(ecc.MODES))
def test_roundtrip_invariants(mode):
    """test/test_ecc.py:66-82: error <= 2^log_ulp / (2 smax), improvement > 100x (int8) / 10^4x (int16)."""
    pd, cd = ecc.MODES[mode]
    torch.manual_seed(42)
    x = torch.randn(4096)
    e = ecc.EccTensor(x.to(pd), torch.zeros(4096, dtype=cd))
    e.compute_correction(x, torch.rand(4096))
    out = e.decode()
    err, naive = (x - out).abs(), (x - e.primary.float()).abs()
    assert naive.max().item() / max(err.max().item(), 1e-45) > (100 if cd == torch.int8 else 10000)
    bound = torch.exp2(ecc.log_ulp(e.primary).float()) / (2 * e.smax)
    assert (err <= bound + 1e-10).all()
    assert e.corr.abs().max() <= e.smax


def test_boundary_values():
    """test/test_ecc.py:85-94."""
    for vals in [torch.zeros(256), torch.tensor([1e4, -1e4, 3e10, -3e10, 1e-10, -1e-10])]:
        e = ecc.EccTensor(vals.to(torch.bfloat16), torch.zeros(vals.shape, dtype=torch.int8))
        e.compute_correction(vals, torch.rand(vals.shape))
        bound = torch.exp2(ecc.log_ulp(e.primary).float()) / (2 * 127.0)
        assert ((vals - e.decode()).abs() <= bound + 1e-10).all()


def test_exhaustive_bf16_patterns():
    """every finite bf16 primary x a spread of fp32 values in its rounding interval: decode(encode(x)) stays inside
    one correction unit, the primary is the round-to-nearest-even bf16, and corrections stay in [-127, 127]."""
    bits = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16)
    prim = bits.view(torch.bfloat16)
    finite = torch.isfinite(prim.float())
    base = (bits.to(torch.int32) << 16)[finite]
    for low in (0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1234, 0xABCD):
        x = (base | low).view(torch.float32)
        x = x[torch.isfinite(x)]
        e = ecc.EccTensor.zeros(x.shape, "bf16+8")
        e.encode(x, torch.full(x.shape, 0.5))
        assert torch.equal(e.primary.view(torch.int16), x.to(torch.bfloat16).view(torch.int16))
        assert e.corr.abs().max() <= 127
        ok = torch.isfinite(e.primary.float())
        unit = torch.exp2(ecc.log_ulp(e.primary).float() - 1) / 127.0
        assert ((x - e.decode()).abs()[ok] <= unit[ok] * (1 + 1e-6)).all()


def test_sr_bracket_and_unbiased():
    """test/test_stochastic_utils_cpu.py:34-42: result is one of the two neighbouring bf16 values; the mean over many
    draws approaches the source (here with the Philox stream the kernels use)."""
    gen = torch.Generator().manual_seed(0x5566AA)
    x = torch.randn(2048, generator=gen) * 3
    lo = (x.view(torch.int32) & -65536).view(torch.float32)
    hi = ((x.view(torch.int32) & -65536) + 65536).view(torch.float32)
    acc = torch.zeros_like(x)
    trials = 256
    for t in range(trials):
        r = PhiloxRounding(seed=99, step=t)
        out = ecc.stochastic_round(x, r.noise16(0, 0, x.shape)).float()
        assert ((out == lo) | (out == hi)).all()
        acc += out
    err = (acc / trials - x).abs()
    assert err.mean() < 5e-3 and err.max() < 2.5e-2


def test_sr_accumulation_beats_rne():
    """test/test_utils_cpu.py:262-286: 2048 increments of 1e-3 onto a bf16 accumulator."""
    acc_sr = torch.zeros(64, dtype=torch.bfloat16)
    acc_rne = torch.zeros(64, dtype=torch.bfloat16)
    for t in range(2048):
        r = PhiloxRounding(seed=5, step=t)
        acc_sr.copy_(ecc.stochastic_round(acc_sr.float() + 1e-3, r.noise16(0, 0, (64,))))
        acc_rne.copy_((acc_rne.float() + 1e-3).bfloat16())
    assert (acc_sr.float().mean() - 2.048).abs() < 0.2
    assert (acc_rne.float().mean() - 2.048).abs() > 1.0


def test_half_rounding_is_round_half_up_on_magnitude():
    x = torch.tensor([1.0 + 2**-8, 1.0 + 2**-9, -(1.0 + 2**-8), 1.0 + 3 * 2**-9])
    out = ecc.stochastic_round(x, HalfRounding().noise16(0, 0, x.shape)).float()
    assert out.tolist() == [1.0 + 2**-7, 1.0, -(1.0 + 2**-7), 1.0 + 2**-7]


def test_ecc_uniform16_is_exactly_unbiased_for_bf16_int8():
    """scaled = 127 k / 2^15 has at most 15 fractional bits, so a uniform on the grid j / 2^16 rounds up with
    probability exactly frac(scaled): summing floor(scaled + j/65536) over all j gives 65536*floor + 65536*frac."""
    x = torch.tensor([1.0 + 37 * 2**-23, 1.0 + 12345 * 2**-23, -(1.0 + 30001 * 2**-23)])
    narrow = x.to(torch.bfloat16)
    e = x - narrow.float()
    ls = (ecc.log_ulp(narrow) - 1).float()
    scaled = (ecc.scale_by_exp2(e, -ls).clamp(-1, 1) * 127.0).double()
    j = torch.arange(65536, dtype=torch.float32) / 65536.0
    total = (scaled.float()[:, None] + j[None, :]).floor().double().sum(1)
    assert torch.allclose(total / 65536.0, scaled, rtol=0, atol=1e-12)
