"""GPU parity of the ECC codec, bf16 stochastic rounding and the Philox stream, called through the C ABI and compared
bit for bit with the CPU oracle and with the vectors recorded from the reference (tests/golden/ecc.pt)."""

import os

import numpy as np
import pytest
import torch

from heavyball_amd import _lib
from oracle import ecc, philox

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
DEV = "cuda:0"


def _encode(x, mode, rng_mode, seed=0, step=0, stream=2, base=0):
    L = _lib.lib()
    pd, cd = ecc.MODES[mode]
    xd = x.to(DEV).contiguous()
    prim = torch.zeros(x.shape, dtype=pd, device=DEV)
    corr = torch.zeros(x.shape, dtype=cd, device=DEV)
    _lib.check(L.hb_ecc_encode(xd.data_ptr(), prim.data_ptr(), corr.data_ptr(), x.numel(), _lib.ECC_FMT[mode], rng_mode, seed, step, stream, base, None))
    torch.cuda.synchronize()
    return prim, corr


def _decode(prim, corr, mode):
    L = _lib.lib()
    out = torch.empty(prim.shape, dtype=torch.float32, device=DEV)
    _lib.check(L.hb_ecc_decode(prim.data_ptr(), corr.data_ptr(), out.data_ptr(), prim.numel(), _lib.ECC_FMT[mode], None))
    torch.cuda.synchronize()
    return out.cpu()


def test_philox_words_match_numpy():
    L = _lib.lib()
    n, q0, seed, step, stream = 1000, (1 << 33) - 500, 0xDEADBEEF12345678, 42, 3
    out = torch.zeros(4 * n, dtype=torch.int32, device=DEV)
    _lib.check(L.hb_philox_words(out.data_ptr(), n, q0, seed, step, stream, None))
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint32).reshape(n, 4)
    q = np.arange(q0, q0 + n, dtype=np.uint64)
    want = np.stack(
        philox.philox4x32_10(q & np.uint64(0xFFFFFFFF), q >> np.uint64(32), np.full_like(q, step), np.full_like(q, stream), seed & 0xFFFFFFFF, seed >> 32),
        axis=-1,
    ).astype(np.uint32)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("mode", list(ecc.MODES))
def test_decode_matches_reference_vectors(mode):
    d = torch.load(os.path.join(GOLDEN, "ecc.pt"), weights_only=True)
    out = _decode(d[f"{mode}/primary"].to(DEV), d[f"{mode}/corr"].to(DEV), mode)
    assert torch.equal(out.view(torch.int32), d[f"{mode}/decoded"].view(torch.int32))


@pytest.mark.parametrize("mode", list(ecc.MODES))
def test_encode_half_and_philox_match_oracle(mode):
    d = torch.load(os.path.join(GOLDEN, "ecc.pt"), weights_only=True)
    gen = torch.Generator().manual_seed(7)
    x = torch.cat([d["x"], torch.randn(100_003, generator=gen) * torch.exp(torch.randn(100_003, generator=gen) * 4),
                   # second moments of small gradients: below the smallest normal fp16 value, where the residual against an fp16
                   # primary keeps up to 24 significant bits and the correction depends on every rounding of the reference's sequence
                   torch.randn(400_000, generator=gen).square() * 1e-6, torch.randn(100_000, generator=gen) * 3e-8])
    if mode.startswith("fp16"):
        x = x.clamp(-6e4, 6e4)
    for rng_mode, base in ((_lib.RNG_HALF, 0), (_lib.RNG_PHILOX, 8 * 12345 + 3)):
        prim, corr = _encode(x, mode, rng_mode, seed=99, step=5, stream=2, base=base)
        e = ecc.EccTensor.zeros(x.shape, mode)
        if rng_mode == _lib.RNG_HALF:
            u = torch.full(x.shape, 0.5)
        else:
            b = philox.bits16(99, 5, 2, np.arange(base, base + x.numel(), dtype=np.uint64))
            u = torch.from_numpy(b.astype(np.float32)) / 65536.0
        e.encode(x, u)
        assert torch.equal(prim.cpu().view(torch.int16), e.primary.view(torch.int16))
        assert torch.equal(corr.cpu(), e.corr), f"{(corr.cpu() != e.corr).sum().item()} corrections differ"
        assert torch.equal(_decode(prim, corr, mode).view(torch.int32), e.decode().view(torch.int32))


@pytest.mark.parametrize("mode", ["bf16+8", "bf16+16", "fp16+8", "fp16+16"])
def test_encode_of_overflowing_and_non_finite_values_matches_oracle(mode):
    """Values beyond the primary's range (1e5 in fp16), infinities and NaN: the primary overflows to infinity, and the
    correction follows torch's arithmetic (clamp keeps a NaN, the conversion to the integer type makes it 0; a finite value
    under an infinite primary gives -smax or +smax).  ADOPT's momentum, which divides by a root that can be 1e-8, gets
    there on fp16 primaries."""
    x = torch.tensor([float("inf"), float("-inf"), float("nan"), 1e5, -1e5, 65519.9, 65520.0, -65520.0, 3.4e38, -3.4e38, 3.3e38,
                      1e-45, -1e-45, 0.0, -0.0, 1.0, 6e4] * 3)  # fmt: skip
    for rng_mode in (_lib.RNG_HALF, _lib.RNG_PHILOX):
        prim, corr = _encode(x, mode, rng_mode, seed=3, step=1, stream=2, base=64)
        e = ecc.EccTensor.zeros(x.shape, mode)
        if rng_mode == _lib.RNG_HALF:
            u = torch.full(x.shape, 0.5)
        else:
            u = torch.from_numpy(philox.bits16(3, 1, 2, np.arange(64, 64 + x.numel(), dtype=np.uint64)).astype(np.float32)) / 65536.0
        e.encode(x, u)
        got_p, want_p = prim.cpu().float(), e.primary.float()
        assert torch.equal(torch.isnan(got_p), torch.isnan(want_p))
        ok = ~torch.isnan(want_p)
        assert torch.equal(prim.cpu()[ok].view(torch.int16), e.primary[ok].view(torch.int16))
        assert torch.equal(corr.cpu(), e.corr), (mode, rng_mode, corr.cpu().tolist(), e.corr.tolist())


def test_exhaustive_bf16_patterns_roundtrip():
    """all 65,536 bf16 primaries x all 255 int8 corrections: GPU decode == oracle decode, bit for bit."""
    bits = torch.arange(-32768, 32768, dtype=torch.int32).to(torch.int16)
    prim = bits.view(torch.bfloat16).repeat_interleave(255)
    corr = torch.arange(-127, 128, dtype=torch.int16).to(torch.int8).repeat(65536)
    got = _decode(prim.to(DEV), corr.to(DEV), "bf16+8")
    want = ecc.EccTensor(prim, corr).decode()
    ok = torch.isfinite(want)
    assert torch.equal(got[ok].view(torch.int32), want[ok].view(torch.int32))
    # encode every fp32 value with a given low half across all bf16 high halves
    base = (bits.to(torch.int32) << 16)
    for low in (0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x1234):
        x = (base | low).view(torch.float32)
        x = x[torch.isfinite(x) & torch.isfinite(x.to(torch.bfloat16).float())]
        p, c = _encode(x, "bf16+8", _lib.RNG_HALF)
        e = ecc.EccTensor.zeros(x.shape, "bf16+8")
        e.encode(x, torch.full(x.shape, 0.5))
        assert torch.equal(p.cpu().view(torch.int16), e.primary.view(torch.int16))
        assert torch.equal(c.cpu(), e.corr)


def test_sr_matches_reference_vectors_and_oracle():
    L = _lib.lib()
    gen = torch.Generator().manual_seed(3)
    x = torch.randn(50_001, generator=gen) * 3
    xd = x.to(DEV)
    out = torch.zeros(x.shape, dtype=torch.bfloat16, device=DEV)
    base = 77
    _lib.check(L.hb_sr_bf16(xd.data_ptr(), out.data_ptr(), x.numel(), _lib.RNG_PHILOX, 11, 3, 0, base, None))
    torch.cuda.synchronize()
    noise = torch.from_numpy(philox.bits16(11, 3, 0, np.arange(base, base + x.numel(), dtype=np.uint64)).astype(np.int32))
    want = ecc.stochastic_round(x, noise)
    assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
    _lib.check(L.hb_sr_bf16(xd.data_ptr(), out.data_ptr(), x.numel(), _lib.RNG_HALF, 0, 0, 0, 0, None))
    torch.cuda.synchronize()
    want = ecc.stochastic_round(x, torch.full(x.shape, 1 << 15, dtype=torch.int32))
    assert torch.equal(out.cpu().view(torch.int16), want.view(torch.int16))
