"""Philox4x32-10 in numpy (test infrastructure; see oracle/__init__.py).

The reference draws its rounding noise from torch's global generator
(heavyball/utils.py:1316 ``rand_like``, :2352 ``randint_like``) in a
data-dependent order that a GPU kernel cannot reproduce.  The kernels instead
use the counter-based generator of Salmon et al., "Parallel random numbers: as
easy as 1, 2, 3" (SC'11), Philox4x32 with 10 rounds, keyed so that any element's
noise is a pure function of (seed, step, stream, flat element index).  This file
is the CPU statement of that layout:

    quartet q = flat_index >> 2            (4 consecutive elements, for the two streams 2p and 2p + 1 of a
                                            stream pair p, share one call)
    counter = (q & 0xffffffff, q >> 32, step & 0xffffffff, stream >> 1)
    key     = (seed & 0xffffffff, seed >> 32)
    element j = flat_index & 3 of stream s takes 16 bits: word (s & 1) * 2 + (j >> 1), low half if j even else
    high half

exp_avg (stream 2) and exp_avg_sq (stream 3) form a pair, so a lane that owns a quartet of the slab makes one call
for both moments.

Known-answer vectors from the Random123 distribution (kat_vectors) are checked
in tests/test_oracle_philox.py.
"""

import numpy as np

_M0 = np.uint64(0xD2511F53)
_M1 = np.uint64(0xCD9E8D57)
_W0 = 0x9E3779B9
_W1 = 0xBB67AE85
_MASK = np.uint64(0xFFFFFFFF)
_S32 = np.uint64(32)

# stream ids: which rounding site inside the step consumes the numbers
STREAM_MARS_SR = 0  # bf16 stochastic rounding of the MARS-corrected gradient
STREAM_PARAM = 1  # ECC / SR write of the parameter (shares its calls with STREAM_MARS_SR)
STREAM_EXP_AVG = 2  # ECC / SR write of exp_avg
STREAM_EXP_AVG_SQ = 3  # ECC / SR write of exp_avg_sq (shares its calls with STREAM_EXP_AVG)
STREAM_OLD_GRAD = 4  # ECC / SR write of mars_old_grad
STREAM_INIT_PARAM = 5  # param::ecc initial correction at construction
STREAM_NS_INPUT = 6  # bf16 stochastic rounding of the Newton-Schulz input (the legacy variant also uses 7)
STREAM_CLIP = 8  # bf16 stochastic rounding of a clipped bf16 gradient
STREAM_EXP_AVG_SLOW = 9  # ECC / SR write of AdEMAMix's slow momentum
STREAM_UPDATE = 10  # rounding of an un-fused transform's update into a 16-bit update buffer (update clipping)
STREAM_SOAP_ROTATE = 11  # ECC / SR write of SOAP's exp_avg after its rotation into a refreshed eigenbasis
STREAM_UPDATE_CLIP = 12  # bf16 stochastic rounding of a clipped bf16 update (independent of STREAM_CLIP, the gradient clip's)
STREAM_SOAP_GG = 16  # SR write of a SOAP factor kept in bf16 (16-bit gradients): 16 + 2 * side
STREAM_SOAP_Q = 17  # SR write of a refreshed SOAP eigenbasis kept in bf16: 17 + 2 * side


def philox4x32_10(c0, c1, c2, c3, k0, k1):
    """Vectorised Philox4x32-10.  Counters are uint64 arrays holding 32-bit values; keys are ints."""
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint64) & _MASK for c in (c0, c1, c2, c3))
    k0 = int(k0) & 0xFFFFFFFF
    k1 = int(k1) & 0xFFFFFFFF
    for _ in range(10):
        p0 = _M0 * c0
        p1 = _M1 * c2
        hi0, lo0 = p0 >> _S32, p0 & _MASK
        hi1, lo1 = p1 >> _S32, p1 & _MASK
        c0, c1, c2, c3 = hi1 ^ c1 ^ np.uint64(k0), lo1, hi0 ^ c3 ^ np.uint64(k1), lo0
        k0 = (k0 + _W0) & 0xFFFFFFFF
        k1 = (k1 + _W1) & 0xFFFFFFFF
    return c0, c1, c2, c3


def bits16(seed: int, step: int, stream: int, flat_index) -> np.ndarray:
    """16 random bits per element, int64 array with values in [0, 65536).

    ``flat_index`` is the element's index in the flat slab (tensor base offset +
    index inside the tensor), any integer array.
    """
    f = np.asarray(flat_index, dtype=np.uint64)
    q = f >> np.uint64(2)
    j = (f & np.uint64(3)).astype(np.int64)
    stream = int(stream) & 0xFFFFFFFF
    out = philox4x32_10(
        q & _MASK,
        q >> _S32,
        np.full_like(q, int(step) & 0xFFFFFFFF),
        np.full_like(q, stream >> 1),
        int(seed) & 0xFFFFFFFF,
        (int(seed) >> 32) & 0xFFFFFFFF,
    )
    words = np.stack(out, axis=-1)  # [..., 4]
    w = np.take_along_axis(words, ((stream & 1) * 2 + (j >> 1))[..., None].astype(np.int64), axis=-1)[..., 0]
    shift = ((j & 1) * 16).astype(np.uint64)
    return ((w >> shift) & np.uint64(0xFFFF)).astype(np.int64)
