// Device-side building blocks shared by the gfx950 kernels: Philox4x32-10, the ECC codec, bf16 stochastic
// rounding, octet (8-element) loads/stores and wavefront reductions.  Compiled with -ffp-contract=off: the
// reference's eager ops round after every multiply and add, and so must these.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/hbstep.h"

namespace hb {

constexpr int kWave = 64;
constexpr int kDyn = -1;  // template value: format decided at run time

// ---------------------------------------------------------------------------------------------------------
// bit casts / narrow floats
// ---------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float u2f(uint32_t u) { return __builtin_bit_cast(float, u); }
__device__ __forceinline__ uint32_t f2u(float f) { return __builtin_bit_cast(uint32_t, f); }
__device__ __forceinline__ float bf16_to_f32(uint32_t h) { return u2f(h << 16); }
__device__ __forceinline__ uint32_t f32_to_bf16_rne(float x) {  // v_cvt_pk_bf16_f32 on gfx950
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
}
__device__ __forceinline__ float f16_to_f32(uint32_t h) { return (float)__builtin_bit_cast(_Float16, (uint16_t)h); }
// The empty asm makes x an fp32 value in a register first.  Without it the compiler folds a product or sum that feeds the
// conversion into v_fma_mixlo_f16, which rounds the exact result once; the reference rounds to fp32, then to fp16 (torch computes
// float16 tensors in fp32 and converts), and the two differ where the fp32 rounding lands on a float16 tie.
__device__ __forceinline__ uint32_t f32_to_f16_rne_plain(float x) { return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x); }  // x is no product or sum
__device__ __forceinline__ uint32_t f32_to_f16_rne(float x) {
  asm("" : "+v"(x));
  return f32_to_f16_rne_plain(x);
}

// ---------------------------------------------------------------------------------------------------------
// Philox4x32-10 (Salmon et al., SC'11).  One call yields 128 bits: 16 bits for each of the 4 elements of a quartet
// (4 consecutive elements, flat index a multiple of 4), for the two rounding sites of a stream pair:
//   counter = (q lo, q hi, step, stream >> 1) with q = flat_index >> 2,  key = seed
//   element j = flat_index & 3 of stream s takes word (s & 1) * 2 + (j >> 1), low half if j is even else high half.
// exp_avg (2) and exp_avg_sq (3) share a call, so a lane that owns a quartet needs one call for both moments.
// ---------------------------------------------------------------------------------------------------------
struct Rand8 {  // the four words of one call; also: the noise of an octet for one stream (two calls, see Rng::octet)
  uint32_t w[4];
  // selects instead of an indexed read: with a run-time j an indexed array would live in scratch memory
  __device__ __forceinline__ uint32_t bits16(int j) const {
    const int k = j >> 1;
    const uint32_t x = k == 0 ? w[0] : k == 1 ? w[1] : k == 2 ? w[2] : w[3];
    return (x >> ((j & 1) * 16)) & 0xFFFFu;
  }
};
// noise of E consecutive elements for one stream: 16 bits each, element j in word j >> 1
template <int E>
struct Noise {
  uint32_t w[E / 2];
  __device__ __forceinline__ uint32_t bits16(int j) const { return (w[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu; }
};

__device__ __forceinline__ Rand8 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)M0 * c0;
    uint64_t p1 = (uint64_t)M1 * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += W0;
    k1 += W1;
  }
  return Rand8{{c0, c1, c2, c3}};
}

struct Rng {
  uint32_t seed_lo, seed_hi, step;
  int mode;
  // the call that serves the quartet holding flat index `flat` for the stream pair `pair` (= stream >> 1)
  __device__ __forceinline__ Rand8 call(int64_t flat, uint32_t pair) const {
    const uint64_t q = (uint64_t)flat >> 2;
    return philox4x32_10((uint32_t)q, (uint32_t)(q >> 32), step, pair, seed_lo, seed_hi);
  }
  // noise of the E elements starting at flat index `flat` (a multiple of E; E = 2, 4 or 8) for both streams of a
  // pair: `even` for stream 2 * pair, `odd` for stream 2 * pair + 1
  template <int E>
  __device__ __forceinline__ void noise_pair(int64_t flat, uint32_t pair, Noise<E>& even, Noise<E>& odd) const {
    static_assert(E == 2 || E == 4 || E == 8, "2, 4 or 8 elements per lane");
#pragma unroll
    for (int i = 0; i < E / 2; ++i) even.w[i] = odd.w[i] = 0x80008000u;
    if (mode != HB_RNG_PHILOX) return;
    const Rand8 r = call(flat, pair);
    if constexpr (E == 2) {  // half a quartet: the lanes of both halves make the same call and take their word
      const bool hi = (flat & 2) != 0;
      even.w[0] = hi ? r.w[1] : r.w[0];
      odd.w[0] = hi ? r.w[3] : r.w[2];
    } else {  // written out per quartet: a loop over the quartets is left rolled and indexes the words through scratch
      even.w[0] = r.w[0];
      even.w[1] = r.w[1];
      odd.w[0] = r.w[2];
      odd.w[1] = r.w[3];
      if constexpr (E == 8) {
        const Rand8 r2 = call(flat + 4, pair);
        even.w[2] = r2.w[0];
        even.w[3] = r2.w[1];
        odd.w[2] = r2.w[2];
        odd.w[3] = r2.w[3];
      }
    }
  }
  template <int E>
  __device__ __forceinline__ Noise<E> noise(int64_t flat, uint32_t stream) const {
    static_assert(E == 2 || E == 4 || E == 8, "2, 4 or 8 elements per lane");
    Noise<E> out;
#pragma unroll
    for (int i = 0; i < E / 2; ++i) out.w[i] = 0x80008000u;
    if (mode == HB_RNG_PHILOX) {
      const bool second = (stream & 1) != 0;
      const Rand8 r = call(flat, stream >> 1);
      if constexpr (E == 2) {
        const uint32_t lo = second ? r.w[2] : r.w[0], hi = second ? r.w[3] : r.w[1];
        out.w[0] = (flat & 2) ? hi : lo;
      } else {
        out.w[0] = second ? r.w[2] : r.w[0];
        out.w[1] = second ? r.w[3] : r.w[1];
        if constexpr (E == 8) {
          const Rand8 r2 = call(flat + 4, stream >> 1);
          out.w[2] = second ? r2.w[2] : r2.w[0];
          out.w[3] = second ? r2.w[3] : r2.w[1];
        }
      }
    }
    return out;
  }
  // noise for the octet whose first element has flat slab index `flat` (a multiple of 8), one stream
  __device__ __forceinline__ Rand8 octet(int64_t flat, uint32_t stream) const {
    const Noise<8> n = noise<8>(flat, stream);
    return Rand8{{n.w[0], n.w[1], n.w[2], n.w[3]}};
  }
};

__device__ __forceinline__ float uniform16(uint32_t bits) { return (float)bits * (1.0f / 65536.0f); }

// fp32 -> bf16 by adding 16 noise bits and truncating (heavyball/utils.py:2341-2355, dither_steps = 1)
__device__ __forceinline__ uint32_t sr_bf16(float x, uint32_t noise16) { return (f2u(x) + noise16) >> 16; }

// ---------------------------------------------------------------------------------------------------------
// ECC codec (heavyball/utils.py:1288-1324, :3380-3392)
// ---------------------------------------------------------------------------------------------------------
template <bool PRIM_BF16>
__device__ __forceinline__ int ecc_log_scale(uint32_t h) {  // log_ulp(primary) - 1
  if (PRIM_BF16) {
    int e = (h >> 7) & 0xFF;
    return max(e, 1) - 135;  // bias + mantissa = 134
  } else {
    int e = (h >> 10) & 0x1F;
    return max(e, 1) - 26;  // bias + mantissa = 25
  }
}

template <bool PRIM_BF16>
__device__ __forceinline__ float prim_to_f32(uint32_t h) {
  return PRIM_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}

// corr / smax, correctly rounded: one Newton correction of c * (1/smax) is exact for every int16 value with
// smax = 127 and smax = 32767 (checked exhaustively on the host in tests/test_host_logic.py)
template <bool CORR8>
__device__ __forceinline__ float corr_over_smax(int c) {
  constexpr float smax = CORR8 ? 127.0f : 32767.0f;
  constexpr float r = 1.0f / smax;
  float cf = (float)c;
  float q0 = cf * r;
  float rem = __builtin_fmaf(-q0, smax, cf);
  return __builtin_fmaf(rem, r, q0);
}

template <bool PRIM_BF16, bool CORR8>
__device__ __forceinline__ float ecc_decode(uint32_t h, int c) {
  return prim_to_f32<PRIM_BF16>(h) + ldexpf(corr_over_smax<CORR8>(c), ecc_log_scale<PRIM_BF16>(h));
}

// float -> int with the hardware's saturating conversion (NaN -> 0), never undefined
__device__ __forceinline__ int f2i_sat(float x) {
  int r;
  asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(x));
  return r;
}

// correction of x against its primary h: floor(clamp((x - primary) * 2^-ls, -1, 1) * smax + u), u = noise16 / 65536.
//
// int8 on a bf16 primary: e = x - primary has at most 16 significant bits (also when x or the primary is denormal), so
// scaled = clamp(..) * 127 is exact in fp32 with at most 15 fractional bits, scaled + u is exact as well, and
// floor(scaled + k / 65536) == (scaled * 65536 + k) >> 16 in integers: one multiply, one convert, one add and one shift
// replace convert + multiply + add + floor + convert.
// int16: scaled has up to 31 significant bits before the add, so the reference's fp32 rounding of (scaled + u) matters
// and the float formulation is kept.
template <bool PRIM_BF16, bool CORR8>
__device__ __forceinline__ int ecc_correction(float x, uint32_t h, uint32_t noise16) {
  const float e = x - prim_to_f32<PRIM_BF16>(h);
  const float en = ldexpf(e, -ecc_log_scale<PRIM_BF16>(h));
  // A NaN (x is NaN, or x and its primary are the same infinity) goes through torch's clamp as NaN and becomes
  // correction 0 in the conversion to the integer type; the hardware's min / max would turn it into -1 instead.
  if (CORR8 && PRIM_BF16) {
    // clamp after the (saturating, NaN -> 0) conversion: the same integer for every finite en, since the conversion truncates
    int t = f2i_sat(en * (127.0f * 65536.0f));
    t = t < -127 * 65536 ? -127 * 65536 : (t > 127 * 65536 ? 127 * 65536 : t);
    return (t + (int)noise16) >> 16;
  } else {
    // fp16 primaries: below the smallest normal fp16 value (6e-5: second moments of small gradients live there) the residual
    // keeps up to 24 significant bits, scaled is rounded, and only the reference's own fp32 sequence reproduces it
    constexpr float smax = CORR8 ? 127.0f : 32767.0f;
    float cl = __builtin_fminf(__builtin_fmaxf(en, -1.0f), 1.0f);
    cl = en != en ? en : cl;
    const float scaled = cl * smax;
    return f2i_sat(__builtin_floorf(scaled + uniform16(noise16)));
  }
}

// primary = RNE(x); correction as above
template <bool PRIM_BF16, bool CORR8>
__device__ __forceinline__ void ecc_encode(float x, uint32_t noise16, uint32_t& h, int& c) {
  h = PRIM_BF16 ? f32_to_bf16_rne(x) : f32_to_f16_rne(x);
  c = ecc_correction<PRIM_BF16, CORR8>(x, h, noise16);
}

typedef float hb_float2 __attribute__((ext_vector_type(2)));
typedef __bf16 hb_bf16x2 __attribute__((ext_vector_type(2)));
// two fp32 -> packed bf16 pair (lo = a, hi = b) in one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t pack_bf16_rne(float a, float b) {
  hb_float2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, hb_bf16x2));
}
// low bytes of four ints -> one dword (v_perm_b32 x3)
__device__ __forceinline__ uint32_t pack_bytes(int c0, int c1, int c2, int c3) {
  const uint32_t p01 = __builtin_amdgcn_perm((uint32_t)c1, (uint32_t)c0, 0x0c0c0400u);
  const uint32_t p23 = __builtin_amdgcn_perm((uint32_t)c3, (uint32_t)c2, 0x0c0c0400u);
  return __builtin_amdgcn_perm(p23, p01, 0x05040100u);
}

// ---------------------------------------------------------------------------------------------------------
// Runs of E consecutive elements per lane (E = 8: octet, 4: quartet, 2: pair) of each role
// ---------------------------------------------------------------------------------------------------------
template <int E>
struct RawT {          // what the loads of one role bring in, before decoding
  uint32_t a[E];       // F32: E floats; 16-bit primaries: E / 2 words
  uint32_t c[E / 2];   // corrections: int8 -> E / 4 words (E = 2: the low half of c[0]); int16 -> E / 2 words
};
using Raw = RawT<8>;

__host__ __device__ __forceinline__ constexpr bool fmt_is_ecc(int f) { return f >= HB_FMT_ECC_BF16_8; }
__host__ __device__ __forceinline__ constexpr bool fmt_prim_bf16(int f) {
  return f == HB_FMT_BF16 || f == HB_FMT_ECC_BF16_8 || f == HB_FMT_ECC_BF16_16;
}
__host__ __device__ __forceinline__ constexpr bool fmt_corr8(int f) { return f == HB_FMT_ECC_BF16_8 || f == HB_FMT_ECC_F16_8; }
__host__ __device__ __forceinline__ constexpr int fmt_prim_bytes(int f) { return f == HB_FMT_F32 ? 4 : 2; }
__host__ __device__ __forceinline__ constexpr int fmt_corr_bytes(int f) { return !fmt_is_ecc(f) ? 0 : (fmt_corr8(f) ? 1 : 2); }

// Accesses of the slab, BYTES = 2 .. 32 per lane.  HB_NT = 1 marks them nontemporal: every byte of the slab is touched
// exactly once per step, so nothing is gained by keeping it in the caches.
#ifndef HB_NT
#define HB_NT 1
#endif
typedef uint32_t hb_u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t hb_u32x2 __attribute__((ext_vector_type(2)));
template <typename T>
__device__ __forceinline__ T ld_as(const char* p) {
#if HB_NT
  return __builtin_nontemporal_load(reinterpret_cast<const T*>(p));
#else
  return *reinterpret_cast<const T*>(p);
#endif
}
template <typename T>
__device__ __forceinline__ void st_as(char* p, T v) {
#if HB_NT
  __builtin_nontemporal_store(v, reinterpret_cast<T*>(p));
#else
  *reinterpret_cast<T*>(p) = v;
#endif
}
template <int BYTES>
__device__ __forceinline__ void ld_slab(const char* p, uint32_t* d) {
  static_assert(BYTES == 2 || BYTES == 4 || BYTES == 8 || BYTES == 16 || BYTES == 32, "access width");
  if constexpr (BYTES == 2) {
    d[0] = ld_as<uint16_t>(p);
  } else if constexpr (BYTES == 4) {
    d[0] = ld_as<uint32_t>(p);
  } else if constexpr (BYTES == 8) {
    const hb_u32x2 v = ld_as<hb_u32x2>(p);
    d[0] = v.x;
    d[1] = v.y;
  } else {
#pragma unroll
    for (int h = 0; h < BYTES / 16; ++h) {
      const hb_u32x4 v = ld_as<hb_u32x4>(p + 16 * h);
      d[4 * h] = v.x;
      d[4 * h + 1] = v.y;
      d[4 * h + 2] = v.z;
      d[4 * h + 3] = v.w;
    }
  }
}
template <int BYTES>
__device__ __forceinline__ void st_slab(char* p, const uint32_t* d) {
  static_assert(BYTES == 2 || BYTES == 4 || BYTES == 8 || BYTES == 16 || BYTES == 32, "access width");
  if constexpr (BYTES == 2) {
    st_as<uint16_t>(p, (uint16_t)d[0]);
  } else if constexpr (BYTES == 4) {
    st_as<uint32_t>(p, d[0]);
  } else if constexpr (BYTES == 8) {
    const hb_u32x2 v = {d[0], d[1]};
    st_as<hb_u32x2>(p, v);
  } else {
#pragma unroll
    for (int h = 0; h < BYTES / 16; ++h) {
      const hb_u32x4 v = {d[4 * h], d[4 * h + 1], d[4 * h + 2], d[4 * h + 3]};
      st_as<hb_u32x4>(p + 16 * h, v);
    }
  }
}

template <int F, int E>
__device__ __forceinline__ void raw_load_s(RawT<E>& r, const char* prim, const char* corr, int64_t idx) {
  if (F == HB_FMT_F32) {
    ld_slab<4 * E>(prim + idx * 4, r.a);
  } else {
    ld_slab<2 * E>(prim + idx * 2, r.a);
    if (fmt_is_ecc(F)) {
      if (fmt_corr8(F)) ld_slab<E>(corr + idx, r.c);
      else ld_slab<2 * E>(corr + idx * 2, r.c);
    }
  }
}

template <int F, int E>
__device__ __forceinline__ void raw_decode_s(const RawT<E>& r, float (&x)[E]) {
  if (F == HB_FMT_F32) {
#pragma unroll
    for (int j = 0; j < E; ++j) x[j] = u2f(r.a[j]);
    return;
  }
#pragma unroll
  for (int j = 0; j < E; ++j) {
    uint32_t h = (r.a[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu;
    if (F == HB_FMT_BF16) {
      x[j] = bf16_to_f32(h);
    } else if (F == HB_FMT_F16) {
      x[j] = f16_to_f32(h);
    } else {
      int c;
      if (fmt_corr8(F)) {
        c = (int)(int8_t)((r.c[j >> 2] >> ((j & 3) * 8)) & 0xFFu);
      } else {
        c = (int)(int16_t)((r.c[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu);
      }
      x[j] = ecc_decode<fmt_prim_bf16(F), fmt_corr8(F)>(h, c);
    }
  }
}

// encode E fp32 values into the storage format; `rnd` supplies the 16 noise bits of each element
template <int F, int E>
__device__ __forceinline__ void raw_encode_s(RawT<E>& r, const float (&x)[E], const Noise<E>& rnd) {
  if (F == HB_FMT_F32) {
#pragma unroll
    for (int j = 0; j < E; ++j) r.a[j] = f2u(x[j]);
    return;
  }
  uint32_t w[E / 2];
  uint32_t cw[E / 2];
#pragma unroll
  for (int i = 0; i < E / 2; ++i) w[i] = cw[i] = 0;
  if (F == HB_FMT_ECC_BF16_8) {
    // hot format: convert in pairs, keep the primaries packed, take exponent and value straight from the packed word
    int c[E];
#pragma unroll
    for (int q = 0; q < E / 2; ++q) {
      const uint32_t pk = pack_bf16_rne(x[2 * q], x[2 * q + 1]);
      w[q] = pk;
      c[2 * q] = ecc_correction<true, true>(x[2 * q], pk & 0xFFFFu, rnd.w[q] & 0xFFFFu);
      c[2 * q + 1] = ecc_correction<true, true>(x[2 * q + 1], pk >> 16, rnd.w[q] >> 16);
    }
    if constexpr (E == 2) {
      cw[0] = __builtin_amdgcn_perm((uint32_t)c[1], (uint32_t)c[0], 0x0c0c0400u);
    } else {
#pragma unroll
      for (int q = 0; q < E / 4; ++q) cw[q] = pack_bytes(c[4 * q], c[4 * q + 1], c[4 * q + 2], c[4 * q + 3]);
    }
  } else {
#pragma unroll
    for (int j = 0; j < E; ++j) {
      uint32_t h;
      if (F == HB_FMT_BF16) {
        h = sr_bf16(x[j], rnd.bits16(j));
      } else if (F == HB_FMT_F16) {
        h = f32_to_f16_rne(x[j]);
      } else {
        int c;
        ecc_encode<fmt_prim_bf16(F), fmt_corr8(F)>(x[j], rnd.bits16(j), h, c);
        if (fmt_corr8(F)) {
          cw[j >> 2] |= ((uint32_t)c & 0xFFu) << ((j & 3) * 8);
        } else {
          cw[j >> 1] |= ((uint32_t)c & 0xFFFFu) << ((j & 1) * 16);
        }
      }
      w[j >> 1] |= (h & 0xFFFFu) << ((j & 1) * 16);
    }
  }
#pragma unroll
  for (int i = 0; i < E / 2; ++i) {
    r.a[i] = w[i];
    r.c[i] = cw[i];
  }
}

template <int F, int E>
__device__ __forceinline__ void raw_store_s(const RawT<E>& r, char* prim, char* corr, int64_t idx) {
  if (F == HB_FMT_F32) {
    st_slab<4 * E>(prim + idx * 4, r.a);
  } else {
    st_slab<2 * E>(prim + idx * 2, r.a);
    if (fmt_is_ecc(F)) {
      if (fmt_corr8(F)) st_slab<E>(corr + idx, r.c);
      else st_slab<2 * E>(corr + idx * 2, r.c);
    }
  }
}

// run-time format dispatch: F == kDyn switches on `f` (wave-uniform), otherwise the format is compiled in
#define HB_FMT_SWITCH(F, f, CALL)                                 \
  do {                                                            \
    if constexpr ((F) != kDyn) {                                  \
      CALL(F);                                                    \
    } else {                                                      \
      switch (f) {                                                \
        case HB_FMT_F32: CALL(HB_FMT_F32); break;                 \
        case HB_FMT_BF16: CALL(HB_FMT_BF16); break;               \
        case HB_FMT_F16: CALL(HB_FMT_F16); break;                 \
        case HB_FMT_ECC_BF16_8: CALL(HB_FMT_ECC_BF16_8); break;   \
        case HB_FMT_ECC_BF16_16: CALL(HB_FMT_ECC_BF16_16); break; \
        case HB_FMT_ECC_F16_8: CALL(HB_FMT_ECC_F16_8); break;     \
        default: CALL(HB_FMT_ECC_F16_16); break;                  \
      }                                                           \
    }                                                             \
  } while (0)

template <int F, int E>
__device__ __forceinline__ void raw_load(RawT<E>& r, int f, const char* prim, const char* corr, int64_t idx) {
#define HB_CALL(X) raw_load_s<X, E>(r, prim, corr, idx)
  HB_FMT_SWITCH(F, f, HB_CALL);
#undef HB_CALL
}
template <int F, int E>
__device__ __forceinline__ void raw_decode(const RawT<E>& r, int f, float (&x)[E]) {
#define HB_CALL(X) raw_decode_s<X, E>(r, x)
  HB_FMT_SWITCH(F, f, HB_CALL);
#undef HB_CALL
}
template <int F, int E>
__device__ __forceinline__ void raw_encode(RawT<E>& r, int f, const float (&x)[E], const Noise<E>& rnd) {
#define HB_CALL(X) raw_encode_s<X, E>(r, x, rnd)
  HB_FMT_SWITCH(F, f, HB_CALL);
#undef HB_CALL
}
template <int F, int E>
__device__ __forceinline__ void raw_store(const RawT<E>& r, int f, char* prim, char* corr, int64_t idx) {
#define HB_CALL(X) raw_store_s<X, E>(r, prim, corr, idx)
  HB_FMT_SWITCH(F, f, HB_CALL);
#undef HB_CALL
}
// encode + store in one dispatch: the packed words live inside one case of the switch.  (Shared between an encode switch and
// a store switch they are written and read with a different type in every case, and the compiler then keeps them in scratch
// memory.)
template <int F, int E>
__device__ __forceinline__ void raw_put(int f, const float (&x)[E], const Noise<E>& rnd, char* prim, char* corr, int64_t idx) {
#define HB_CALL(X)                     \
  do {                                 \
    RawT<E> r_;                        \
    raw_encode_s<X, E>(r_, x, rnd);    \
    raw_store_s<X, E>(r_, prim, corr, idx); \
  } while (0)
  HB_FMT_SWITCH(F, f, HB_CALL);
#undef HB_CALL
}
template <int F>
__device__ __forceinline__ void raw_put(int f, const float (&x)[8], const Rand8& rnd, char* prim, char* corr, int64_t idx) {
  raw_put<F, 8>(f, x, Noise<8>{{rnd.w[0], rnd.w[1], rnd.w[2], rnd.w[3]}}, prim, corr, idx);
}
// octet kernels hand their noise over as the four words of a Rand8
template <int F>
__device__ __forceinline__ void raw_encode(Raw& r, int f, const float (&x)[8], const Rand8& rnd) {
  raw_encode<F, 8>(r, f, x, Noise<8>{{rnd.w[0], rnd.w[1], rnd.w[2], rnd.w[3]}});
}

// element-wise (tail) access to a plain gradient buffer that is NOT slab-padded
__device__ __forceinline__ float load_elem(const char* base, int f, int64_t i) {
  if (f == HB_FMT_F32) return reinterpret_cast<const float*>(base)[i];
  uint32_t h = reinterpret_cast<const uint16_t*>(base)[i];
  return f == HB_FMT_BF16 ? bf16_to_f32(h) : f16_to_f32(h);
}
__device__ __forceinline__ void store_elem(char* base, int f, int64_t i, float x) {
  if (f == HB_FMT_F32) {
    reinterpret_cast<float*>(base)[i] = x;
  } else {
    reinterpret_cast<uint16_t*>(base)[i] = (uint16_t)(f == HB_FMT_BF16 ? (f2u(x) >> 16) : f32_to_f16_rne(x));
  }
}

// ---------------------------------------------------------------------------------------------------------
// Correctly rounded sqrt for x that is zero or a normal number: the hardware estimate (<= 1 ulp off) is corrected by
// testing its two neighbours with exact FMA residuals.  Skips the denormal pre-scaling of the general routine; callers
// use it only where a denormal input cannot matter (its root is far below the eps the result is clamped to).
// ---------------------------------------------------------------------------------------------------------
__device__ __forceinline__ float sqrt_rn_normal(float x) {
  float s = __builtin_amdgcn_sqrtf(x);
  const float lo = u2f(f2u(s) - 1u);
  const float hi = u2f(f2u(s) + 1u);
  const float r_lo = __builtin_fmaf(-lo, s, x);
  const float r_hi = __builtin_fmaf(-hi, s, x);
  s = r_lo <= 0.0f ? lo : s;
  s = r_hi > 0.0f ? hi : s;
  return s;
}

// fmaxf(x, lo) for an x that is never a signalling NaN (the result of a square root) and a lo that is a number: the
// hardware maximum returns the operand that is not a NaN, as fmaxf does; the builtin would first canonicalise both.
__device__ __forceinline__ float max_nonnan(float x, float lo) {
  float r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(lo));
  return r;
}

// ---------------------------------------------------------------------------------------------------------
// wavefront reductions (64 lanes) by shuffles
// ---------------------------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ T wave_sum(T v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

}  // namespace hb
