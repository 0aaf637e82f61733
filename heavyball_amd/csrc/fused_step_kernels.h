// Kernel templates of the fused optimizer step, shared by fused_step.hip (host side, un-fused update kernel) and
// fused_step_algo.hip (which instantiates the kernels of one algorithm per object file, so that they build in parallel).
#pragma once
#include <type_traits>
#include <utility>

#include "hb_device.h"
#include "hb_host.h"

namespace hb {

// Work decomposition of the step kernel: every lane owns E consecutive elements of each role per group, a workgroup of
// kThreads lanes takes kWork = kThreads * E * G consecutive elements (G groups per lane, all loads issued before any
// arithmetic), and a chunk of the chunk table is kSub such work units.  Measured on MI355X over E = 2, 4, 8, G = 1, 2, 4
// and 64 ... 512 lanes: the pass that reads and writes every role is fastest with narrow runs (an arithmetic-free kernel
// with the access pattern of the ECC LaProp step moves 5.8 TB/s with 8 elements per lane, 6.0 with 4, 6.3 with 2; the real
// kernel turns compute-bound at 2), the read-only count pass of caution with wide ones.
#ifndef HB_THREADS
#define HB_THREADS 256
#endif
constexpr int kThreads = HB_THREADS;
template <int E_, int G_>
struct Geo {
  static constexpr int E = E_, G = G_;
  static constexpr int kWork = kThreads * E * G;
  static constexpr int kSub = HB_CHUNK / kWork;
  static_assert(E == 2 || E == 4 || E == 8, "2, 4 or 8 elements per lane");
  static_assert(kSub >= 1 && kSub * kWork == HB_CHUNK, "a chunk must be a whole number of work units");
};
#ifndef HB_GEO_STEP
#define HB_GEO_STEP Geo<4, 2>
#endif
#ifndef HB_GEO_COUNT
#define HB_GEO_COUNT Geo<8, 2>
#endif
#ifndef HB_GEO_F32  // the all-fp32 triple: no codec work at all
#define HB_GEO_F32 Geo<2, 2>
#endif

struct StepArgs {
  char* param;
  char* param_corr;
  const char* grad;
  const char* const* grad_ptrs;
  char* m;
  char* m_corr;
  char* v;
  char* v_corr;
  char* og;
  char* og_corr;
  char* s3;  // AdEMAMix: slow momentum
  char* s3_corr;
  char* upd;           // HB_FLAG_UPDATE_ONLY: fp32 slab that takes the update (null: a.param does)
  const float* tscal;  // NAdam: two weights per tensor
  const int64_t* offsets;
  const int64_t* numel;
  const int2* chunks;
  uint32_t* counts;
  int64_t n_chunks;
  int pf, gf, sf;
  uint32_t flags;
  float a1, oma1, a2, oma2, amars, omamars, neg_lr, omdl, eps;
  float a3, oma3, alpha, wd;
  Rng rng;
};

enum { kNoCaution = 0, kCautionCount = 1, kCautionApply = 2 };

// f(integral_constant<int, 0>), f(integral_constant<int, 1>), ... in order
template <class F, int... K>
__device__ __forceinline__ void for_each_index(F&& f, std::integer_sequence<int, K...>) {
  (f(std::integral_constant<int, K>{}), ...);
}

// The masked elements a workgroup counted go into one of the tensor's HB_CAUTION_SLOTS counters: one addition per workgroup
// (wavefront shuffles, then four words of LDS), and neighbouring workgroups add into different words.  Additions to one
// address queue up in the L2 (about 200 M a second measured): with one counter per tensor and one addition per wavefront
// the count pass of a training-like state, where every wavefront has masked elements, spent five times its streaming time there.
__device__ __forceinline__ void add_masked(uint32_t* counts, int t, int slot, uint32_t masked) {
  __shared__ uint32_t per_wave[kThreads / kWave];
  masked = wave_sum(masked);
  const int wave = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) per_wave[wave] = masked;
  __syncthreads();
  if (threadIdx.x == 0) {
    uint32_t total = 0;
#pragma unroll
    for (int i = 0; i < kThreads / kWave; ++i) total += per_wave[i];
    if (total) atomicAdd(&counts[(size_t)t * HB_CAUTION_SLOTS + slot], total);
  }
  __syncthreads();  // the words are reused by the workgroup's next work unit
}

// the masked elements of tensor t: the sum of its counters
__device__ __forceinline__ int64_t masked_of(const uint32_t* counts, int t) {
  const uint32_t* c = counts + (size_t)t * HB_CAUTION_SLOTS;
  uint32_t total = 0;  // a tensor has fewer than 2^32 elements
#pragma unroll
  for (int i = 0; i < HB_CAUTION_SLOTS; ++i) total += c[i];
  return (int64_t)total;
}

// One work unit.  FULL = every lane's elements are inside the tensor (the common case): no bounds tests at all.
template <int ALGO, bool MARS, int CAUTION, int PF, int GF, int SF, bool FULL, class GEO>
__device__ __forceinline__ void step_chunk(const StepArgs& a, const int pf, const int gf, const int sf, const int t, const int valid,
                                           const int64_t flat0, const char* gbase, const int64_t g0, const bool g_slab, const float scale,
                                           const float gw, const float ew, const int slot) {
  constexpr int kE = GEO::E, kGroups = GEO::G;
  constexpr bool kCount = CAUTION == kCautionCount;
  constexpr bool kAdopt = ALGO == HB_ALGO_ADOPT, kMix = ALGO == HB_ALGO_ADEMAMIX, kNadam = ALGO == HB_ALGO_NADAM;
  // the count pass of Adam and AdEMAMix needs only the sign of the numerator of the update
  constexpr bool kNeedV = !(kCount && (ALGO == HB_ALGO_ADAM || kMix));
  // Adam's count pass over bf16 + int8 state with bf16 gradients reads the bf16 primaries alone and decides the sign of
  // the update from them wherever the corrections (at most half a bf16 ulp of the primary) and the rounding of the MARS
  // gradient (less than one bf16 ulp) cannot change it; a lane with an element too close to call loads the corrections
  // and takes the exact route.  Bit-identical counts, 6 instead of 8 bytes per element on almost every lane, and no
  // random numbers on the short route.
  constexpr bool kLazy = kCount && ALGO == HB_ALGO_ADAM && SF == HB_FMT_ECC_BF16_8 && GF == HB_FMT_BF16;
  // ADOPT's warm-up step (heavyball/chainable.py:945-946) is the lerp of exp_avg_sq with weights (a2, oma2) = (1, 0) and
  // nothing else: exp_avg and the parameter are neither loaded nor stored (their registers hold zeros meanwhile)
  const bool warmup = kAdopt && (a.flags & HB_FLAG_ADOPT_WARMUP) != 0;
  const bool coupled = kNadam && (a.flags & HB_FLAG_COUPLED_WD) != 0;  // the decay enters through the gradient
  const bool cautious_wd = (a.flags & HB_FLAG_CAUTIOUS_WD) != 0;
  const bool update_only = (a.flags & HB_FLAG_UPDATE_ONLY) != 0;
  const bool write_grad = MARS && !kCount && (a.flags & HB_FLAG_WRITE_GRAD) != 0;
  const bool mars_only = MARS && (a.flags & HB_FLAG_MARS_ONLY) != 0;  // the prologue alone: corrected gradient -> a.param (fp32)
  const bool state_rounds = sf != HB_FMT_F32;
  // raw gradient -> old_grad: exact (no noise needed) when both are bf16, or the target is fp32
  const bool og_rounds = MARS && state_rounds && !(gf == HB_FMT_BF16 && fmt_prim_bf16(sf));
  // sqrt(v) is clamped to eps: with eps >= 1e-18 a denormal v (root < 1.1e-19) never reaches the result
  const bool fast_sqrt = a.eps >= 1e-18f;

  RawT<kE> rp[kGroups], rg[kGroups], rm[kGroups], rv[kGroups], ro[kGroups], rs[kGroups];
  bool tail[kGroups];  // the group's gradient came by element loads: rg[k].a holds fp32 values whatever the gradient's format
  // the loads of one group
  auto fetch = [&](auto kc) {
    constexpr int k = decltype(kc)::value;
    const int e = k * (kThreads * kE) + threadIdx.x * kE;
    tail[k] = false;
    if (FULL || e < valid) {
      const int64_t idx = flat0 + e;
      if (FULL || g_slab || e + kE <= valid) {
        raw_load<GF>(rg[k], gf, gbase, nullptr, g0 + e);
      } else {  // last, partial run of a gradient that is not padded: element loads
        tail[k] = true;
#pragma unroll
        for (int j = 0; j < kE; ++j) rg[k].a[j] = e + j < valid ? f2u(load_elem(gbase, gf, g0 + e + j)) : 0u;
      }
      if (kAdopt) rm[k] = rp[k] = RawT<kE>{};
      if constexpr (kLazy) {  // primaries only
        ld_slab<2 * kE>(a.m + idx * 2, rm[k].a);
        if (MARS) ld_slab<2 * kE>(a.og + idx * 2, ro[k].a);
        return;
      }
      if (MARS) raw_load<SF>(ro[k], sf, a.og, a.og_corr, idx);
      if (mars_only) {
        rm[k] = rv[k] = rs[k] = rp[k] = RawT<kE>{};
      } else {
        if (!kAdopt || !warmup) raw_load<SF>(rm[k], sf, a.m, a.m_corr, idx);
        if (kNeedV) raw_load<SF>(rv[k], sf, a.v, a.v_corr, idx);
        if (kMix) raw_load<SF>(rs[k], sf, a.s3, a.s3_corr, idx);
        if ((!kCount && (!kAdopt || !warmup)) || (kNadam && coupled)) raw_load<PF>(rp[k], pf, a.param, a.param_corr, idx);
      }
    }
  };
  for_each_index(fetch, std::make_integer_sequence<int, kGroups>{});

  uint32_t masked = 0;
  // One group.  A generic lambda over a compile-time index instead of an unrolled loop: with run-time format codes
  // the body is too large for the unroller, and a rolled loop would index the register arrays above dynamically.
  auto group = [&](auto kc) {
    constexpr int k = decltype(kc)::value;
    const int e = k * (kThreads * kE) + threadIdx.x * kE;
    if (!FULL && e >= valid) return;
    const int64_t idx = flat0 + e;
    float p[kE], g[kE], m[kE], v[kE], og[kE], u[kE], sl[kE];
    Noise<kE> rn_p{};  // noise of the parameter's rounding
    if (!FULL && tail[k]) {
#pragma unroll
      for (int j = 0; j < kE; ++j) g[j] = u2f(rg[k].a[j]);
    } else {
      raw_decode<GF>(rg[k], gf, g);
    }
    if constexpr (kLazy) {
      uint32_t undecided = 0;  // bit j: element j is too close to call from the primaries
      uint32_t fast = 0;
      // Bounds, all on the safe side.  A bf16 + int8 pair lies within 2^(max(e, 1) - 135) of its primary x (e its exponent
      // field), which is at most max(|x| 2^-8, 2^-126) <= |x| 2^-8 + 2^-126: with x times a coefficient already at hand
      // (t2, s1) the bound costs one multiply.  The factors 1.01 cover the roundings of the bound arithmetic itself.
      const float k_ulp = 1.01f * 0x1p-8f;
      const float c_o = __builtin_fabsf(a.amars) * (1.01f * 0x1p-126f);
      const float c_m = __builtin_fabsf(a.oma1) * (1.01f * 0x1p-126f);
      const float k_a1 = __builtin_fabsf(a.a1) * 1.01f;
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        const uint32_t hm = (rm[k].a[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu;
        const float mp = bf16_to_f32(hm);
        float gs = g[j], dg = 0.0f;
        bool sure = true;
        if (MARS) {
          const uint32_t ho = (ro[k].a[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu;
          const float t1 = g[j] * a.omamars, t2 = bf16_to_f32(ho) * a.amars;
          gs = t1 + t2;  // the corrected gradient before its rounding, from the primary of old_grad
          // what the correction of old_grad and the fp32 roundings can move
          // (the bounds are not part of the reference's arithmetic: fused multiply-adds, whose single rounding the 1.01 covers)
          const float eo = __builtin_fmaf(__builtin_fabsf(t2), k_ulp, __builtin_fmaf(__builtin_fabsf(t1) + __builtin_fabsf(t2), 0x1p-22f, c_o));
          sure = __builtin_fabsf(gs) > eo;  // its sign is settled (the stochastic rounding to bf16 keeps the sign)
          dg = __builtin_fmaf(__builtin_fabsf(gs) + eo, 0x1p-7f, eo) + 1e-39f;  // ... and its value to within one bf16 ulp more
        }
        const float s1 = mp * a.oma1, s2 = gs * a.a1;
        const float mn = s1 + s2;
        const float em = __builtin_fmaf(__builtin_fabsf(s1), k_ulp,
                                        __builtin_fmaf(k_a1, dg, __builtin_fmaf(__builtin_fabsf(s1) + __builtin_fabsf(s2), 0x1p-21f, c_m)));
        sure = sure && __builtin_fabsf(mn) > em;  // NaN compares false: the exact route decides
        const bool inside = FULL || e + j < valid;
        if (inside && !sure) undecided |= 1u << j;
        else fast += (inside && ((f2u(gs) ^ f2u(mn)) >> 31) != 0) ? 1u : 0u;
      }
      masked += fast;
      // The exact route, element by element: 0.2-0.3 % of the elements of a training-like state need it, which still is
      // three quarters of the wavefronts (64 lanes of 8 elements), so it has to cost a wavefront little: one quartet's random
      // numbers and the flagged elements alone, not the whole group with every lane but one idle.
      if (undecided) {
        // both correction words first, so that the flagged elements wait for memory once and not one after the other
        ld_slab<kE>(a.m_corr + idx, rm[k].c);
        if (MARS) ld_slab<kE>(a.og_corr + idx, ro[k].c);
#pragma unroll
        for (int q = 0; q < kE / 4; ++q) {
          if (!(undecided & (0xFu << (4 * q)))) continue;
          Rand8 r{{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u}};
          if (MARS && a.rng.mode == HB_RNG_PHILOX) r = a.rng.call(idx + 4 * q, HB_STREAM_MARS_SR >> 1);
#pragma unroll
          for (int jj = 0; jj < 4; ++jj) {
            const int j = 4 * q + jj;
            if (!((undecided >> j) & 1u)) continue;
            const uint32_t hm = (rm[k].a[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu;
            const float mx = ecc_decode<true, true>(hm, (int)(int8_t)(rm[k].c[j >> 2] >> ((j & 3) * 8)));
            float gc = g[j];
            if (MARS) {
              const uint32_t ho = (ro[k].a[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu;
              const float ox = ecc_decode<true, true>(ho, (int)(int8_t)(ro[k].c[j >> 2] >> ((j & 3) * 8)));
              gc = g[j] * a.omamars + ox * a.amars;  // heavyball/utils.py:1048, then its rounding to the gradient's bf16
              gc = bf16_to_f32(sr_bf16(gc, (r.w[jj >> 1] >> ((jj & 1) * 16)) & 0xFFFFu));  // word and half of HB_STREAM_MARS_SR
            }
            const float mn = mx * a.oma1 + gc * a.a1;  // heavyball/utils.py:1939; the sign of m / den is the sign of m
            masked += ((f2u(gc) ^ f2u(mn)) >> 31) != 0 ? 1u : 0u;
          }
        }
      }
      return;
    }
    raw_decode<SF>(rm[k], sf, m);
    if (kNeedV) raw_decode<SF>(rv[k], sf, v);
    if (kMix) raw_decode<SF>(rs[k], sf, sl);
    if (!kCount || (kNadam && coupled)) raw_decode<PF>(rp[k], pf, p);

    if (MARS) {
      raw_decode<SF>(ro[k], sf, og);
      Noise<kE> rn{};  // HB_STREAM_MARS_SR shares its Philox calls with HB_STREAM_PARAM (rn_p, used at the end)
      if (gf == HB_FMT_BF16) a.rng.noise_pair<kE>(idx, HB_STREAM_MARS_SR >> 1, rn, rn_p);
      else if (pf != HB_FMT_F32 && !kCount) rn_p = a.rng.noise<kE>(idx, HB_STREAM_PARAM);
#pragma unroll
      for (int j = 0; j < kE; ++j) {
        float gc = g[j] * a.omamars + og[j] * a.amars;  // heavyball/utils.py:1048
        if (gf == HB_FMT_BF16) gc = bf16_to_f32(sr_bf16(gc, rn.bits16(j)));
        else if (gf == HB_FMT_F16) gc = f16_to_f32(f32_to_f16_rne(gc));
        og[j] = g[j];  // old_grad <- the raw gradient (heavyball/utils.py:3619)
        g[j] = gc;
      }
      if (!kCount) {
        // a bf16 gradient stored into a bf16 primary is its own encoding: the primary takes the gradient's bits and the
        // correction is zero (what the encoder would compute: the residual is 0 and floor(0 + noise / 65536) = 0)
        constexpr bool kCopy = GF == HB_FMT_BF16 && (SF == HB_FMT_BF16 || SF == HB_FMT_ECC_BF16_8 || SF == HB_FMT_ECC_BF16_16);
        if constexpr (kCopy) {  // a compiled-in format: one store behind both ways of filling the words
          RawT<kE> w;
          if (FULL || !tail[k]) {
#pragma unroll
            for (int i = 0; i < kE / 2; ++i) {
              w.a[i] = rg[k].a[i];
              w.c[i] = 0;
            }
          } else {
            const Noise<kE> rn_og = og_rounds ? a.rng.noise<kE>(idx, HB_STREAM_OLD_GRAD) : Noise<kE>{};
            raw_encode<SF>(w, sf, og, rn_og);
          }
          raw_store<SF>(w, sf, a.og, a.og_corr, idx);
        } else {
          const Noise<kE> rn_og = og_rounds ? a.rng.noise<kE>(idx, HB_STREAM_OLD_GRAD) : Noise<kE>{};
          raw_put<SF>(sf, og, rn_og, a.og, a.og_corr, idx);
        }
        if (write_grad) {
#pragma unroll
          for (int j = 0; j < kE; ++j)
            if (FULL || e + j < valid) store_elem(const_cast<char*>(gbase), gf, g0 + e + j, g[j]);
        }
        if (mars_only) {
          raw_put<HB_FMT_F32>(HB_FMT_F32, g, Noise<kE>{}, a.param, nullptr, idx);
          return;
        }
      }
    }

    // The denominators of the group first, with one wave-uniform choice of the square-root routine for all of them
    // (taken per element the choice costs two branches each).
    float den[kE];
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      if (kNadam && coupled) g[j] = __builtin_fmaf(p[j], a.wd, g[j]);  // heavyball/utils.py:363-364, add_ with alpha
      // heavyball/utils.py:426-427; ADOPT (:2300-2304) takes the denominator from v as the steps before left it
      if (kNeedV && !kAdopt) v[j] = v[j] * a.oma2 + (g[j] * g[j]) * a.a2;
      den[j] = 1.0f;
    }
    if (kNeedV || kAdopt) {
      if (fast_sqrt) {
#pragma unroll
        for (int j = 0; j < kE; ++j) den[j] = max_nonnan(sqrt_rn_normal(v[j]), a.eps);  // heavyball/utils.py:413-414
      } else {
#pragma unroll
        for (int j = 0; j < kE; ++j) den[j] = max_nonnan(__builtin_sqrtf(v[j]), a.eps);
      }
    }
#pragma unroll
    for (int j = 0; j < kE; ++j) {
      if (kAdopt) v[j] = v[j] * a.oma2 + (g[j] * g[j]) * a.a2;
      if (ALGO == HB_ALGO_ADAM) {
        m[j] = m[j] * a.oma1 + g[j] * a.a1;  // heavyball/utils.py:1939
        u[j] = kNeedV ? m[j] / den[j] : m[j];   // :1943 (count pass: the sign of m is the sign of m / den)
      } else if (kMix) {
        m[j] = m[j] * a.oma1 + g[j] * a.a1;     // heavyball/utils.py:2104 (fast)
        sl[j] = sl[j] * a.oma3 + g[j] * a.a3;   // :2105 (slow, beta3 is not debiased)
        const float num = m[j] + sl[j] * a.alpha;  // :2108
        u[j] = kNeedV ? num / den[j] : num;
      } else if (kNadam) {
        m[j] = m[j] * a.oma1 + g[j] * a.a1;              // heavyball/utils.py:394 (beta1 is not debiased)
        u[j] = (g[j] / den[j]) * gw + (m[j] / den[j]) * ew;    // :409
        if (coupled) u[j] = u[j] - p[j] * a.wd;          // :378
      } else {  // LaProp, and ADOPT with the denominator chosen above
        m[j] = m[j] * a.oma1 + (g[j] / den[j]) * a.a1;  // heavyball/utils.py:2267-2268, :2300
        u[j] = m[j];
      }
      if (CAUTION != kNoCaution) {
        const bool mk = ((f2u(g[j]) ^ f2u(u[j])) >> 31) != 0;  // heavyball/utils.py:3654
        if (kCount) {
          masked += (mk && (FULL || e + j < valid)) ? 1u : 0u;
        } else {
          u[j] = (mk ? 0.0f : u[j]) * scale;
        }
      }
    }

    if (!kCount) {
      if (update_only) {  // un-fused transform: the update itself is the output, in the precision of the reference's update buffer
        if (gf == HB_FMT_BF16) {
          const Noise<kE> rn_u = a.rng.noise<kE>(idx, HB_STREAM_UPDATE);
#pragma unroll
          for (int j = 0; j < kE; ++j) u[j] = bf16_to_f32(sr_bf16(u[j], rn_u.bits16(j)));
        } else if (gf == HB_FMT_F16) {
#pragma unroll
          for (int j = 0; j < kE; ++j) u[j] = f16_to_f32(f32_to_f16_rne(u[j]));
        }
#pragma unroll
        for (int j = 0; j < kE; ++j) p[j] = u[j];
      } else if (cautious_wd) {  // heavyball/utils.py:2388-2389
#pragma unroll
        for (int j = 0; j < kE; ++j) {
          const float om = ((f2u(p[j]) ^ f2u(u[j])) >> 31) ? 1.0f : a.omdl;
          p[j] = p[j] * om + u[j] * a.neg_lr;
        }
      } else {
#pragma unroll
        for (int j = 0; j < kE; ++j) p[j] = p[j] * a.omdl + u[j] * a.neg_lr;  // heavyball/utils.py:2389
      }
      Noise<kE> rn_m{}, rn_v{};  // exp_avg and exp_avg_sq share their Philox calls
      if (state_rounds) a.rng.noise_pair<kE>(idx, HB_STREAM_EXP_AVG >> 1, rn_m, rn_v);
      if (!kAdopt || !warmup) {
        raw_put<SF>(sf, m, rn_m, a.m, a.m_corr, idx);
      }
      raw_put<SF>(sf, v, rn_v, a.v, a.v_corr, idx);
      if (kMix) {
        const Noise<kE> rn = state_rounds ? a.rng.noise<kE>(idx, HB_STREAM_EXP_AVG_SLOW) : Noise<kE>{};
        raw_put<SF>(sf, sl, rn, a.s3, a.s3_corr, idx);
      }
      if (update_only && a.upd != nullptr) {
        raw_put<HB_FMT_F32>(HB_FMT_F32, p, Noise<kE>{}, a.upd, nullptr, idx);
      } else if (!kAdopt || !warmup) {
        if (!MARS && pf != HB_FMT_F32) rn_p = a.rng.noise<kE>(idx, HB_STREAM_PARAM);
        raw_put<PF>(pf, p, rn_p, a.param, a.param_corr, idx);
      }
    }
  };
  for_each_index(group, std::make_integer_sequence<int, kGroups>{});

  if (kCount) add_masked(a.counts, t, slot, masked);
}

#ifndef HB_COUNT_WAVES  // wavefronts per SIMD the compiler must leave room for (its register budget) in the count pass ...
#define HB_COUNT_WAVES 1
#endif
#ifndef HB_STEP_WAVES  // ... and in the passes that write
#define HB_STEP_WAVES 1
#endif
template <int ALGO, bool MARS, int CAUTION, int PF, int GF, int SF, class GEO>
__global__ __launch_bounds__(kThreads, CAUTION == kCautionCount ? HB_COUNT_WAVES : HB_STEP_WAVES) void fused_step_kernel(const StepArgs a) {
  constexpr int kWork = GEO::kWork, kSub = GEO::kSub;
  const int pf = PF == kDyn ? a.pf : PF;
  const int gf = GF == kDyn ? a.gf : GF;
  const int sf = SF == kDyn ? a.sf : SF;
  for (int64_t w = blockIdx.x; w < a.n_chunks * kSub; w += gridDim.x) {
    const int2 ent = a.chunks[w / kSub];
    const int t = ent.x;
    const int64_t off = a.offsets[t];
    const int64_t n = a.numel[t];
    const int64_t local0 = (int64_t)ent.y * HB_CHUNK + (int64_t)(w % kSub) * kWork;
    const int64_t rem = n - local0;
    if (rem <= 0) continue;  // a work unit behind the end of the tensor's last chunk
    const int valid = rem < kWork ? (int)rem : kWork;
    const int64_t flat0 = off + local0;
    const bool g_slab = a.grad_ptrs == nullptr;
    const char* gbase = g_slab ? a.grad : a.grad_ptrs[t];
    const int64_t g0 = g_slab ? flat0 : local0;
    float scale = 1.0f;
    if (CAUTION == kCautionApply) {
      const int64_t kept = n - masked_of(a.counts, t);
      // heavyball/utils.py:3656: `numel / kept_tensor` is Tensor.__rtruediv__, i.e. reciprocal(kept) * numel in fp32
      scale = (1.0f / (float)(kept < 1 ? 1 : kept)) * (float)n;
    }
    float gw = 0.0f, ew = 0.0f;
    if (ALGO == HB_ALGO_NADAM) {
      gw = a.tscal[2 * t];
      ew = a.tscal[2 * t + 1];
    }
    const int slot = (int)(w & (HB_CAUTION_SLOTS - 1));
    if (valid == kWork) step_chunk<ALGO, MARS, CAUTION, PF, GF, SF, true, GEO>(a, pf, gf, sf, t, valid, flat0, gbase, g0, g_slab, scale, gw, ew, slot);
    else step_chunk<ALGO, MARS, CAUTION, PF, GF, SF, false, GEO>(a, pf, gf, sf, t, valid, flat0, gbase, g0, g_slab, scale, gw, ew, slot);
  }
}

// a kernel and the number of its work units per chunk (the grid is n_chunks * sub workgroups)
struct StepKernel {
  void (*fn)(const StepArgs);
  int sub;
};

template <int ALGO, int PF, int GF, int SF, class S = HB_GEO_STEP>
inline StepKernel pick_pass(bool mars, int caution) {
  using C = HB_GEO_COUNT;
  if (mars) {
    if (caution == kNoCaution) return {fused_step_kernel<ALGO, true, kNoCaution, PF, GF, SF, S>, S::kSub};
    if (caution == kCautionCount) return {fused_step_kernel<ALGO, true, kCautionCount, PF, GF, SF, C>, C::kSub};
    return {fused_step_kernel<ALGO, true, kCautionApply, PF, GF, SF, S>, S::kSub};
  }
  if (caution == kNoCaution) return {fused_step_kernel<ALGO, false, kNoCaution, PF, GF, SF, S>, S::kSub};
  if (caution == kCautionCount) return {fused_step_kernel<ALGO, false, kCautionCount, PF, GF, SF, C>, C::kSub};
  return {fused_step_kernel<ALGO, false, kCautionApply, PF, GF, SF, S>, S::kSub};
}

// The kernel of one algorithm for a (param, grad, state) format triple: three triples are statically specialised,
// everything else takes the kernel that switches on run-time format codes.  Explicitly instantiated per algorithm in
// fused_step_algo.hip.
//
// The geometry goes with the triple: the less arithmetic a step carries per byte, the less a lane should hold.  Measured on one
// MI355X (fraction of 8 TB/s, Geo<4,2> / <4,1> / <2,2> / <2,4>): (f32,f32,f32) 0.733 / 0.776 / 0.778 / 0.763, (f32,bf16,f32)
// 0.766 / 0.803 / 0.808 / 0.772, (bf16,bf16,f32) 0.775 / 0.806 / 0.767 / 0.792, (f32,f32,bf16) 0.760 / 0.787 / 0.738 / 0.799,
// (f32,f32,ecc) 0.757 / 0.773 / 0.711 / 0.754, while the triples with the most arithmetic, (f32,bf16,ecc) 0.767 / 0.735 / 0.689 /
// 0.722, (ecc,bf16,ecc) with MARS 0.722 / 0.712 / 0.636 / 0.629 and (bf16,bf16,bf16) 0.679 / 0.611 / 0.510 / 0.561, want Geo<4,2>.
template <int ALGO>
StepKernel pick_algo(bool mars, int caution, int pf, int gf, int sf) {
  if (pf == HB_FMT_F32 && gf == HB_FMT_F32 && sf == HB_FMT_F32)
    return pick_pass<ALGO, HB_FMT_F32, HB_FMT_F32, HB_FMT_F32, HB_GEO_F32>(mars, caution);
  if (pf == HB_FMT_F32 && gf == HB_FMT_BF16 && sf == HB_FMT_ECC_BF16_8)
    return pick_pass<ALGO, HB_FMT_F32, HB_FMT_BF16, HB_FMT_ECC_BF16_8>(mars, caution);
  if (pf == HB_FMT_ECC_BF16_8 && gf == HB_FMT_BF16 && sf == HB_FMT_ECC_BF16_8)
    return pick_pass<ALGO, HB_FMT_ECC_BF16_8, HB_FMT_BF16, HB_FMT_ECC_BF16_8>(mars, caution);
  // mixed-precision set-ups without ECC: bf16 parameters and gradients over fp32 moments, fp32 parameters with bf16 gradients
  // (measured 4.6 / 5.2 TB/s on the run-time-format kernel), for every algorithm
  if (pf == HB_FMT_BF16 && gf == HB_FMT_BF16 && sf == HB_FMT_F32)
    return pick_pass<ALGO, HB_FMT_BF16, HB_FMT_BF16, HB_FMT_F32, Geo<4, 1>>(mars, caution);
  if (pf == HB_FMT_F32 && gf == HB_FMT_BF16 && sf == HB_FMT_F32)
    return pick_pass<ALGO, HB_FMT_F32, HB_FMT_BF16, HB_FMT_F32, Geo<2, 2>>(mars, caution);
  // for the two optimizers that are mostly run: bf16 moments, and the wide correction of the bf16 ECC pair
  if constexpr (ALGO == HB_ALGO_ADAM || ALGO == HB_ALGO_LAPROP) {
    if (pf == HB_FMT_BF16 && gf == HB_FMT_BF16 && sf == HB_FMT_BF16) return pick_pass<ALGO, HB_FMT_BF16, HB_FMT_BF16, HB_FMT_BF16>(mars, caution);
    if (pf == HB_FMT_F32 && gf == HB_FMT_BF16 && sf == HB_FMT_ECC_BF16_16)
      return pick_pass<ALGO, HB_FMT_F32, HB_FMT_BF16, HB_FMT_ECC_BF16_16>(mars, caution);
    if (pf == HB_FMT_ECC_BF16_16 && gf == HB_FMT_BF16 && sf == HB_FMT_ECC_BF16_16)
      return pick_pass<ALGO, HB_FMT_ECC_BF16_16, HB_FMT_BF16, HB_FMT_ECC_BF16_16>(mars, caution);
    // fp32 parameters and gradients over narrow moments (storage_dtype="bfloat16", ecc="bf16+8")
    if (pf == HB_FMT_F32 && gf == HB_FMT_F32 && sf == HB_FMT_BF16)
      return pick_pass<ALGO, HB_FMT_F32, HB_FMT_F32, HB_FMT_BF16, Geo<2, 4>>(mars, caution);
    if (pf == HB_FMT_F32 && gf == HB_FMT_F32 && sf == HB_FMT_ECC_BF16_8)
      return pick_pass<ALGO, HB_FMT_F32, HB_FMT_F32, HB_FMT_ECC_BF16_8, Geo<4, 1>>(mars, caution);
  }
  return pick_pass<ALGO, kDyn, kDyn, kDyn>(mars, caution);
}

}  // namespace hb
