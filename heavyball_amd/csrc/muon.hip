// Muon's momentum on an fp32 slab, in the four forms heavyball.Muon can be built with (heavyball/__init__.py:723-737):
//   HB_MOM_NESTEROV_EMA        m <- m*(1-a) + g*a ; u <- g + m        heavyball/utils.py:766-769, raw beta (a = 1 - beta)
//   HB_MOM_EMA                 m <- m*(1-a) + g*a ; u <- m            :457-460, debiased beta (chainable.py:652-653)
//   HB_MOM_HEAVYBALL           m <- m*beta + g    ; u <- m            :737-741
//   HB_MOM_NESTEROV_HEAVYBALL  m <- m*beta + g    ; u <- g + m*beta   :745-749
// Same chunked, one-workgroup-per-chunk traversal as the fused first-order step.
#include "hb_device.h"
#include "hb_host.h"

namespace hb {

constexpr int kMThreads = 256;
// A lane owns kME consecutive elements and a workgroup kMWork of them; a chunk of the chunk table is kMSub such work units.
// Streams of plain fp32 want short runs per lane (the fused step measured the same): 4 elements per lane and one group per
// workgroup moved 6.0 TB/s where 8 elements in two groups moved 4.9.
#ifndef HB_MOM_E
#define HB_MOM_E 4
#endif
constexpr int kME = HB_MOM_E;
constexpr int kMWork = kMThreads * kME;
constexpr int kMSub = HB_CHUNK / kMWork;
static_assert(kMSub * kMWork == HB_CHUNK && (kME == 4 || kME == 8), "a chunk is a whole number of work units");

// MF: storage format of the momentum (HB_FMT_F32 compiled in, or kDyn for bf16 / ECC pairs decided at run time)
template <int MF>
__global__ __launch_bounds__(kMThreads) void momentum_kernel(char* __restrict__ mom, char* __restrict__ mom_corr, int mf, float* __restrict__ upd,
                                                              const char* __restrict__ grad, const char* const* __restrict__ grad_ptrs, int gf,
                                                              const int64_t* __restrict__ offsets, const int64_t* __restrict__ numel,
                                                              const int2* __restrict__ chunks, int64_t n_chunks, float a, float oma, int mode,
                                                              Rng rng, double* __restrict__ sumsq_parts) {
  for (int64_t w = blockIdx.x; w < n_chunks * kMSub; w += gridDim.x) {
    const int2 ent = chunks[w / kMSub];
    const int64_t local0 = (int64_t)ent.y * HB_CHUNK + (int64_t)(w % kMSub) * kMWork;
    const int64_t rem = numel[ent.x] - local0;
    // sumsq_parts: the sum of squares of the update this wavefront writes, one double per wavefront and work unit (no barrier,
    // no atomics: whoever adds them up gets the same sum in every run); zero for a unit or a wavefront past the tensor's end
    double* const part = sumsq_parts ? sumsq_parts + w * (kMThreads / 64) + (threadIdx.x >> 6) : nullptr;
    if (rem <= 0) {  // a work unit behind the end of the tensor's last chunk
      if (part && (threadIdx.x & 63) == 0) *part = 0.0;
      continue;
    }
    const int valid = rem < kMWork ? (int)rem : kMWork;
    const int64_t flat0 = offsets[ent.x] + local0;
    const bool g_slab = grad_ptrs == nullptr;
    const char* gbase = g_slab ? grad : grad_ptrs[ent.x];
    const int64_t g0 = g_slab ? flat0 : local0;
    const int e = threadIdx.x * kME;
    double ss = 0.0;  // this lane's share of the unit's sum of squares; lanes past the tensor's end add nothing
    if (e < valid) {
      const int64_t idx = flat0 + e;
      RawT<kME> rm;
      float m[kME], g[kME], u[kME];
      raw_load<MF>(rm, mf, mom, mom_corr, idx);
      if (g_slab || e + kME <= valid) {  // a whole run: one wide load (gradient buffers are 16-byte aligned)
        RawT<kME> rg;
        raw_load<kDyn>(rg, gf, gbase, nullptr, g0 + e);
        raw_decode<kDyn>(rg, gf, g);
      } else {  // last, partial run of a gradient that is not padded
#pragma unroll
        for (int j = 0; j < kME; ++j) g[j] = e + j < valid ? load_elem(gbase, gf, g0 + e + j) : 0.0f;
      }
      raw_decode<MF>(rm, mf, m);
#pragma unroll
      for (int j = 0; j < kME; ++j) {
        if (mode == HB_MOM_NESTEROV_EMA) {
          m[j] = m[j] * oma + g[j] * a;  // heavyball/utils.py:1048 via _lerp (:1847)
          u[j] = g[j] + m[j] * 1.0f;     // stochastic_add_(grad, ema32, 1), heavyball/utils.py:1127-1130
        } else if (mode == HB_MOM_EMA) {
          m[j] = m[j] * oma + g[j] * a;
          u[j] = m[j];
        } else {  // a carries beta
          m[j] = m[j] * a + g[j];
          u[j] = mode == HB_MOM_HEAVYBALL ? m[j] : g[j] + m[j] * a;
        }
      }
      // the update buffer of the reference has the gradient's dtype: a 16-bit gradient rounds the update as
      // copy_stochastic_ does (bf16: stochastic, fp16: to nearest), heavyball/utils.py:2363-2370
      if (gf == HB_FMT_BF16) {
        const Noise<kME> rn = rng.noise<kME>(idx, HB_STREAM_MARS_SR);
#pragma unroll
        for (int j = 0; j < kME; ++j) u[j] = bf16_to_f32(sr_bf16(u[j], rn.bits16(j)));
      } else if (gf == HB_FMT_F16) {
#pragma unroll
        for (int j = 0; j < kME; ++j) u[j] = f16_to_f32(f32_to_f16_rne(u[j]));
      }
      const bool state_rounds = MF == kDyn;  // bf16 storage rounds stochastically, ECC pairs draw their correction
      const Noise<kME> rn_m = state_rounds ? rng.noise<kME>(idx, HB_STREAM_EXP_AVG) : Noise<kME>{};
      raw_put<MF>(mf, m, rn_m, mom, mom_corr, idx);
      raw_put<HB_FMT_F32>(0, u, Noise<kME>{}, reinterpret_cast<char*>(upd), nullptr, idx);
      if (part) {
#pragma unroll
        for (int j = 0; j < kME; ++j)
          if (e + j < valid) ss += (double)u[j] * (double)u[j];
      }
    }
    if (part) {  // every lane of the wavefront is here: a wavefront-wide sum
      ss = wave_sum(ss);
      if ((threadIdx.x & 63) == 0) *part = ss;
    }
  }
}

}  // namespace hb

extern "C" int hb_momentum_sumsq_parts_per_chunk(void) { return hb::kMSub * (hb::kMThreads / 64); }

extern "C" int hb_momentum(void* momentum, void* momentum_corr, int32_t momentum_fmt, float* update, const void* grad,
                           const void* const* grad_ptrs, int32_t grad_fmt, const int64_t* offsets, const int64_t* numel, const int32_t* chunks,
                           int64_t n_chunks, int32_t mode, float a, float one_minus_a, int32_t rng_mode, uint64_t seed, uint32_t step,
                           void* stream_) {
  return hb_momentum_sumsq(momentum, momentum_corr, momentum_fmt, update, grad, grad_ptrs, grad_fmt, offsets, numel, chunks, n_chunks, mode, a,
                           one_minus_a, rng_mode, seed, step, nullptr, stream_);
}

extern "C" int hb_momentum_sumsq(void* momentum, void* momentum_corr, int32_t momentum_fmt, float* update, const void* grad,
                                 const void* const* grad_ptrs, int32_t grad_fmt, const int64_t* offsets, const int64_t* numel,
                                 const int32_t* chunks, int64_t n_chunks, int32_t mode, float a, float one_minus_a, int32_t rng_mode,
                                 uint64_t seed, uint32_t step, double* sumsq_parts, void* stream_) {
  using namespace hb;
  if (mode < HB_MOM_NESTEROV_EMA || mode > HB_MOM_NESTEROV_HEAVYBALL) return set_error(HB_EINVAL, "hb_momentum: bad mode");
  if (n_chunks < 0) return set_error(HB_EINVAL, "hb_momentum: negative size");
  if (n_chunks == 0) return HB_OK;
  if (!momentum || !update || !offsets || !numel || !chunks) return set_error(HB_EINVAL, "hb_momentum: null pointer");
  if ((grad == nullptr) == (grad_ptrs == nullptr)) return set_error(HB_EINVAL, "hb_momentum: exactly one of grad / grad_ptrs");
  if (grad_fmt != HB_FMT_F32 && grad_fmt != HB_FMT_BF16 && grad_fmt != HB_FMT_F16) return set_error(HB_EINVAL, "hb_momentum: bad grad_fmt");
  if (momentum_fmt < HB_FMT_F32 || momentum_fmt > HB_FMT_ECC_F16_16 || momentum_fmt == HB_FMT_F16)
    return set_error(HB_EINVAL, "hb_momentum: momentum is stored as float32, bfloat16 or an ECC pair");
  if (fmt_is_ecc(momentum_fmt) && !momentum_corr) return set_error(HB_EINVAL, "hb_momentum: ECC momentum needs its correction buffer");
  if (rng_mode != HB_RNG_HALF && rng_mode != HB_RNG_PHILOX) return set_error(HB_EINVAL, "hb_momentum: bad rng_mode");
  const int grid = persistent_grid(n_chunks * kMSub);
  if (grid <= 0) return set_error(HB_ELAUNCH, "could not query the device");
  Rng rng{(uint32_t)seed, (uint32_t)(seed >> 32), step, rng_mode};
  hipStream_t s = static_cast<hipStream_t>(stream_);
  char* m = static_cast<char*>(momentum);
  char* mc = static_cast<char*>(momentum_corr);
  const char* g = static_cast<const char*>(grad);
  const char* const* gp = reinterpret_cast<const char* const*>(grad_ptrs);
  const int2* ch = reinterpret_cast<const int2*>(chunks);
  if (momentum_fmt == HB_FMT_F32)
    momentum_kernel<HB_FMT_F32><<<grid, kMThreads, 0, s>>>(m, mc, momentum_fmt, update, g, gp, grad_fmt, offsets, numel, ch, n_chunks, a, one_minus_a, mode, rng,
                                                           sumsq_parts);
  else
    momentum_kernel<kDyn><<<grid, kMThreads, 0, s>>>(m, mc, momentum_fmt, update, g, gp, grad_fmt, offsets, numel, ch, n_chunks, a, one_minus_a, mode, rng,
                                                     sumsq_parts);
  return check_launch("hb_momentum");
}

extern "C" int hb_nesterov_ema(float* momentum, float* update, const void* grad, const void* const* grad_ptrs, int32_t grad_fmt,
                               const int64_t* offsets, const int64_t* numel, const int32_t* chunks, int64_t n_chunks, float a, float one_minus_a,
                               void* stream_) {
  return hb_momentum(momentum, nullptr, HB_FMT_F32, update, grad, grad_ptrs, grad_fmt, offsets, numel, chunks, n_chunks, HB_MOM_NESTEROV_EMA, a,
                     one_minus_a, HB_RNG_HALF, 0, 0, stream_);
}
