// Fused AdamW / LaProp / ADOPT / AdEMAMix / NAdam optimizer step over a slab of tensors, for gfx950 (MI355X).
//
// One launch streams every operand once: parameter, gradient, exp_avg, exp_avg_sq (and mars_old_grad) are read as
// octets (8 consecutive elements per lane: one 128-bit load of a 16-bit role, two of an fp32 role, one 64-bit load
// of an int8 correction), decoded in registers, updated, re-encoded and written back.  The arithmetic follows the
// reference's eager op order (heavyball/utils.py:1921-1943 Adam, :2247-2269 LaProp, :2294-2304 ADOPT, :2086-2132
// AdEMAMix, :382-410 NAdam, :3616-3620 MARS, :3652-3658 caution, :2373-2390 update, :1288-1324 ECC) with one rounding
// per multiply/add (-ffp-contract=off), IEEE divide and sqrt, so fp32 results are bit-identical to the CPU path of
// the reference.
//
// Work decomposition: the slab is cut in chunks of HB_CHUNK elements that never span two tensors; one 256-thread
// workgroup per chunk (the grid-stride loop only matters when the chunk list is longer than the largest grid), so
// the dispatcher sweeps the slab as a compact moving window and neighbouring workgroups touch neighbouring DRAM
// pages at the same time.  Per chunk, 5 wave-uniform scalar loads fetch the tensor's offset, size and gradient
// pointer.
//
// Caution needs, per tensor, the number of masked elements before any parameter is written (the rescale multiplies
// the update ahead of the rounding of the parameter), so it runs in two launches: a count pass that recomputes the
// sign of the update from (g, m[, v]) without storing anything, then the full pass with the counts.
#include "fused_step_kernels.h"

namespace hb {

extern template StepKernel pick_algo<HB_ALGO_ADAM>(bool, int, int, int, int);
extern template StepKernel pick_algo<HB_ALGO_LAPROP>(bool, int, int, int, int);
extern template StepKernel pick_algo<HB_ALGO_ADOPT>(bool, int, int, int, int);
extern template StepKernel pick_algo<HB_ALGO_ADEMAMIX>(bool, int, int, int, int);
extern template StepKernel pick_algo<HB_ALGO_NADAM>(bool, int, int, int, int);

// chain()'s non-fused tail (heavyball/utils.py:2393-2406): the update is an fp32 slab (in a.m), optional caution
// against the gradient.  COUNT = 1 only counts masked elements.
constexpr int kUThreads = 256;                 // update_param_kernel: a lane owns kUE consecutive elements, a workgroup kUWork,
#ifndef HB_UPD_E
#define HB_UPD_E 4
#endif
constexpr int kUE = HB_UPD_E;                   // and a chunk is kUSub such work units (short runs per lane: see muon.hip)
constexpr int kUWork = kUThreads * kUE;
constexpr int kUSub = HB_CHUNK / kUWork;
static_assert(kUThreads == kThreads, "add_masked sizes its LDS words for kThreads lanes");
static_assert(kUSub * kUWork == HB_CHUNK && (kUE == 4 || kUE == 8), "a chunk is a whole number of work units");
template <int CAUTION, int PF>
__global__ __launch_bounds__(kUThreads) void update_param_kernel(const StepArgs a) {
  const int pf = PF == kDyn ? a.pf : PF;
  constexpr bool kCount = CAUTION == kCautionCount;
  const bool cautious_wd = (a.flags & HB_FLAG_CAUTIOUS_WD) != 0;
  for (int64_t w = blockIdx.x; w < a.n_chunks * kUSub; w += gridDim.x) {
    const int2 ent = a.chunks[w / kUSub];
    const int t = ent.x;
    const int64_t off = a.offsets[t];
    const int64_t n = a.numel[t];
    const int64_t local0 = (int64_t)ent.y * HB_CHUNK + (int64_t)(w % kUSub) * kUWork;
    const int64_t rem = n - local0;
    if (rem <= 0) continue;  // a work unit behind the end of the tensor's last chunk
    const int valid = rem < kUWork ? (int)rem : kUWork;
    const int64_t flat0 = off + local0;
    const bool g_slab = a.grad_ptrs == nullptr;
    const char* gbase = CAUTION != kNoCaution ? (g_slab ? a.grad : a.grad_ptrs[t]) : nullptr;
    const int64_t g0 = g_slab ? flat0 : local0;
    float scale = 1.0f;
    if (CAUTION == kCautionApply) {
      const int64_t kept = n - masked_of(a.counts, t);
      scale = (1.0f / (float)(kept < 1 ? 1 : kept)) * (float)n;  // reciprocal(kept) * numel, as in the fused step
    }
    uint32_t masked = 0;
    const int e = threadIdx.x * kUE;
    if (e < valid) {
      const int64_t idx = flat0 + e;
      RawT<kUE> ru, rp;
      float u[kUE], p[kUE], g[kUE];
      if (a.sf == HB_FMT_BF16) raw_load<HB_FMT_BF16>(ru, HB_FMT_BF16, a.m, nullptr, idx);  // the update as a bf16 slab
      else raw_load<HB_FMT_F32>(ru, HB_FMT_F32, a.m, nullptr, idx);
      if (!kCount) raw_load<PF>(rp, pf, a.param, a.param_corr, idx);
      if (CAUTION != kNoCaution) {
#pragma unroll
        for (int j = 0; j < kUE; ++j) g[j] = e + j < valid ? load_elem(gbase, a.gf, g0 + e + j) : 0.0f;
      }
      if (a.sf == HB_FMT_BF16) raw_decode<HB_FMT_BF16>(ru, HB_FMT_BF16, u);
      else raw_decode<HB_FMT_F32>(ru, HB_FMT_F32, u);
      if (!kCount) raw_decode<PF>(rp, pf, p);
#pragma unroll
      for (int j = 0; j < kUE; ++j) {
        if (CAUTION != kNoCaution) {
          const bool mk = ((f2u(g[j]) ^ f2u(u[j])) >> 31) != 0;
          if (kCount) masked += (mk && e + j < valid) ? 1u : 0u;
          else u[j] = (mk ? 0.0f : u[j]) * scale;
        }
        if (!kCount) {
          float om = a.omdl;
          if (cautious_wd && ((f2u(p[j]) ^ f2u(u[j])) >> 31)) om = 1.0f;
          p[j] = p[j] * om + u[j] * a.neg_lr;
        }
      }
      if (!kCount) {
        const Noise<kUE> rn = pf != HB_FMT_F32 ? a.rng.noise<kUE>(idx, HB_STREAM_PARAM) : Noise<kUE>{};
        raw_put<PF>(pf, p, rn, a.param, a.param_corr, idx);
      }
    }
    if (kCount) add_masked(a.counts, t, (int)(w & (HB_CAUTION_SLOTS - 1)), masked);
  }
}

__global__ void zero_u32_kernel(uint32_t* p, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0;
}

// -----------------------------------------------------------------------------------------------------------
// host side
// -----------------------------------------------------------------------------------------------------------
static StepKernel pick_kernel(int algo, bool mars, int caution, int pf, int gf, int sf) {
  switch (algo) {
    case HB_ALGO_ADAM: return pick_algo<HB_ALGO_ADAM>(mars, caution, pf, gf, sf);
    case HB_ALGO_LAPROP: return pick_algo<HB_ALGO_LAPROP>(mars, caution, pf, gf, sf);
    case HB_ALGO_ADOPT: return pick_algo<HB_ALGO_ADOPT>(mars, caution, pf, gf, sf);
    case HB_ALGO_ADEMAMIX: return pick_algo<HB_ALGO_ADEMAMIX>(mars, caution, pf, gf, sf);
    default: return pick_algo<HB_ALGO_NADAM>(mars, caution, pf, gf, sf);
  }
}

static bool fmt_ok_state(int f) { return f == HB_FMT_F32 || f == HB_FMT_BF16 || fmt_is_ecc(f); }
static bool fmt_ok_grad(int f) { return f == HB_FMT_F32 || f == HB_FMT_BF16 || f == HB_FMT_F16; }
static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int fill_args(const HbStepDesc* d, StepArgs& a, bool need_states, bool need_counts = true) {
  if (!d) return set_error(HB_EINVAL, "null descriptor");
  if (d->n_chunks < 0 || d->n_tensors < 0) return set_error(HB_EINVAL, "negative sizes");
  if (!d->offsets || !d->numel || !d->chunks) return set_error(HB_EINVAL, "offsets, numel and chunks are required");
  if (!fmt_ok_state(d->param_fmt) || d->param_fmt > HB_FMT_ECC_F16_16) return set_error(HB_EINVAL, "bad param_fmt");
  if (!d->param || !aligned16(d->param)) return set_error(HB_EINVAL, "param must be a 16-byte aligned device pointer");
  if (fmt_is_ecc(d->param_fmt) && (!d->param_corr || !aligned16(d->param_corr)))
    return set_error(HB_EINVAL, "param_corr required (16-byte aligned) for an ECC param_fmt");
  const bool caution = (d->flags & HB_FLAG_CAUTION) != 0;
  if ((d->flags & HB_FLAG_UPDATE_ONLY) && (caution || (d->update_out == nullptr && d->param_fmt != HB_FMT_F32) ||
                                           (d->update_out != nullptr && !aligned16(d->update_out))))
    return set_error(HB_EINVAL, "HB_FLAG_UPDATE_ONLY writes an fp32 update slab (update_out, or param with param_fmt F32) and takes no caution flag");
  if ((d->flags & HB_FLAG_MARS_ONLY) && (!(d->flags & HB_FLAG_MARS) || caution || d->param_fmt != HB_FMT_F32 || !need_states))
    return set_error(HB_EINVAL, "HB_FLAG_MARS_ONLY goes with HB_FLAG_MARS, writes an fp32 slab and takes no caution flag");
  const bool need_grad = need_states || caution;
  if (need_grad) {
    if (!fmt_ok_grad(d->grad_fmt)) return set_error(HB_EINVAL, "bad grad_fmt");
    if ((d->grad == nullptr) == (d->grad_ptrs == nullptr)) return set_error(HB_EINVAL, "exactly one of grad / grad_ptrs must be set");
    if (d->grad && !aligned16(d->grad)) return set_error(HB_EINVAL, "grad slab must be 16-byte aligned");
  }
  if (caution && need_counts && !d->caution_count) return set_error(HB_EINVAL, "caution_count scratch required with HB_FLAG_CAUTION");
  if (need_states) {
    if (d->algo < HB_ALGO_ADAM || d->algo > HB_ALGO_NADAM) return set_error(HB_EINVAL, "bad algo");
    if ((d->flags & HB_FLAG_ADOPT_WARMUP) && (d->algo != HB_ALGO_ADOPT || caution || (d->flags & HB_FLAG_UPDATE_ONLY)))
      return set_error(HB_EINVAL, "HB_FLAG_ADOPT_WARMUP goes with HB_ALGO_ADOPT alone and takes no caution");
    if ((d->flags & HB_FLAG_COUPLED_WD) && d->algo != HB_ALGO_NADAM) return set_error(HB_EINVAL, "HB_FLAG_COUPLED_WD goes with HB_ALGO_NADAM");
    if ((d->flags & HB_FLAG_UPDATE_ONLY) && (d->flags & HB_FLAG_COUPLED_WD) && d->update_out == nullptr)
      return set_error(HB_EINVAL, "HB_FLAG_UPDATE_ONLY with HB_FLAG_COUPLED_WD reads the parameters: give the update its own slab in update_out");
    if (d->algo == HB_ALGO_NADAM && !d->tensor_scalars) return set_error(HB_EINVAL, "tensor_scalars required with HB_ALGO_NADAM");
    if (!fmt_ok_state(d->state_fmt) || d->state_fmt > HB_FMT_ECC_F16_16) return set_error(HB_EINVAL, "bad state_fmt");
    const bool ecc = fmt_is_ecc(d->state_fmt);
    const bool mars_only = (d->flags & HB_FLAG_MARS_ONLY) != 0;
    if (!mars_only && (!d->exp_avg || !d->exp_avg_sq || !aligned16(d->exp_avg) || !aligned16(d->exp_avg_sq)))
      return set_error(HB_EINVAL, "exp_avg / exp_avg_sq must be 16-byte aligned device pointers");
    if (!mars_only && ecc && (!d->exp_avg_corr || !d->exp_avg_sq_corr || !aligned16(d->exp_avg_corr) || !aligned16(d->exp_avg_sq_corr)))
      return set_error(HB_EINVAL, "state corrections required (16-byte aligned) for an ECC state_fmt");
    if (d->algo == HB_ALGO_ADEMAMIX && !mars_only) {
      if (!d->exp_avg_slow || !aligned16(d->exp_avg_slow)) return set_error(HB_EINVAL, "exp_avg_slow required with HB_ALGO_ADEMAMIX");
      if (ecc && (!d->exp_avg_slow_corr || !aligned16(d->exp_avg_slow_corr))) return set_error(HB_EINVAL, "exp_avg_slow_corr required");
    }
    if (d->flags & HB_FLAG_MARS) {
      if (!d->old_grad || !aligned16(d->old_grad)) return set_error(HB_EINVAL, "old_grad required with HB_FLAG_MARS");
      if (ecc && (!d->old_grad_corr || !aligned16(d->old_grad_corr))) return set_error(HB_EINVAL, "old_grad_corr required");
    }
  } else if (!d->exp_avg || !aligned16(d->exp_avg) || (d->state_fmt != HB_FMT_F32 && d->state_fmt != HB_FMT_BF16)) {
    return set_error(HB_EINVAL, "hb_update_param reads the update from exp_avg, an fp32 or (state_fmt HB_FMT_BF16) bf16 slab");
  }
  if (d->rng_mode != HB_RNG_HALF && d->rng_mode != HB_RNG_PHILOX) return set_error(HB_EINVAL, "bad rng_mode");
  a.param = static_cast<char*>(d->param);
  a.param_corr = static_cast<char*>(d->param_corr);
  a.grad = static_cast<const char*>(d->grad);
  a.grad_ptrs = reinterpret_cast<const char* const*>(d->grad_ptrs);
  a.m = static_cast<char*>(d->exp_avg);
  a.m_corr = static_cast<char*>(d->exp_avg_corr);
  a.v = static_cast<char*>(d->exp_avg_sq);
  a.v_corr = static_cast<char*>(d->exp_avg_sq_corr);
  a.og = static_cast<char*>(d->old_grad);
  a.og_corr = static_cast<char*>(d->old_grad_corr);
  a.s3 = static_cast<char*>(d->exp_avg_slow);
  a.s3_corr = static_cast<char*>(d->exp_avg_slow_corr);
  a.tscal = d->tensor_scalars;
  a.upd = static_cast<char*>(d->update_out);
  a.offsets = d->offsets;
  a.numel = d->numel;
  a.chunks = reinterpret_cast<const int2*>(d->chunks);
  a.counts = d->caution_count;
  a.n_chunks = d->n_chunks;
  a.pf = d->param_fmt;
  a.gf = d->grad_fmt;
  a.sf = d->state_fmt;
  a.flags = d->flags;
  a.a1 = d->a1;
  a.oma1 = d->one_minus_a1;
  a.a2 = d->a2;
  a.oma2 = d->one_minus_a2;
  a.amars = d->mars_a;
  a.omamars = d->one_minus_mars_a;
  a.neg_lr = d->neg_lr;
  a.omdl = d->one_minus_decay_lr;
  a.eps = d->eps;
  a.a3 = d->a3;
  a.oma3 = d->one_minus_a3;
  a.alpha = d->alpha;
  a.wd = d->coupled_wd;
  a.rng = Rng{(uint32_t)d->seed, (uint32_t)(d->seed >> 32), d->step, d->rng_mode};
  return HB_OK;
}

}  // namespace hb

namespace hb {

// Both entry points of the fused step.  `counts`: the per-tensor caution counters the two caution launches share
// (zeroed here by a fill kernel, not by hipMemsetAsync, so that a caller may capture the call in a graph).
static int run_fused_step(const HbStepDesc* d, StepArgs& a, uint32_t* counts, hipStream_t stream, const char* what) {
  const bool mars = (d->flags & HB_FLAG_MARS) != 0;
  const bool caution = (d->flags & HB_FLAG_CAUTION) != 0;
  a.counts = counts;
  auto launch = [&](int pass) {
    const StepKernel k = pick_kernel(d->algo, mars, pass, a.pf, a.gf, a.sf);
    const int grid = persistent_grid(d->n_chunks * k.sub);
    if (grid <= 0) return false;
    k.fn<<<grid, kThreads, 0, stream>>>(a);
    return true;
  };
  bool ok;
  if (caution) {
    zero_u32_kernel<<<(d->n_tensors * HB_CAUTION_SLOTS + 255) / 256, 256, 0, stream>>>(counts, d->n_tensors * HB_CAUTION_SLOTS);
    ok = launch(kCautionCount) && launch(kCautionApply);
  } else {
    ok = launch(kNoCaution);
  }
  if (!ok) return set_error(HB_ELAUNCH, "could not query the device");
  return check_launch(what);
}

// Scratch of hb_fused_step_noalloc: the caution counters live in the library's own device memory.  Every device the
// library runs on holds its own copy of this array at its own address, for the life of the process.
static __device__ __align__(256) uint32_t scratch[HB_NOALLOC_MAX_TENSORS * HB_CAUTION_SLOTS];

constexpr int kMaxDevices = 64;
static std::atomic<uint32_t*> g_scratch_ptr[kMaxDevices];  // device address of `scratch` per device, resolved once

// The device address of `scratch` on the current device.  The array's name is only a host-side handle: what kernels
// and fills are given is the address hipGetSymbolAddress reports for the device that is current.
static int scratch_of_current_device(uint32_t** out) {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return set_error(HB_ELAUNCH, "hb_fused_step_noalloc: no current device");
  uint32_t* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return set_error(HB_ELAUNCH, "hb_fused_step_noalloc: hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);  // concurrent first calls resolve the same address
  }
  *out = ptr;
  return HB_OK;
}

}  // namespace hb

extern "C" int hb_fused_step(const HbStepDesc* d, void* stream_) {
  using namespace hb;
  StepArgs a;
  if (int rc = fill_args(d, a, true, true)) return rc;
  if (d->n_chunks == 0) return HB_OK;
  return run_fused_step(d, a, d->caution_count, static_cast<hipStream_t>(stream_), "hb_fused_step");
}

extern "C" int hb_fused_step_noalloc(const HbStepDesc* d, void* stream_) {
  using namespace hb;
  StepArgs a;
  if (int rc = fill_args(d, a, true, false)) return rc;
  if (d->n_tensors > HB_NOALLOC_MAX_TENSORS)
    return set_error(HB_EINVAL, "hb_fused_step_noalloc: %d tensors, the built-in scratch holds counters for at most %d", d->n_tensors,
                     HB_NOALLOC_MAX_TENSORS);
  if (d->n_chunks == 0) return HB_OK;
  uint32_t* counts = nullptr;
  if (int rc = scratch_of_current_device(&counts)) return rc;
  return run_fused_step(d, a, counts, static_cast<hipStream_t>(stream_), "hb_fused_step_noalloc");
}

extern "C" int hb_update_param(const HbStepDesc* d, void* stream_) {
  using namespace hb;
  StepArgs a;
  if (int rc = fill_args(d, a, false)) return rc;
  if (d->n_chunks == 0) return HB_OK;
  hipStream_t stream = static_cast<hipStream_t>(stream_);
  const bool caution = (d->flags & HB_FLAG_CAUTION) != 0;
  const int grid = persistent_grid(d->n_chunks * kUSub);
  if (grid <= 0) return set_error(HB_ELAUNCH, "could not query the device");
  if (caution) {
    zero_u32_kernel<<<(d->n_tensors * HB_CAUTION_SLOTS + 255) / 256, 256, 0, stream>>>(d->caution_count, d->n_tensors * HB_CAUTION_SLOTS);
    update_param_kernel<kCautionCount, kDyn><<<grid, kUThreads, 0, stream>>>(a);
    update_param_kernel<kCautionApply, kDyn><<<grid, kUThreads, 0, stream>>>(a);
  } else if (a.pf == HB_FMT_F32) {
    update_param_kernel<kNoCaution, HB_FMT_F32><<<grid, kUThreads, 0, stream>>>(a);
  } else {
    update_param_kernel<kNoCaution, kDyn><<<grid, kUThreads, 0, stream>>>(a);
  }
  return check_launch("hb_update_param");
}
