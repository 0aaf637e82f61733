// Per-tensor sum of squares over a slab (the reduction behind the clipping norms, heavyball/utils.py:3235-3297) and the
// matching in-place scale.  Two deterministic stages: each workgroup reduces one chunk (fp32 per lane over 16 elements,
// fp64 across lanes by wavefront shuffles, then across the 4 wavefronts through LDS) into partial[chunk]; a second
// kernel adds each tensor's partials in chunk order.  No atomics, so the result does not depend on scheduling.
#include "hb_device.h"
#include "hb_host.h"

namespace hb {

constexpr int kRThreads = 256;
constexpr int kRGroups = HB_CHUNK / (kRThreads * 8);

template <int F>
__global__ __launch_bounds__(kRThreads) void sumsq_chunk_kernel(const char* __restrict__ x, int f, const int64_t* __restrict__ offsets,
                                                                 const int64_t* __restrict__ numel, const int2* __restrict__ chunks,
                                                                 int64_t n_chunks, double* __restrict__ partial) {
  __shared__ double lds[kRThreads / kWave];
  for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
    const int2 ent = chunks[c];
    const int64_t local0 = (int64_t)ent.y * HB_CHUNK;
    const int64_t rem = numel[ent.x] - local0;
    const int valid = rem < HB_CHUNK ? (int)rem : HB_CHUNK;
    const int64_t flat0 = offsets[ent.x] + local0;
    float acc = 0.0f;
#pragma unroll
    for (int k = 0; k < kRGroups; ++k) {
      const int e = k * (kRThreads * 8) + threadIdx.x * 8;
      if (e < valid) {
        Raw r;
        float v[8];
        raw_load<F>(r, f, x, nullptr, flat0 + e);
        raw_decode<F>(r, f, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) acc += (e + j < valid) ? v[j] * v[j] : 0.0f;
      }
    }
    double s = wave_sum((double)acc);
    if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
      double tot = 0.0;
#pragma unroll
      for (int w = 0; w < kRThreads / kWave; ++w) tot += lds[w];
      partial[c] = tot;
    }
    __syncthreads();
  }
}

// The chunk list is sorted by tensor, so tensor t's partials are one contiguous run: find its bounds by bisection, then
// add them in chunk order (strided over the workgroup, combined in a fixed order).
__device__ __forceinline__ int64_t first_chunk_of(const int2* chunks, int64_t n_chunks, int t) {
  int64_t lo = 0, hi = n_chunks;
  while (lo < hi) {
    const int64_t mid = (lo + hi) >> 1;
    if (chunks[mid].x < t) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

__global__ void sumsq_final_kernel(const int2* __restrict__ chunks, int64_t n_chunks, int n_tensors, const double* __restrict__ partial,
                                   double* __restrict__ out) {
  const int t = blockIdx.x;
  __shared__ double lds[kWave];
  const int64_t begin = first_chunk_of(chunks, n_chunks, t);
  const int64_t end = first_chunk_of(chunks, n_chunks, t + 1);
  double acc = 0.0;
  for (int64_t c = begin + threadIdx.x; c < end; c += blockDim.x) acc += partial[c];
  acc = wave_sum(acc);
  if ((threadIdx.x & (kWave - 1)) == 0) lds[threadIdx.x / kWave] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double tot = 0.0;
    for (int w = 0; w < (int)(blockDim.x / kWave); ++w) tot += lds[w];
    out[t] = tot;
  }
}

__global__ __launch_bounds__(kRThreads) void scale_kernel(float* __restrict__ x, const float* __restrict__ scale, int per_tensor,
                                                           const int64_t* __restrict__ offsets, const int64_t* __restrict__ numel,
                                                           const int2* __restrict__ chunks, int64_t n_chunks) {
  for (int64_t c = blockIdx.x; c < n_chunks; c += gridDim.x) {
    const int2 ent = chunks[c];
    const int64_t local0 = (int64_t)ent.y * HB_CHUNK;
    const int64_t rem = numel[ent.x] - local0;
    const int valid = rem < HB_CHUNK ? (int)rem : HB_CHUNK;
    const int64_t flat0 = offsets[ent.x] + local0;
    const float s = scale[per_tensor ? ent.x : 0];
#pragma unroll
    for (int k = 0; k < kRGroups; ++k) {
      const int e = k * (kRThreads * 8) + threadIdx.x * 8;
      if (e < valid) {
        Raw r;
        float v[8];
        raw_load<HB_FMT_F32>(r, 0, reinterpret_cast<const char*>(x), nullptr, flat0 + e);
        raw_decode<HB_FMT_F32>(r, 0, v);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] *= s;
        Rand8 none{{0, 0, 0, 0}};
        raw_put<HB_FMT_F32>(0, v, none, reinterpret_cast<char*>(x), nullptr, flat0 + e);
      }
    }
  }
}

}  // namespace hb

extern "C" int hb_sumsq(const void* x, int32_t fmt, const int64_t* offsets, const int64_t* numel, const int32_t* chunks, int64_t n_chunks,
                        int32_t n_tensors, double* partial, double* out, void* stream_) {
  using namespace hb;
  if (n_chunks < 0 || n_tensors < 0) return set_error(HB_EINVAL, "hb_sumsq: negative sizes");
  if (n_tensors == 0) return HB_OK;
  if (!x || !offsets || !numel || !chunks || !partial || !out) return set_error(HB_EINVAL, "hb_sumsq: null pointer");
  if (fmt != HB_FMT_F32 && fmt != HB_FMT_BF16 && fmt != HB_FMT_F16) return set_error(HB_EINVAL, "hb_sumsq: plain formats only");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  const int2* ch = reinterpret_cast<const int2*>(chunks);
  if (n_chunks > 0) {
    const int grid = persistent_grid(n_chunks);
    if (grid <= 0) return set_error(HB_ELAUNCH, "could not query the device");
    const char* xc = static_cast<const char*>(x);
    if (fmt == HB_FMT_F32) sumsq_chunk_kernel<HB_FMT_F32><<<grid, kRThreads, 0, s>>>(xc, fmt, offsets, numel, ch, n_chunks, partial);
    else sumsq_chunk_kernel<kDyn><<<grid, kRThreads, 0, s>>>(xc, fmt, offsets, numel, ch, n_chunks, partial);
  }
  sumsq_final_kernel<<<n_tensors, 256, 0, s>>>(ch, n_chunks, n_tensors, partial, out);
  return check_launch("hb_sumsq");
}

extern "C" int hb_scale(float* x, const float* scale, int32_t per_tensor, const int64_t* offsets, const int64_t* numel, const int32_t* chunks,
                        int64_t n_chunks, void* stream_) {
  using namespace hb;
  if (n_chunks < 0) return set_error(HB_EINVAL, "hb_scale: negative size");
  if (n_chunks == 0) return HB_OK;
  if (!x || !scale || !offsets || !numel || !chunks) return set_error(HB_EINVAL, "hb_scale: null pointer");
  const int grid = persistent_grid(n_chunks);
  if (grid <= 0) return set_error(HB_ELAUNCH, "could not query the device");
  scale_kernel<<<grid, kRThreads, 0, static_cast<hipStream_t>(stream_)>>>(x, scale, per_tensor, offsets, numel,
                                                                           reinterpret_cast<const int2*>(chunks), n_chunks);
  return check_launch("hb_scale");
}
