// Test hooks for the ECC codec, bf16 stochastic rounding and the Philox stream: the same device functions the fused
// step uses, on flat arrays, so that the codec can be compared bit for bit with the CPU oracle in isolation
// (heavyball/utils.py:1288-1324, :2341-2355).
#include "hb_device.h"
#include "hb_host.h"

namespace hb {

template <bool PRIM_BF16, bool CORR8>
__global__ void ecc_encode_kernel(const float* __restrict__ src, uint16_t* __restrict__ prim, void* __restrict__ corr,
                                  int64_t n, Rng rng, uint32_t stream_id, int64_t flat_base) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t flat = flat_base + i;
    const Rand8 r = rng.octet(flat & ~int64_t(7), stream_id);
    uint32_t h;
    int c;
    ecc_encode<PRIM_BF16, CORR8>(src[i], r.bits16((int)(flat & 7)), h, c);
    prim[i] = (uint16_t)h;
    if (CORR8) static_cast<int8_t*>(corr)[i] = (int8_t)c;
    else static_cast<int16_t*>(corr)[i] = (int16_t)c;
  }
}

template <bool PRIM_BF16, bool CORR8>
__global__ void ecc_decode_kernel(const uint16_t* __restrict__ prim, const void* __restrict__ corr, float* __restrict__ dst, int64_t n) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int c = CORR8 ? (int)static_cast<const int8_t*>(corr)[i] : (int)static_cast<const int16_t*>(corr)[i];
    dst[i] = ecc_decode<PRIM_BF16, CORR8>(prim[i], c);
  }
}

__global__ void sr_bf16_kernel(const float* __restrict__ src, uint16_t* __restrict__ dst, int64_t n, Rng rng, uint32_t stream_id, int64_t flat_base) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t flat = flat_base + i;
    const Rand8 r = rng.octet(flat & ~int64_t(7), stream_id);
    dst[i] = (uint16_t)sr_bf16(src[i], r.bits16((int)(flat & 7)));
  }
}

__global__ void philox_words_kernel(uint32_t* out, int64_t n, uint64_t q0, Rng rng, uint32_t stream_id) {
  for (int64_t i = blockIdx.x * (int64_t)blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const Rand8 r = rng.mode == HB_RNG_PHILOX ? rng.call((int64_t)((q0 + (uint64_t)i) << 2), stream_id)
                                               : Rand8{{0x80008000u, 0x80008000u, 0x80008000u, 0x80008000u}};
    out[4 * i + 0] = r.w[0];
    out[4 * i + 1] = r.w[1];
    out[4 * i + 2] = r.w[2];
    out[4 * i + 3] = r.w[3];
  }
}

// plain 16-byte copy of known size: the yardstick that the FETCH_SIZE / WRITE_SIZE counters are scaled against
__global__ __launch_bounds__(256) void copy_probe_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst, int64_t n16) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n16) dst[i] = src[i];
}

static int flat_grid(int64_t n) {
  int64_t b = (n + 255) / 256;
  return (int)(b < 1 ? 1 : (b > 65536 ? 65536 : b));
}

}  // namespace hb

extern "C" int hb_ecc_encode(const float* src, void* primary, void* corr, int64_t n, int32_t fmt, int32_t rng_mode, uint64_t seed,
                             uint32_t step, uint32_t stream_id, int64_t flat_base, void* stream_) {
  using namespace hb;
  if (n < 0 || !fmt_is_ecc(fmt) || fmt > HB_FMT_ECC_F16_16) return set_error(HB_EINVAL, "hb_ecc_encode: bad size or format");
  if (n == 0) return HB_OK;
  if (!src || !primary || !corr) return set_error(HB_EINVAL, "hb_ecc_encode: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  Rng rng{(uint32_t)seed, (uint32_t)(seed >> 32), step, rng_mode};
  uint16_t* p = static_cast<uint16_t*>(primary);
  const int g = flat_grid(n);
  switch (fmt) {
    case HB_FMT_ECC_BF16_8: ecc_encode_kernel<true, true><<<g, 256, 0, s>>>(src, p, corr, n, rng, stream_id, flat_base); break;
    case HB_FMT_ECC_BF16_16: ecc_encode_kernel<true, false><<<g, 256, 0, s>>>(src, p, corr, n, rng, stream_id, flat_base); break;
    case HB_FMT_ECC_F16_8: ecc_encode_kernel<false, true><<<g, 256, 0, s>>>(src, p, corr, n, rng, stream_id, flat_base); break;
    default: ecc_encode_kernel<false, false><<<g, 256, 0, s>>>(src, p, corr, n, rng, stream_id, flat_base); break;
  }
  return check_launch("hb_ecc_encode");
}

extern "C" int hb_ecc_decode(const void* primary, const void* corr, float* dst, int64_t n, int32_t fmt, void* stream_) {
  using namespace hb;
  if (n < 0 || !fmt_is_ecc(fmt) || fmt > HB_FMT_ECC_F16_16) return set_error(HB_EINVAL, "hb_ecc_decode: bad size or format");
  if (n == 0) return HB_OK;
  if (!dst || !primary || !corr) return set_error(HB_EINVAL, "hb_ecc_decode: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  const uint16_t* p = static_cast<const uint16_t*>(primary);
  const int g = flat_grid(n);
  switch (fmt) {
    case HB_FMT_ECC_BF16_8: ecc_decode_kernel<true, true><<<g, 256, 0, s>>>(p, corr, dst, n); break;
    case HB_FMT_ECC_BF16_16: ecc_decode_kernel<true, false><<<g, 256, 0, s>>>(p, corr, dst, n); break;
    case HB_FMT_ECC_F16_8: ecc_decode_kernel<false, true><<<g, 256, 0, s>>>(p, corr, dst, n); break;
    default: ecc_decode_kernel<false, false><<<g, 256, 0, s>>>(p, corr, dst, n); break;
  }
  return check_launch("hb_ecc_decode");
}

extern "C" int hb_sr_bf16(const float* src, void* dst, int64_t n, int32_t rng_mode, uint64_t seed, uint32_t step, uint32_t stream_id,
                          int64_t flat_base, void* stream_) {
  using namespace hb;
  if (n < 0) return set_error(HB_EINVAL, "hb_sr_bf16: negative size");
  if (n == 0) return HB_OK;
  if (!src || !dst) return set_error(HB_EINVAL, "hb_sr_bf16: null pointer");
  Rng rng{(uint32_t)seed, (uint32_t)(seed >> 32), step, rng_mode};
  sr_bf16_kernel<<<flat_grid(n), 256, 0, static_cast<hipStream_t>(stream_)>>>(src, static_cast<uint16_t*>(dst), n, rng, stream_id, flat_base);
  return check_launch("hb_sr_bf16");
}

extern "C" int hb_philox_words(uint32_t* out, int64_t n, uint64_t q0, uint64_t seed, uint32_t step, uint32_t stream_id, void* stream_) {
  using namespace hb;
  if (n < 0) return set_error(HB_EINVAL, "hb_philox_words: negative size");
  if (n == 0) return HB_OK;
  if (!out) return set_error(HB_EINVAL, "hb_philox_words: null pointer");
  Rng rng{(uint32_t)seed, (uint32_t)(seed >> 32), step, HB_RNG_PHILOX};
  philox_words_kernel<<<flat_grid(n), 256, 0, static_cast<hipStream_t>(stream_)>>>(out, n, q0, rng, stream_id);
  return check_launch("hb_philox_words");
}

extern "C" int hb_copy_probe(const void* src, void* dst, int64_t nbytes, void* stream_) {
  using namespace hb;
  if (nbytes < 0 || (nbytes & 15) || !src || !dst) return set_error(HB_EINVAL, "hb_copy_probe: size must be a non-negative multiple of 16");
  const int64_t n16 = nbytes / 16;
  if (n16 == 0) return HB_OK;
  if ((n16 + 255) / 256 > 0x7FFFFFFF) return set_error(HB_EINVAL, "hb_copy_probe: too large");
  copy_probe_kernel<<<(unsigned)((n16 + 255) / 256), 256, 0, static_cast<hipStream_t>(stream_)>>>(static_cast<const uint4*>(src), static_cast<uint4*>(dst), n16);
  return check_launch("hb_copy_probe");
}
