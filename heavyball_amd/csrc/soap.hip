// SOAP on gfx950: fp32 MFMA GEMM for the eigenbasis projections and the factor EMAs, and Adam in the rotated basis.
//
// Reference: project (heavyball/utils.py:1391-1411: Ql^T G Qr and Ql P Qr^T as two chained products), update_ggt
// (:1205-1221: GG <- GG*(1-a) + (G G^T | G^T G)*a, the lerp of :1048 fused into the product's epilogue), the products
// inside get_orthogonal_matrix_QR (:829-900) and _compilable_adam_ (:1852-1868).
//
// GEMM: C[M,N] = op(A) op(B) in fp32 on v_mfma_f32_32x32x2_f32 (true fp32 multiply-accumulate).  Workgroup tile
// 128 x 128 x 16, four wavefronts (2 x 2), each 64 x 64 as 2 x 2 MFMA tiles.  Both operand tiles sit in LDS k-major
// ([k][row], row stride 132 floats), so the single-float MFMA fragments are read by 32 consecutive lanes from 32
// consecutive words whichever way the operand lies in memory; operands that are k-contiguous in memory are transposed
// on their way into LDS (the 4-word pad keeps those scattered stores conflict free).  Global loads of tile t+1 are
// staged in registers while tile t is multiplied.  Any M, N, K and leading dimensions: edges are predicated.
#include <stdlib.h>

#include "hb_device.h"
#include "hb_host.h"

namespace hb {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kGM = 128, kGN = 128, kGK = 16, kGLD = 132, kGThreads = 256;

struct SgemmArgs {
  const float* A;
  const float* B;
  float* C;
  int M, N, K, lda, ldb, ldc;
  int accumulate;
  float alpha_acc, beta_c;
  int k_chunk;   // split-K: workgroup (x, y) multiplies k in [y * k_chunk, (y + 1) * k_chunk); a multiple of the k-tile
  float* part;   // split-K: raw partial products [gridDim.y][M][N]; null for a plain launch
  int sym;       // symmetric output (A A^T or A^T A, M == N a multiple of 256): the big-tile kernel takes the 256 x 256 tiles
                 // strictly above the diagonal, the 128 x 128 kernel the three upper tiles of every diagonal 256 x 256 block,
                 // and every off-diagonal tile is also stored transposed
};

// Several problems of one shape in one launch (the batched orthonormalisation): the arguments describe problem 0 and
// problem z = blockIdx.z differs only in where its matrix and its workspace lie, so every operand moves by the byte
// distance of its home (matrix or workspace) from that of problem 0.  n <= 1: a plain launch.
constexpr int kMaxBatch = HB_ORTHO_MAX_BATCH;  // Batch travels as a kernel argument beside the product's own (1.6 of 4 KiB)
struct Batch {
  int n;
  int64_t dq[kMaxBatch];    // byte distance of matrix z from matrix 0
  int64_t dws[kMaxBatch];   // byte distance of workspace z from workspace 0
  int* status[kMaxBatch];   // status word of problem z
};
enum { kAInWs = 1, kBInWs = 2, kCInWs = 4 };  // which operands of a GEMM live in the workspace (the others in the matrix)
template <class T>
__device__ __forceinline__ T* shifted(T* p, int64_t bytes) {
  return reinterpret_cast<T*>(reinterpret_cast<uintptr_t>(p) + bytes);
}

typedef float f32x4 __attribute__((ext_vector_type(4)));  // a native vector: stays in registers where arrays of HIP's float4 struct end up in scratch

// One of the two float4 a thread holds of a (rows x 16) operand tile (q = 0, 1), with every edge predicated.
// KMAJOR: memory is [k][row] (row contiguous); otherwise [row][k] (k contiguous).
template <bool KMAJOR>
__device__ __forceinline__ f32x4 sgemm_load(const float* __restrict__ P, int ld, int row0, int k0, int rows, int K, int q) {
  const int idx = threadIdx.x + q * kGThreads;
  f32x4 v = {0.0f, 0.0f, 0.0f, 0.0f};
  if (KMAJOR) {
    const int k = k0 + idx / 32, c = row0 + (idx % 32) * 4;
    if (k < K) {
      const float* p = P + (size_t)k * ld + c;
      if (c + 3 < rows && ((reinterpret_cast<uintptr_t>(p) & 15) == 0)) {
        v = *reinterpret_cast<const f32x4*>(p);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (c + e < rows) v[e] = p[e];
      }
    }
  } else {
    const int row = row0 + idx / 4, k = k0 + (idx % 4) * 4;
    if (row < rows) {
      const float* p = P + (size_t)row * ld + k;
      if (k + 3 < K && ((reinterpret_cast<uintptr_t>(p) & 15) == 0)) {
        v = *reinterpret_cast<const f32x4*>(p);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (k + e < K) v[e] = p[e];
      }
    }
  }
  return v;
}

template <bool KMAJOR>
__device__ __forceinline__ void sgemm_store(float* __restrict__ S, const f32x4 r, int q) {
  const int idx = threadIdx.x + q * kGThreads;
  if (KMAJOR) {
    *reinterpret_cast<f32x4*>(S + (idx / 32) * kGLD + (idx % 32) * 4) = r;
  } else {
    const int row = idx / 4, k = (idx % 4) * 4;
    S[(k + 0) * kGLD + row] = r[0];
    S[(k + 1) * kGLD + row] = r[1];
    S[(k + 2) * kGLD + row] = r[2];
    S[(k + 3) * kGLD + row] = r[3];
  }
}

typedef float float2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t lds_addr(const float* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) float*)p;
}
// rows r and r + 32 of one k-row of an operand tile: the two single-float fragments of a wavefront's two MFMA tiles
__device__ __forceinline__ float2v lds_read2_f32(uint32_t addr) {
  float2v v;
  asm volatile("ds_read2_b32 %0, %1 offset1:32" : "=v"(v) : "v"(addr));
  return v;
}

// Interior tiles (the whole 128 x 128 x k-range block inside the matrices, 16-byte aligned rows): the same two float4
// per thread without any predication; `p` points at the thread's first element of the current k-tile.
template <bool KMAJOR>
__device__ __forceinline__ const float* sgemm_fast_ptr(const float* __restrict__ P, int ld, int row0, int k0) {
  const int tid = threadIdx.x;
  return KMAJOR ? P + (size_t)(k0 + tid / 32) * ld + row0 + (tid % 32) * 4 : P + (size_t)(row0 + tid / 4) * ld + k0 + (tid % 4) * 4;
}
template <bool KMAJOR>
__device__ __forceinline__ f32x4 sgemm_fast_load(const float* __restrict__ p, int ld, int q) {
  // the second float4 belongs to thread id + 256: 8 k-rows further (k-major) or 64 rows further
  return *reinterpret_cast<const f32x4*>(p + (size_t)(q ? (KMAJOR ? 8 : 64) : 0) * ld);
}

// The k-loop of one workgroup.  FAST: interior tile, no predication.  Per k-tile: issue the global loads of the next
// tile, multiply the current one out of LDS (the fragments of k-step s+1 are fetched while step s is multiplied), then
// park the staged registers in the other LDS buffer; one barrier per k-tile.
template <bool TA, bool TB, bool FAST>
__device__ __forceinline__ void sgemm_mainloop(const SgemmArgs& g, float (*As)[kGK * kGLD], float (*Bs)[kGK * kGLD], int row0, int col0, int kb,
                                               int ke, floatx16 (&acc)[2][2]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  f32x4 ra0, ra1, rb0, rb1;  // the next k-tile on its way from memory to LDS
  const int KT = (ke - kb + kGK - 1) / kGK;
  const float* pa = nullptr;
  const float* pb = nullptr;
  const size_t step_a = TA ? (size_t)kGK * g.lda : (size_t)kGK, step_b = !TB ? (size_t)kGK * g.ldb : (size_t)kGK;
  // A is k-major in memory exactly when it is given transposed, B exactly when it is NOT
#define HB_SG_LOAD(k0)                                                                                                   \
  if (FAST) {                                                                                                            \
    ra0 = sgemm_fast_load<TA>(pa, g.lda, 0), ra1 = sgemm_fast_load<TA>(pa, g.lda, 1);                                    \
    rb0 = sgemm_fast_load<!TB>(pb, g.ldb, 0), rb1 = sgemm_fast_load<!TB>(pb, g.ldb, 1);                                  \
  } else {                                                                                                               \
    ra0 = sgemm_load<TA>(g.A, g.lda, row0, (k0), g.M, ke, 0), ra1 = sgemm_load<TA>(g.A, g.lda, row0, (k0), g.M, ke, 1);   \
    rb0 = sgemm_load<!TB>(g.B, g.ldb, col0, (k0), g.N, ke, 0), rb1 = sgemm_load<!TB>(g.B, g.ldb, col0, (k0), g.N, ke, 1); \
  }
#define HB_SG_STORE(buf) \
  sgemm_store<TA>(As[buf], ra0, 0), sgemm_store<TA>(As[buf], ra1, 1), sgemm_store<!TB>(Bs[buf], rb0, 0), sgemm_store<!TB>(Bs[buf], rb1, 1)
  if (FAST) {
    pa = sgemm_fast_ptr<TA>(g.A, g.lda, row0, kb);
    pb = sgemm_fast_ptr<!TB>(g.B, g.ldb, col0, kb);
  }
  HB_SG_LOAD(kb)
  HB_SG_STORE(0);
  __syncthreads();
  const int fr = lane & 31, fk = lane >> 5;
  for (int kt = 0; kt < KT; ++kt) {
    if (kt + 1 < KT) {
      if (FAST) {
        pa += step_a;
        pb += step_b;
      }
      HB_SG_LOAD(kb + (kt + 1) * kGK)
    }
    // fragment reads through inline assembly with explicit waits: left to itself the compiler fetches each k-step's
    // fragments right before its matrix instructions and waits for them, one LDS round trip per k-step
    const uint32_t a = lds_addr(As[kt & 1] + wm * 64 + fr + fk * kGLD);
    const uint32_t b = lds_addr(Bs[kt & 1] + wn * 64 + fr + fk * kGLD);
    float2v af[2], bf[2];
    af[0] = lds_read2_f32(a);
    bf[0] = lds_read2_f32(b);
#pragma unroll
    for (int ks = 0; ks < kGK / 2; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < kGK / 2) {
        af[nxt] = lds_read2_f32(a + (ks + 1) * 2 * kGLD * 4);
        bf[nxt] = lds_read2_f32(b + (ks + 1) * 2 * kGLD * 4);
        __builtin_amdgcn_s_waitcnt(0xC07F | (2 << 8));  // lgkmcnt(2): this step's pair has landed, the next may be in flight
      } else {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][i], bf[cur][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kt + 1 < KT) HB_SG_STORE((kt + 1) & 1);
    __syncthreads();
  }
#undef HB_SG_LOAD
#undef HB_SG_STORE
}

// One 128 x 128 tile of one product: workgroup `tile` of the problem's grid, k chunk `split` of a split-K launch.
// TA: A is given as [K, M] (op(A) = A^T); TB: B is given as [N, K] (op(B) = B^T)
template <bool TA, bool TB>
__device__ __forceinline__ void sgemm_tile(const SgemmArgs& g, const int tile, const int split) {
  __shared__ __attribute__((aligned(16))) float As[2][kGK * kGLD];
  __shared__ __attribute__((aligned(16))) float Bs[2][kGK * kGLD];
  const int tiles_n = (g.N + kGN - 1) / kGN;
  int bi = tile / tiles_n, bj = tile % tiles_n;
  bool mirror = false;
  if (g.sym) {  // workgroups 3d, 3d+1, 3d+2: tiles (2d, 2d), (2d, 2d+1) and (2d+1, 2d+1) of diagonal block d
    const int d = tile / 3, w = tile % 3;
    bi = 2 * d + (w == 2);
    bj = 2 * d + (w >= 1);
    mirror = w == 1;
  }
  const int row0 = bi * kGM, col0 = bj * kGN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  floatx16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int kb = g.part ? split * g.k_chunk : 0;
  const int ke = g.part ? (kb + g.k_chunk < g.K ? kb + g.k_chunk : g.K) : g.K;
  const bool interior = row0 + kGM <= g.M && col0 + kGN <= g.N && (ke - kb) % kGK == 0 && kb % 4 == 0 && g.lda % 4 == 0 && g.ldb % 4 == 0 &&
                        ((reinterpret_cast<uintptr_t>(g.A) | reinterpret_cast<uintptr_t>(g.B)) & 15) == 0;
  if (interior) sgemm_mainloop<TA, TB, true>(g, As, Bs, row0, col0, kb, ke, acc);
  else sgemm_mainloop<TA, TB, false>(g, As, Bs, row0, col0, kb, ke, acc);

  const int erow = (lane >> 5) * 4, ecol = lane & 31;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int col = col0 + wn * 64 + j * 32 + ecol;
      if (col >= g.N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = row0 + wm * 64 + i * 32 + (r >> 2) * 8 + erow + (r & 3);
        if (row >= g.M) continue;
        const float v = acc[i][j][r];
        if (g.part) {  // split-K: the epilogue runs in splitk_reduce_kernel
          g.part[((size_t)split * g.M + row) * g.N + col] = v;
          continue;
        }
        float* c = g.C + (size_t)row * g.ldc + col;
        // accumulate: the lerp of heavyball/utils.py:1048, m*(1-a) + outer*a, one rounding per operation
        const float out = g.accumulate ? (*c) * g.beta_c + v * g.alpha_acc : v;
        *c = out;
        if (mirror) g.C[(size_t)col * g.ldc + row] = out;
      }
    }
}

template <bool TA, bool TB>
__global__ __launch_bounds__(kGThreads, 3) void sgemm_kernel(const SgemmArgs g0, const Batch bt, const unsigned where) {
  SgemmArgs g = g0;
  if (bt.n > 1) {
    const int z = blockIdx.z;
    g.A = shifted(g0.A, where & kAInWs ? bt.dws[z] : bt.dq[z]);
    g.B = shifted(g0.B, where & kBInWs ? bt.dws[z] : bt.dq[z]);
    g.C = shifted(g0.C, where & kCInWs ? bt.dws[z] : bt.dq[z]);
    if (g0.part) g.part = shifted(g0.part, bt.dws[z]);
  }
  sgemm_tile<TA, TB>(g, (int)blockIdx.x, (int)blockIdx.y);
}

// Several independent products of one orientation in one launch: workgroup b belongs to the problem whose range of tiles holds b.
// The products of SOAP on a model of many mid-sized matrices (a 768 x 2304 projection is 108 tiles) leave most of the chip idle one
// at a time; together they fill it.  The tile body is the one of sgemm_kernel, so a product's bits do not depend on its company.
constexpr int kMaxGroup = 40;
struct SgemmGroup {
  SgemmArgs it[kMaxGroup];
  int tile_begin[kMaxGroup + 1];
  int n;
};
static_assert(sizeof(SgemmGroup) <= 4096, "the group travels as a kernel argument");
template <bool TA, bool TB>
__global__ __launch_bounds__(kGThreads, 3) void sgemm_group_kernel(const SgemmGroup grp) {
  typedef const __attribute__((address_space(4))) SgemmGroup* group_ptr_t;
  const group_ptr_t ka = (group_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
  int lo = 0, hi = ka->n - 1;  // the last problem whose first tile is not past this workgroup
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int)blockIdx.x >= ka->tile_begin[mid]) lo = mid;
    else hi = mid - 1;
  }
  SgemmArgs g;
  g.A = ka->it[lo].A; g.B = ka->it[lo].B; g.C = ka->it[lo].C;
  g.M = ka->it[lo].M; g.N = ka->it[lo].N; g.K = ka->it[lo].K;
  g.lda = ka->it[lo].lda; g.ldb = ka->it[lo].ldb; g.ldc = ka->it[lo].ldc;
  g.accumulate = ka->it[lo].accumulate; g.alpha_acc = ka->it[lo].alpha_acc; g.beta_c = ka->it[lo].beta_c;
  g.k_chunk = 0; g.part = nullptr; g.sym = 0;
  sgemm_tile<TA, TB>(g, (int)blockIdx.x - ka->tile_begin[lo], 0);
}

// ---------------------------------------------------------------------------------------------------------------
// The same product on 256 x 256 x 16 tiles, for operands whose sizes are multiples of the tile (the square and 4:1 factors
// and projections of SOAP).  Four wavefronts (2 x 2), each 128 x 128 = 4 x 4 MFMA tiles: 16 matrix instructions of 64
// cycles per k-step of 2 against 8 single-float fragments per lane, so one wavefront per SIMD keeps the matrix pipe busy
// while the next k-step's fragments (inline-assembly LDS reads, explicit waits) and the next k-tile's global loads
// (registers, parked in the other LDS buffer at the end of the tile) are in flight; one barrier per 8192 matrix cycles.
// Half the L2 -> LDS and LDS -> register traffic per flop of the 128 x 128 kernel.  No predication: the host only
// launches it on interior-only problems.
// ---------------------------------------------------------------------------------------------------------------
constexpr int kBM = 256, kBN = 256, kBLD = 260;
#ifndef HB_SGEMM_BIG_BK
#define HB_SGEMM_BIG_BK 16
#endif
constexpr int kBK = HB_SGEMM_BIG_BK;              // k-tile of the big kernel
constexpr int kBParts = kBK / 4;                  // float4 per thread and operand: 256 rows x kBK floats over 256 threads
constexpr int kBigLds = 2 * 2 * kBK * kBLD * (int)sizeof(float);  // two buffers x two operands

// Part q of a thread's share of an operand tile, NT threads per workgroup.  k-major memory ([k][row]): k-row
// tid/64 + (NT/64) q, rows (tid%64)*4..+3.  k-contiguous memory ([row][k]): kBK/4 threads per row, row
// tid/(kBK/4) + (NT*4/kBK) q, k (tid % (kBK/4)) * 4..+3.
template <bool KMAJOR, int NT>
__device__ __forceinline__ const float* big_ptr(const float* __restrict__ P, int ld, int row0) {
  const int tid = threadIdx.x;
  return KMAJOR ? P + (size_t)(tid / 64) * ld + row0 + (tid % 64) * 4 : P + (size_t)(row0 + tid / (kBK / 4)) * ld + (tid % (kBK / 4)) * 4;
}
template <bool KMAJOR, int NT>
__device__ __forceinline__ f32x4 big_load_part(const float* __restrict__ p, int ld, int q) {
  return *reinterpret_cast<const f32x4*>(p + (size_t)(KMAJOR ? (NT / 64) * q : (NT * 4 / kBK) * q) * ld);
}
template <bool KMAJOR, int NT>
__device__ __forceinline__ void big_store_part(float* __restrict__ S, const f32x4 r, int q) {
  const int tid = threadIdx.x;
  if (KMAJOR) {
    *reinterpret_cast<f32x4*>(S + (tid / 64 + (NT / 64) * q) * kBLD + (tid % 64) * 4) = r;
  } else {
    const int row = tid / (kBK / 4) + (NT * 4 / kBK) * q, k = (tid % (kBK / 4)) * 4;
    S[(k + 0) * kBLD + row] = r[0];
    S[(k + 1) * kBLD + row] = r[1];
    S[(k + 2) * kBLD + row] = r[2];
    S[(k + 3) * kBLD + row] = r[3];
  }
}
// rows r, r + 32 (offset 0) or r + 64, r + 96 (offset 64) of one k-row
__device__ __forceinline__ float2v lds_read2_f32_hi(uint32_t addr) {
  float2v v;
  asm volatile("ds_read2_b32 %0, %1 offset0:64 offset1:96" : "=v"(v) : "v"(addr));
  return v;
}

// WM x 2 wavefronts; each owns (256 / WM) x 128 of the tile.  WM = 4: eight wavefronts, two per SIMD, 64 x 128 each: a
// single wavefront cannot issue this matrix instruction back to back (a register-only loop of it reaches 139 TFLOP/s
// with one wavefront per SIMD and 155 with two), so two per SIMD fill each other's gaps.
template <bool TA, bool TB, int WM>
__global__ __launch_bounds__(WM * 128) void sgemm_big_kernel(const SgemmArgs g) {
  constexpr int NT = WM * 128;                       // threads
  constexpr int TM = 256 / WM / 32;                  // MFMA tiles per wavefront along M (4 or 2); 4 along N
  constexpr int PARTS = 256 * kBK / 4 / NT;          // float4 per thread and operand
  constexpr int READS = TM / 2 + 2;                  // fragment reads per k-step
  static_assert(TM == 2 || TM == 4, "wavefront tile");
  extern __shared__ __attribute__((aligned(16))) float big_smem[];
  float* As = big_smem;                      // [2][kBK * kBLD]
  float* Bs = big_smem + 2 * kBK * kBLD;     // [2][kBK * kBLD]
  const int tiles_n = g.N / kBN;
  int bi = blockIdx.x / tiles_n, bj = blockIdx.x % tiles_n;
  if (g.sym) {  // the tiles strictly above the diagonal, row by row: row bi holds tiles_n - 1 - bi of them
    int rem = blockIdx.x;
    bi = 0;
    while (bi < tiles_n - 1 && rem >= tiles_n - 1 - bi) {
      rem -= tiles_n - 1 - bi;
      ++bi;
    }
    bj = bi + 1 + rem;
    if (bj >= tiles_n) return;  // a grid larger than the triangle: nothing to do (the host never launches one)
  }
  const int row0 = bi * kBM, col0 = bj * kBN;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  floatx16 acc[TM][4];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int KT = g.K / kBK;
  const float* pa = big_ptr<TA, NT>(g.A, g.lda, row0);
  const float* pb = big_ptr<!TB, NT>(g.B, g.ldb, col0);
  const size_t step_a = TA ? (size_t)kBK * g.lda : (size_t)kBK, step_b = !TB ? (size_t)kBK * g.ldb : (size_t)kBK;
  // the next k-tile on its way from memory to LDS: native vectors, every index a constant after unrolling, so that they
  // stay in registers
  f32x4 ra[PARTS], rb[PARTS];
#pragma unroll
  for (int q = 0; q < PARTS; ++q) {
    ra[q] = big_load_part<TA, NT>(pa, g.lda, q);
    rb[q] = big_load_part<!TB, NT>(pb, g.ldb, q);
  }
#pragma unroll
  for (int q = 0; q < PARTS; ++q) {
    big_store_part<TA, NT>(As, ra[q], q);
    big_store_part<!TB, NT>(Bs, rb[q], q);
  }
  __syncthreads();
  const int fr = lane & 31, fk = lane >> 5;
  constexpr int KS = kBK / 2;  // k-steps per tile
  for (int kt = 0; kt < KT; ++kt) {
    const bool more = kt + 1 < KT;
    if (more) {
      pa += step_a;
      pb += step_b;
#pragma unroll
      for (int q = 0; q < PARTS; ++q) {
        ra[q] = big_load_part<TA, NT>(pa, g.lda, q);
        rb[q] = big_load_part<!TB, NT>(pb, g.ldb, q);
      }
    }
    const uint32_t a = lds_addr(As + (kt & 1) * kBK * kBLD + wm * (TM * 32) + fr + fk * kBLD);
    const uint32_t b = lds_addr(Bs + (kt & 1) * kBK * kBLD + wn * 128 + fr + fk * kBLD);
    float* nextA = As + ((kt + 1) & 1) * kBK * kBLD;
    float* nextB = Bs + ((kt + 1) & 1) * kBK * kBLD;
    float2v af[2][2], bf[2][2];  // [set][low | high pair of tiles]
    af[0][0] = lds_read2_f32(a);
    if (TM == 4) af[0][1] = lds_read2_f32_hi(a);
    bf[0][0] = lds_read2_f32(b);
    bf[0][1] = lds_read2_f32_hi(b);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < KS) {
        const uint32_t off = (ks + 1) * 2 * kBLD * 4;
        af[nxt][0] = lds_read2_f32(a + off);
        if (TM == 4) af[nxt][1] = lds_read2_f32_hi(a + off);
        bf[nxt][0] = lds_read2_f32(b + off);
        bf[nxt][1] = lds_read2_f32_hi(b + off);
        __builtin_amdgcn_s_waitcnt(0xC07F | (READS << 8));  // lgkmcnt(READS): this step's reads have landed
      } else {
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[cur][i >> 1][i & 1], bf[cur][j >> 1][j & 1], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      // The other LDS buffer is idle during this whole k-tile: park the next tile's staged registers in it one part at a
      // time behind the matrix instructions of the last PARTS k-steps, so the LDS writes run under them instead of
      // between the last matrix instruction and the barrier (where they cost 15-25 % of the tile's time).
      if (more && ks >= KS - PARTS) {
        const int q = ks - (KS - PARTS);
        big_store_part<TA, NT>(nextA, ra[q], q);
        big_store_part<!TB, NT>(nextB, rb[q], q);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();
  }

  // epilogue, one MFMA tile at a time (a scheduling barrier between tiles keeps the compiler from hoisting the address
  // arithmetic and the loads of C of all tiles, which does not fit the register file)
  const int erow = (lane >> 5) * 4, ecol = lane & 31;
  float* cbase = g.C + (size_t)(row0 + wm * (TM * 32) + erow) * g.ldc + col0 + wn * 128 + ecol;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float* ct = cbase + (size_t)(i * 32) * g.ldc + j * 32;
      float out[16];
      if (g.accumulate) {
#pragma unroll
        for (int r = 0; r < 16; ++r) out[r] = ct[(size_t)((r >> 2) * 8 + (r & 3)) * g.ldc];
#pragma unroll
        for (int r = 0; r < 16; ++r) out[r] = out[r] * g.beta_c + acc[i][j][r] * g.alpha_acc;  // heavyball/utils.py:1048
      } else {
#pragma unroll
        for (int r = 0; r < 16; ++r) out[r] = acc[i][j][r];
      }
#pragma unroll
      for (int r = 0; r < 16; ++r) ct[(size_t)((r >> 2) * 8 + (r & 3)) * g.ldc] = out[r];
      if (g.sym) {  // the transposed tile: a lane's four consecutive rows are four consecutive columns there
        float* mt = g.C + (size_t)(col0 + wn * 128 + j * 32 + ecol) * g.ldc + row0 + wm * (TM * 32) + i * 32 + erow;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const f32x4 v = {out[4 * q], out[4 * q + 1], out[4 * q + 2], out[4 * q + 3]};
          *reinterpret_cast<f32x4*>(mt + q * 8) = v;
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
}

// _compilable_adam_ (heavyball/utils.py:1852-1868) on flat fp32 arrays: the moments are updated in place and
// out = exp_avg / max(sqrt(exp_avg_sq), eps)
__global__ __launch_bounds__(256) void adam_precond_kernel(float* __restrict__ m, float* __restrict__ v, const float* __restrict__ gr,
                                                           float* __restrict__ out, int64_t n, float a1, float oma1, float a2, float oma2,
                                                           float eps) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    const float x = gr[i];
    const float mm = m[i] * oma1 + x * a1;
    const float vv = v[i] * oma2 + (x * x) * a2;
    m[i] = mm;
    v[i] = vv;
    out[i] = mm / __builtin_fmaxf(__builtin_sqrtf(vv), eps);
  }
}

// The same for several tensors in one launch: tensor t owns workgroups [block_begin[t], block_begin[t + 1]), each of which walks
// its tensor with that many workgroups' stride (a model's vectors are a few hundred elements each: one launch per tensor is all
// launch latency).
constexpr int kMaxAdamGroup = 80;
struct AdamGroup {
  float* m[kMaxAdamGroup];
  float* v[kMaxAdamGroup];
  const float* g[kMaxAdamGroup];
  float* out[kMaxAdamGroup];
  int64_t n[kMaxAdamGroup];
  int block_begin[kMaxAdamGroup + 1];
  int count;
  float a1, oma1, a2, oma2, eps;
};
static_assert(sizeof(AdamGroup) <= 4096, "the group travels as a kernel argument");
__global__ __launch_bounds__(256) void adam_precond_group_kernel(const AdamGroup grp) {
  typedef const __attribute__((address_space(4))) AdamGroup* group_ptr_t;
  const group_ptr_t ka = (group_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
  int lo = 0, hi = ka->count - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int)blockIdx.x >= ka->block_begin[mid]) lo = mid;
    else hi = mid - 1;
  }
  float* __restrict__ m = ka->m[lo];
  float* __restrict__ v = ka->v[lo];
  const float* __restrict__ gr = ka->g[lo];
  float* __restrict__ out = ka->out[lo];
  const int64_t n = ka->n[lo];
  const int first = ka->block_begin[lo], blocks = ka->block_begin[lo + 1] - first;
  const float a1 = ka->a1, oma1 = ka->oma1, a2 = ka->a2, oma2 = ka->oma2, eps = ka->eps;
  for (int64_t i = (int64_t)((int)blockIdx.x - first) * 256 + threadIdx.x; i < n; i += (int64_t)blocks * 256) {
    const float x = gr[i];
    const float mm = m[i] * oma1 + x * a1;
    const float vv = v[i] * oma2 + (x * x) * a2;
    m[i] = mm;
    v[i] = vv;
    out[i] = mm / __builtin_fmaxf(__builtin_sqrtf(vv), eps);
  }
}

// split-K: adds the partial products in a fixed order (deterministic) and applies the epilogue of sgemm_kernel
__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ part, int splits, int M, int N, float* __restrict__ C,
                                                            int ldc, int accumulate, float alpha_acc, float beta_c, const Batch bt,
                                                            const unsigned where) {
  if (bt.n > 1) {
    part = shifted(part, bt.dws[blockIdx.y]);
    C = shifted(C, where & kCInWs ? bt.dws[blockIdx.y] : bt.dq[blockIdx.y]);
  }
  const int64_t n = (int64_t)M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    float v = 0.0f;
    int s = 0;
    for (; s + 8 <= splits; s += 8) {  // eight loads in flight, added in index order
      float q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) q[u] = part[(size_t)(s + u) * n + i];
#pragma unroll
      for (int u = 0; u < 8; ++u) v += q[u];
    }
    for (; s < splits; ++s) v += part[(size_t)s * n + i];
    float* c = C + (size_t)(i / N) * ldc + (i % N);
    *c = accumulate ? (*c) * beta_c + v * alpha_acc : v;
  }
}

// Upper Cholesky factor of one small symmetric matrix, G = R^T R, in place in a [n][n] global array (n <= 128; the
// strict lower triangle is written as zeros), one workgroup of 32 x 16 threads (two wavefronts per SIMD, so that one
// runs while the other waits on LDS or the reciprocal square root).  The matrix lives in registers: thread
// (ty, tx) owns the elements (ty + 32 a, tx + 16 b).  Right-looking, two columns per barrier: the owners of rows j and
// j+1 publish them unscaled (double-buffered in LDS) right after the update of the columns before; every thread derives
// the two pivots and the two scaled rows from them itself (row j+1 needs column j applied first: one fused multiply-add
// per element, the same one the rank-1 update would have done) and applies both rank-1 updates to its 64 elements.  A pivot that is not
// positive (a numerically rank-deficient panel) raises *status and is replaced by a tiny positive number so that the
// kernel still finishes with finite output.
constexpr int kPanel = 128;
constexpr int kPanelLD = kPanel + 1;
#ifndef HB_CHOL_ROW_THREADS
#define HB_CHOL_ROW_THREADS 32
#endif
constexpr int kCholRT = HB_CHOL_ROW_THREADS;  // threads along a column: each owns kPanel / kCholRT rows
constexpr int kCholRows = kPanel / kCholRT;
constexpr int kCholThreads = 16 * kCholRT;
__global__ __launch_bounds__(kCholThreads) void chol_kernel(float* __restrict__ G, int n, const Batch bt) {
  int* __restrict__ status = bt.status[blockIdx.x];  // one workgroup per problem
  G = shifted(G, bt.dws[blockIdx.x]);
  __shared__ float rowbuf[2][2][kPanel];  // [parity of the pair of rows][row of the pair][column]
  const int t = threadIdx.x, tx = t & 15, ty = t >> 4;  // ty = 0..kCholRT-1
  float reg[kCholRows][8];
#pragma unroll
  for (int a = 0; a < kCholRows; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const int r = ty + kCholRT * a, c = tx + 16 * b;
      reg[a][b] = (r < n && c < n && r <= c) ? G[(size_t)r * n + c] : 0.0f;
    }
  if (ty < 2) {  // rows 0 and 1 as they stand
#pragma unroll
    for (int b = 0; b < 8; ++b) rowbuf[0][ty][tx + 16 * b] = reg[0][b];
  }
  __syncthreads();
#pragma unroll
  for (int jb = 0; jb < 8; ++jb) {  // block of 16 columns
    const int ja = jb * 16 / kCholRT;  // the block of kCholRT rows that holds rows 16 jb .. 16 jb + 15
    const int s0 = jb * 16 % kCholRT;  // ty of the owners of row 16 jb
    for (int jp = 0; jp < 8; ++jp) {
      const int j = jb * 16 + 2 * jp;  // this pass of the loop factors columns j and j + 1
      if (j >= n) break;
      const int rj = s0 + 2 * jp;  // ty of the owners of row j
      const bool two = j + 1 < n;
      const float(*rb)[kPanel] = rowbuf[(j >> 1) & 1];
      // column j from row j as published; column j + 1 from row j + 1 after this thread has applied column j to it
      float d0 = rb[0][j];
      if (!(d0 > 0.0f) || !(d0 < 3.0e38f)) {
        if (t == 0) *status = 1;
        d0 = 1e-30f;
      }
      // 1-ulp hardware reciprocal square root: R^T R = G then holds to a few ulps, which is all the callers need
      const float inv0 = __builtin_amdgcn_rsqf(d0), piv0 = d0 * inv0;
      const float r01 = rb[0][j + 1] * inv0;  // R[j][j+1]
      float d1 = __builtin_fmaf(-r01, r01, rb[1][j + 1]);
      if (two && (!(d1 > 0.0f) || !(d1 < 3.0e38f))) {
        if (t == 0) *status = 1;
        d1 = 1e-30f;
      }
      const float inv1 = two ? __builtin_amdgcn_rsqf(d1) : 0.0f, piv1 = d1 * inv1;
      // Only the blocks on and right of the diagonal block, and rows below the pair, are touched.  Elements left of the
      // diagonal inside those blocks pick up meaningless values: nothing reads them and zeros are stored for them.
      // Rows and columns >= n hold zeros throughout, so they need no predicate either.
      float c0[8], c1[8];  // R[j][c] and R[j+1][c] for this thread's columns
#pragma unroll
      for (int b = jb; b < 8; ++b) {
        c0[b] = rb[0][tx + 16 * b] * inv0;
        c1[b] = __builtin_fmaf(-r01, c0[b], rb[1][tx + 16 * b]) * inv1;
      }
      if (ty == rj) {  // the owners of the two rows keep their final values
#pragma unroll
        for (int b = jb; b < 8; ++b) reg[ja][b] = tx + 16 * b == j ? piv0 : c0[b];
      } else if (ty == rj + 1) {
#pragma unroll
        for (int b = jb; b < 8; ++b) reg[ja][b] = tx + 16 * b == j + 1 ? piv1 : c1[b];
      } else if (ty > rj + 1) {
        const float a0 = rb[0][ty + kCholRT * ja] * inv0;
        const float a1 = __builtin_fmaf(-r01, a0, rb[1][ty + kCholRT * ja]) * inv1;
#pragma unroll
        for (int b = jb; b < 8; ++b) reg[ja][b] = __builtin_fmaf(-a1, c1[b], __builtin_fmaf(-a0, c0[b], reg[ja][b]));
      }
#pragma unroll
      for (int a = ja + 1; a < kCholRows; ++a) {
        const float a0 = rb[0][ty + kCholRT * a] * inv0;
        const float a1 = __builtin_fmaf(-r01, a0, rb[1][ty + kCholRT * a]) * inv1;
#pragma unroll
        for (int b = (kCholRT * a / 16 > jb ? kCholRT * a / 16 : jb); b < 8; ++b)  // column blocks left of that lie below the diagonal for these rows
          reg[a][b] = __builtin_fmaf(-a1, c1[b], __builtin_fmaf(-a0, c0[b], reg[a][b]));
      }
      // the owners of the next two rows publish them (updated, unscaled) in the other buffer: one barrier per pair
      if (j + 2 < n) {
        float(*nb)[kPanel] = rowbuf[((j >> 1) + 1) & 1];
        if (jp < 7 || s0 + 16 < kCholRT) {  // rows j+2, j+3 are in the same block of rows
          if (ty == rj + 2 || ty == rj + 3) {
#pragma unroll
            for (int b = jb; b < 8; ++b) nb[ty - (rj + 2)][tx + 16 * b] = reg[ja][b];
          }
        } else if (ja < kCholRows - 1) {  // they open the next block of rows
          const int an = ja < kCholRows - 1 ? ja + 1 : kCholRows - 1;  // a constant once the jb loop is unrolled
          if (ty < 2) {
#pragma unroll
            for (int b = jb; b < 8; ++b) nb[ty][tx + 16 * b] = reg[an][b];
          }
        }
      }
      __syncthreads();
    }
  }
#pragma unroll
  for (int a = 0; a < kCholRows; ++a)
#pragma unroll
    for (int b = 0; b < 8; ++b) {
      const int r = ty + kCholRT * a, c = tx + 16 * b;
      if (r < n && c < n) G[(size_t)r * n + c] = r <= c ? reg[a][b] : 0.0f;
    }
}

// P <- P R^-1 for an upper-triangular R [n][n] (n <= kPanel): every row x of P solves x R = p, blocked by 16 columns.
// A workgroup takes 32 rows, so an 8192-row panel fills the chip (256 workgroups); R, the rows and the explicit inverses
// of R's eight 16 x 16 diagonal blocks live in LDS (R's rows padded to a multiple of four words so that four neighbours
// load as one 128-bit broadcast, the rows of P to kPanelLD words).  The block inverses are computed once per workgroup
// (one thread per column, a 16-step back substitution); after that a block step has no dependent chain: eight threads
// per row form x_b <- x_b D_b^-1 (two columns each) and then eliminate the solved block from the columns to its
// right, four columns at a time.
constexpr int kTrsmBlock = 16;
constexpr int kTrsmRows = 32;
constexpr int kTrsmRLD = kPanel + 4;
constexpr int kTrsmDLD = kTrsmBlock + 1;
constexpr int kTrsmLds = (kPanel * kTrsmRLD + (kPanel / kTrsmBlock) * kTrsmBlock * kTrsmDLD + kTrsmRows * kPanelLD + kTrsmRows * kTrsmBlock) * (int)sizeof(float);
__global__ __launch_bounds__(256) void trsm_right_upper_kernel(float* __restrict__ P, int ld, int rows, const float* __restrict__ Rg, int n,
                                                               const Batch bt) {
  P = shifted(P, bt.dq[blockIdx.y]);  // blockIdx.y: the problem
  Rg = shifted(Rg, bt.dws[blockIdx.y]);
  extern __shared__ __attribute__((aligned(16))) float lds[];
  float* R = lds;                                                   // [kPanel][kTrsmRLD], the identity beyond n
  float* Di = R + kPanel * kTrsmRLD;                                // [8][16][kTrsmDLD]: inverse of diagonal block b, upper
  float* X = Di + (kPanel / kTrsmBlock) * kTrsmBlock * kTrsmDLD;    // [kTrsmRows][kPanelLD]
  float* Xs = X + kTrsmRows * kPanelLD;                             // [kTrsmRows][16]: the block just solved
  const int t = threadIdx.x;
  const int row0 = blockIdx.x * kTrsmRows;
  // Full panels with 16-byte aligned rows (every panel of a matrix whose width is a multiple of 128) move as float4 with
  // all of a thread's loads in flight at once; a rolled loop of single floats would pay one memory round trip per
  // element and, at 66 elements of R per thread, take longer than the solve itself.
  const bool wide = n == kPanel && (ld & 3) == 0 && row0 + kTrsmRows <= rows &&
                    ((reinterpret_cast<uintptr_t>(P) | reinterpret_cast<uintptr_t>(Rg)) & 15) == 0;
  if (wide) {
    f32x4 rv[16], xv[4];
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int idx = t + q * 256;
      rv[q] = *reinterpret_cast<const f32x4*>(Rg + (size_t)(idx >> 5) * kPanel + (idx & 31) * 4);
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = t + q * 256;
      xv[q] = *reinterpret_cast<const f32x4*>(P + (size_t)(row0 + (idx >> 5)) * ld + (idx & 31) * 4);
    }
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int idx = t + q * 256;
      *reinterpret_cast<f32x4*>(R + (idx >> 5) * kTrsmRLD + (idx & 31) * 4) = rv[q];
    }
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = t + q * 256;
      float* xp = X + (idx >> 5) * kPanelLD + (idx & 31) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) xp[e] = xv[q][e];
    }
  } else {
    for (int i = t; i < kPanel * kTrsmRLD; i += 256) {
      const int r = i / kTrsmRLD, c = i % kTrsmRLD;
      R[i] = (r < n && c < n) ? Rg[(size_t)r * n + c] : (r == c ? 1.0f : 0.0f);
    }
    for (int i = t; i < kTrsmRows * kPanel; i += 256) {  // thread column = i % 128: coalesced
      const int r = i / kPanel, c = i % kPanel;
      X[r * kPanelLD + c] = (row0 + r < rows && c < n) ? P[(size_t)(row0 + r) * ld + c] : 0.0f;
    }
  }
  __syncthreads();
  if (t < kPanel) {  // column j of the inverse of diagonal block b: D x = e_j, back substitution from row j upwards
    const int b = t / kTrsmBlock, j = t % kTrsmBlock;
    const float* D = R + (b * kTrsmBlock) * kTrsmRLD + b * kTrsmBlock;
    float x[kTrsmBlock];
#pragma unroll
    for (int k = kTrsmBlock - 1; k >= 0; --k) {
      float sacc = k == j ? 1.0f : 0.0f;
#pragma unroll
      for (int i = k + 1; i < kTrsmBlock; ++i) sacc -= D[k * kTrsmRLD + i] * (i <= j ? x[i] : 0.0f);
      x[k] = k <= j ? sacc / D[k * kTrsmRLD + k] : 0.0f;
    }
#pragma unroll
    for (int k = 0; k < kTrsmBlock; ++k) Di[(b * kTrsmBlock + k) * kTrsmDLD + j] = x[k];
  }
  __syncthreads();
  const int row = t >> 3, sub = t & 7;
  float* x = X + row * kPanelLD;
#pragma unroll 1
  for (int b0 = 0; b0 < n; b0 += kTrsmBlock) {  // columns beyond n are zeros against a unit diagonal: harmless
    const float* Db = Di + b0 * kTrsmDLD;
    float o0 = 0.0f, o1 = 0.0f;
#pragma unroll
    for (int k = 0; k < kTrsmBlock; ++k) {
      const float xv = x[b0 + k];
      o0 += xv * Db[k * kTrsmDLD + 2 * sub];
      o1 += xv * Db[k * kTrsmDLD + 2 * sub + 1];
    }
    Xs[row * kTrsmBlock + 2 * sub] = o0;
    Xs[row * kTrsmBlock + 2 * sub + 1] = o1;
    __syncthreads();  // the block is solved (and everyone has read its old values)
    x[b0 + 2 * sub] = o0;
    x[b0 + 2 * sub + 1] = o1;
    float xb[kTrsmBlock];
#pragma unroll
    for (int k = 0; k < kTrsmBlock; ++k) xb[k] = Xs[row * kTrsmBlock + k];
    for (int c = b0 + kTrsmBlock + 4 * sub; c < kPanel; c += 32) {
      float acc[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[e] = x[c + e];
#pragma unroll
      for (int k = 0; k < kTrsmBlock; ++k) {
        const float4 rv = *reinterpret_cast<const float4*>(R + (b0 + k) * kTrsmRLD + c);
        acc[0] -= xb[k] * rv.x;
        acc[1] -= xb[k] * rv.y;
        acc[2] -= xb[k] * rv.z;
        acc[3] -= xb[k] * rv.w;
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) x[c + e] = acc[e];
    }
    __syncthreads();  // the columns to the right are updated before the next block reads them (and Xs is free again)
  }
  if (wide) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int idx = t + q * 256;
      const float* xp = X + (idx >> 5) * kPanelLD + (idx & 31) * 4;
      f32x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = xp[e];
      *reinterpret_cast<f32x4*>(P + (size_t)(row0 + (idx >> 5)) * ld + (idx & 31) * 4) = v;
    }
  } else {
    for (int i = t; i < kTrsmRows * kPanel; i += 256) {
      const int r = i / kPanel, c = i % kPanel;
      if (row0 + r < rows && c < n) P[(size_t)(row0 + r) * ld + c] = X[r * kPanelLD + c];
    }
  }
}

__global__ void set_status_kernel(const Batch bt, int v) {
  if (threadIdx.x < bt.n) *bt.status[threadIdx.x] = v;
}

// One GEMM of the orthonormalisation: plain launch, or split-K when the output has too few tiles to fill the GPU.
static int sgemm_launch(SgemmArgs g, bool ta, bool tb, float* part, size_t part_elems, hipStream_t s, const Batch& bt, unsigned where) {
  const int nb = bt.n > 1 ? bt.n : 1;
  const int64_t tiles = ((int64_t)(g.M + kGM - 1) / kGM) * ((g.N + kGN - 1) / kGN) * nb;  // of the whole batch
  int splits = 1;
  if (part && tiles < 512 && g.K >= 256) {
    // two workgroups per compute unit, at least 64 of k each: a workgroup spends ~1 us of matrix-core time per 16 of k
    // (one wavefront per SIMD), so a panel product is as long as its deepest chunk (measured on the panel products of
    // hb_orthonormalize_f32: more workgroups than that gain nothing; 64-deep chunks are 15 % faster than 256-deep ones
    // on 2048-row panels, 32-deep ones no faster)
    splits = (int)(512 / tiles);
    if (splits > g.K / 64) splits = g.K / 64;
    if (splits > 128) splits = 128;
    while (splits > 1 && (size_t)splits * g.M * g.N > part_elems) --splits;
  }
  dim3 grid((unsigned)(tiles / nb), 1, (unsigned)nb);
  if (splits > 1) {
    g.k_chunk = ((g.K + splits - 1) / splits + kGK - 1) / kGK * kGK;
    splits = (g.K + g.k_chunk - 1) / g.k_chunk;
    g.part = part;
    grid.y = splits;
  } else {
    g.part = nullptr;
    g.k_chunk = 0;
  }
  if (ta) {
    if (tb) sgemm_kernel<true, true><<<grid, kGThreads, 0, s>>>(g, bt, where);
    else sgemm_kernel<true, false><<<grid, kGThreads, 0, s>>>(g, bt, where);
  } else {
    if (tb) sgemm_kernel<false, true><<<grid, kGThreads, 0, s>>>(g, bt, where);
    else sgemm_kernel<false, false><<<grid, kGThreads, 0, s>>>(g, bt, where);
  }
  if (splits > 1) {
    const int64_t n = (int64_t)g.M * g.N;
    const int blocks = (int)((n + 255) / 256 < 2048 ? (n + 255) / 256 : 2048);
    splitk_reduce_kernel<<<dim3(blocks, nb), 256, 0, s>>>(part, splits, g.M, g.N, g.C, g.ldc, g.accumulate, g.alpha_acc, g.beta_c, bt, where);
  }
  return HB_OK;
}

struct OrthoPlan {
  size_t off_c, off_g, off_part, part_elems, total;
};
static OrthoPlan ortho_plan(int64_t m, int64_t n) {
  OrthoPlan p;
  size_t o = 0;
  auto take = [&](size_t elems) { size_t at = o; o += (elems * sizeof(float) + 255) & ~size_t(255); return at; };
  p.off_c = take((size_t)n * kPanel);
  p.off_g = take((size_t)kPanel * kPanel);
  p.part_elems = (size_t)4 << 20;  // 16 MiB of split-K partials
  p.off_part = take(p.part_elems);
  p.total = o;
  return p;
}

// fewest 256 x 256 tiles worth a launch of the big-tile kernel (one per compute unit fills the chip; below about half
// of that the 128 x 128 kernel, with four times as many workgroups, is faster); HB_SGEMM_BIG_MIN overrides it
static int sgemm_big_min_tiles() {
  static int v = [] {
    const char* e = getenv("HB_SGEMM_BIG_MIN");
    return e ? atoi(e) : 128;
  }();
  return v;
}

}  // namespace hb

extern "C" int hb_gemm_f32(const float* A, const float* B, float* C, int64_t M, int64_t N, int64_t K, int64_t lda, int64_t ldb, int64_t ldc,
                           int32_t trans_a, int32_t trans_b, int32_t accumulate, float alpha_acc, float beta_c, void* stream_) {
  using namespace hb;
  if (!A || !B || !C) return set_error(HB_EINVAL, "hb_gemm_f32: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || M > (1 << 24) || N > (1 << 24) || K > (1 << 24)) return set_error(HB_EINVAL, "hb_gemm_f32: bad shape");
  const int64_t need_a = trans_a ? M : K, need_b = trans_b ? K : N;
  if (lda < need_a || ldb < need_b || ldc < N) return set_error(HB_EINVAL, "hb_gemm_f32: leading dimension too small");
  if (accumulate & ~(HB_GEMM_ACCUMULATE | HB_GEMM_SYMMETRIC)) return set_error(HB_EINVAL, "hb_gemm_f32: unknown flag");
  const bool want_sym = (accumulate & HB_GEMM_SYMMETRIC) != 0;
  if (want_sym && !(A == B && lda == ldb && M == N && (trans_a != 0) != (trans_b != 0)))
    return set_error(HB_EINVAL, "hb_gemm_f32: HB_GEMM_SYMMETRIC takes one matrix as both operands, transposed on exactly one side");
  SgemmArgs g{A, B, C, (int)M, (int)N, (int)K, (int)lda, (int)ldb, (int)ldc, accumulate & HB_GEMM_ACCUMULATE, alpha_acc, beta_c, 0, nullptr, 0};
  const int64_t tiles = ((M + kGM - 1) / kGM) * ((N + kGN - 1) / kGN);
  if (tiles > 0x7FFFFFFF) return set_error(HB_EINVAL, "hb_gemm_f32: too many tiles");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  // 256 x 256 tiles when nothing needs predication and they still fill the chip
  const int64_t big_tiles = (M / kBM) * (N / kBN);
  const bool big = M % kBM == 0 && N % kBN == 0 && K % kBK == 0 && lda % 4 == 0 && ldb % 4 == 0 && ldc >= N &&
                   ((reinterpret_cast<uintptr_t>(A) | reinterpret_cast<uintptr_t>(B)) & 15) == 0 && big_tiles >= sgemm_big_min_tiles();
  if (big) {
#ifndef HB_SGEMM_BIG_WM
#define HB_SGEMM_BIG_WM 4
#endif
    constexpr int WM = HB_SGEMM_BIG_WM;
    static LdsReservation reserved;
    const void* ks[4] = {reinterpret_cast<const void*>(sgemm_big_kernel<false, false, WM>), reinterpret_cast<const void*>(sgemm_big_kernel<false, true, WM>),
                         reinterpret_cast<const void*>(sgemm_big_kernel<true, false, WM>), reinterpret_cast<const void*>(sgemm_big_kernel<true, true, WM>)};
    if (int rc = reserve_lds(reserved, ks, 4, kBigLds, "hb_gemm_f32")) return rc;
    // Symmetric output: the tiles strictly above the diagonal on the big-tile kernel, each also stored transposed, and
    // the diagonal 256 x 256 blocks as three 128 x 128 tiles each.  On 32 x 32 tiles that is 496 workgroups, just under
    // two rounds of the 256 compute units, where the full product takes four (the 32 diagonal tiles on the big-tile
    // kernel as well would start a third round that leaves the chip almost empty).
    const int64_t T = N / kBN, sym_tiles = T * (T - 1) / 2;
    if (want_sym && sym_tiles >= sgemm_big_min_tiles() && ldc % 4 == 0 && (reinterpret_cast<uintptr_t>(C) & 15) == 0) {
      g.sym = 1;
      if (trans_a) {
        sgemm_big_kernel<true, false, WM><<<(unsigned)sym_tiles, WM * 128, kBigLds, s>>>(g);
        sgemm_kernel<true, false><<<(unsigned)(3 * T), kGThreads, 0, s>>>(g, Batch{}, 0u);
      } else {
        sgemm_big_kernel<false, true, WM><<<(unsigned)sym_tiles, WM * 128, kBigLds, s>>>(g);
        sgemm_kernel<false, true><<<(unsigned)(3 * T), kGThreads, 0, s>>>(g, Batch{}, 0u);
      }
      return check_launch("hb_gemm_f32");
    }
    if (trans_a) {
      if (trans_b) sgemm_big_kernel<true, true, WM><<<(unsigned)big_tiles, WM * 128, kBigLds, s>>>(g);
      else sgemm_big_kernel<true, false, WM><<<(unsigned)big_tiles, WM * 128, kBigLds, s>>>(g);
    } else {
      if (trans_b) sgemm_big_kernel<false, true, WM><<<(unsigned)big_tiles, WM * 128, kBigLds, s>>>(g);
      else sgemm_big_kernel<false, false, WM><<<(unsigned)big_tiles, WM * 128, kBigLds, s>>>(g);
    }
    return check_launch("hb_gemm_f32");
  }
  if (trans_a) {
    if (trans_b) sgemm_kernel<true, true><<<(unsigned)tiles, kGThreads, 0, s>>>(g, Batch{}, 0u);
    else sgemm_kernel<true, false><<<(unsigned)tiles, kGThreads, 0, s>>>(g, Batch{}, 0u);
  } else {
    if (trans_b) sgemm_kernel<false, true><<<(unsigned)tiles, kGThreads, 0, s>>>(g, Batch{}, 0u);
    else sgemm_kernel<false, false><<<(unsigned)tiles, kGThreads, 0, s>>>(g, Batch{}, 0u);
  }
  return check_launch("hb_gemm_f32");
}

extern "C" int hb_gemm_f32_grouped(int32_t n, const float* const* A, const float* const* B, float* const* C, const int64_t* M, const int64_t* N,
                                   const int64_t* K, const int64_t* lda, const int64_t* ldb, const int64_t* ldc, int32_t trans_a, int32_t trans_b,
                                   const int32_t* accumulate, const float* alpha_acc, const float* beta_c, void* stream_) {
  using namespace hb;
  if (n < 0) return set_error(HB_EINVAL, "hb_gemm_f32_grouped: negative count");
  if (n == 0) return HB_OK;
  if (!A || !B || !C || !M || !N || !K || !lda || !ldb || !ldc || !accumulate || !alpha_acc || !beta_c)
    return set_error(HB_EINVAL, "hb_gemm_f32_grouped: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  SgemmGroup grp;
  grp.n = 0;
  grp.tile_begin[0] = 0;
  auto flush = [&]() {
    if (grp.n == 0) return;
    const unsigned blocks = (unsigned)grp.tile_begin[grp.n];
    if (trans_a) {
      if (trans_b) sgemm_group_kernel<true, true><<<blocks, kGThreads, 0, s>>>(grp);
      else sgemm_group_kernel<true, false><<<blocks, kGThreads, 0, s>>>(grp);
    } else {
      if (trans_b) sgemm_group_kernel<false, true><<<blocks, kGThreads, 0, s>>>(grp);
      else sgemm_group_kernel<false, false><<<blocks, kGThreads, 0, s>>>(grp);
    }
    grp.n = 0;
  };
  for (int i = 0; i < n; ++i) {
    if (!A[i] || !B[i] || !C[i]) return set_error(HB_EINVAL, "hb_gemm_f32_grouped: null matrix pointer at %d", i);
    if (M[i] <= 0 || N[i] <= 0 || K[i] <= 0 || M[i] > (1 << 24) || N[i] > (1 << 24) || K[i] > (1 << 24))
      return set_error(HB_EINVAL, "hb_gemm_f32_grouped: bad shape at %d", i);
    const int64_t big_tiles = (M[i] / kBM) * (N[i] / kBN);
    const bool big = M[i] % kBM == 0 && N[i] % kBN == 0 && K[i] % kBK == 0 && lda[i] % 4 == 0 && ldb[i] % 4 == 0 && ldc[i] >= N[i] &&
                     ((reinterpret_cast<uintptr_t>(A[i]) | reinterpret_cast<uintptr_t>(B[i])) & 15) == 0 && big_tiles >= sgemm_big_min_tiles();
    const int64_t tiles = ((M[i] + kGM - 1) / kGM) * ((N[i] + kGN - 1) / kGN);
    if (big || tiles > (1 << 22)) {  // fills the chip on its own: the single call's kernels (and its checks)
      if (int rc = hb_gemm_f32(A[i], B[i], C[i], M[i], N[i], K[i], lda[i], ldb[i], ldc[i], trans_a, trans_b, accumulate[i], alpha_acc[i], beta_c[i],
                               stream_))
        return rc;
      continue;
    }
    const int64_t need_a = trans_a ? M[i] : K[i], need_b = trans_b ? K[i] : N[i];
    if (lda[i] < need_a || ldb[i] < need_b || ldc[i] < N[i]) return set_error(HB_EINVAL, "hb_gemm_f32_grouped: leading dimension too small at %d", i);
    if (accumulate[i] & ~(HB_GEMM_ACCUMULATE | HB_GEMM_SYMMETRIC)) return set_error(HB_EINVAL, "hb_gemm_f32_grouped: unknown flag at %d", i);
    if ((accumulate[i] & HB_GEMM_SYMMETRIC) && !(A[i] == B[i] && lda[i] == ldb[i] && M[i] == N[i] && (trans_a != 0) != (trans_b != 0)))
      return set_error(HB_EINVAL, "hb_gemm_f32_grouped: HB_GEMM_SYMMETRIC takes one matrix as both operands, transposed on exactly one side (%d)", i);
    if (grp.n == kMaxGroup || (int64_t)grp.tile_begin[grp.n] + tiles > 0x3FFFFFFF) flush();
    grp.it[grp.n] = SgemmArgs{A[i], B[i], C[i], (int)M[i], (int)N[i], (int)K[i], (int)lda[i], (int)ldb[i], (int)ldc[i],
                              accumulate[i] & HB_GEMM_ACCUMULATE, alpha_acc[i], beta_c[i], 0, nullptr, 0};
    grp.tile_begin[grp.n + 1] = grp.tile_begin[grp.n] + (int)tiles;
    ++grp.n;
  }
  flush();
  return check_launch("hb_gemm_f32_grouped");
}

extern "C" int hb_adam_precond(float* exp_avg, float* exp_avg_sq, const float* grad, float* out, int64_t n, float a1, float one_minus_a1, float a2,
                               float one_minus_a2, float eps, void* stream_) {
  using namespace hb;
  if (n < 0) return set_error(HB_EINVAL, "hb_adam_precond: negative size");
  if (n == 0) return HB_OK;
  if (!exp_avg || !exp_avg_sq || !grad || !out) return set_error(HB_EINVAL, "hb_adam_precond: null pointer");
  const int64_t blocks = (n + 255) / 256;
  adam_precond_kernel<<<(unsigned)(blocks > 65536 ? 65536 : blocks), 256, 0, static_cast<hipStream_t>(stream_)>>>(
      exp_avg, exp_avg_sq, grad, out, n, a1, one_minus_a1, a2, one_minus_a2, eps);
  return check_launch("hb_adam_precond");
}

extern "C" int hb_adam_precond_grouped(int32_t count, float* const* exp_avg, float* const* exp_avg_sq, const float* const* grad, float* const* out,
                                       const int64_t* n, float a1, float one_minus_a1, float a2, float one_minus_a2, float eps, void* stream_) {
  using namespace hb;
  if (count < 0) return set_error(HB_EINVAL, "hb_adam_precond_grouped: negative count");
  if (count == 0) return HB_OK;
  if (!exp_avg || !exp_avg_sq || !grad || !out || !n) return set_error(HB_EINVAL, "hb_adam_precond_grouped: null pointer");
  hipStream_t s = static_cast<hipStream_t>(stream_);
  AdamGroup grp;
  grp.count = 0;
  grp.block_begin[0] = 0;
  grp.a1 = a1; grp.oma1 = one_minus_a1; grp.a2 = a2; grp.oma2 = one_minus_a2; grp.eps = eps;
  auto flush = [&]() {
    if (grp.count == 0) return;
    adam_precond_group_kernel<<<(unsigned)grp.block_begin[grp.count], 256, 0, s>>>(grp);
    grp.count = 0;
  };
  for (int t = 0; t < count; ++t) {
    if (n[t] < 0) return set_error(HB_EINVAL, "hb_adam_precond_grouped: negative size at %d", t);
    if (n[t] == 0) continue;
    if (!exp_avg[t] || !exp_avg_sq[t] || !grad[t] || !out[t]) return set_error(HB_EINVAL, "hb_adam_precond_grouped: null pointer at %d", t);
    const int64_t want = (n[t] + 255) / 256;
    const int blocks = (int)(want > 16384 ? 16384 : want);
    if (grp.count == kMaxAdamGroup || grp.block_begin[grp.count] + blocks > (1 << 22)) flush();
    const int k = grp.count++;
    grp.m[k] = exp_avg[t]; grp.v[k] = exp_avg_sq[t]; grp.g[k] = grad[t]; grp.out[k] = out[t]; grp.n[k] = n[t];
    grp.block_begin[k + 1] = grp.block_begin[k] + blocks;
  }
  flush();
  return check_launch("hb_adam_precond_grouped");
}

extern "C" int hb_orthonormalize_workspace_bytes(int64_t m, int64_t n, int64_t* bytes) {
  using namespace hb;
  if (m <= 0 || n <= 0 || n > m || !bytes) return set_error(HB_EINVAL, "hb_orthonormalize_workspace_bytes: bad arguments (need 0 < n <= m)");
  *bytes = (int64_t)ortho_plan(m, n).total;
  return HB_OK;
}

// The factorisation of n_mats matrices of one shape, every launch covering all of them (blockIdx.z / .y picks the problem).
static int orthonormalize_impl(const char* who, int n_mats, float* const* Q, int64_t m, int64_t n, int64_t ld, void* const* workspace,
                               int64_t workspace_bytes, int32_t* const* status, hipStream_t s) {
  using namespace hb;
  if (n_mats < 1 || n_mats > kMaxBatch) return set_error(HB_EINVAL, "%s: 1 to %d matrices per call", who, kMaxBatch);
  if (!Q || !workspace || !status) return set_error(HB_EINVAL, "%s: null pointer", who);
  if (m <= 0 || n <= 0 || n > m || ld < n || m > (1 << 20)) return set_error(HB_EINVAL, "%s: bad shape (need 0 < n <= m, ld >= n)", who);
  const OrthoPlan p = ortho_plan(m, n);
  if ((int64_t)p.total > workspace_bytes) return set_error(HB_EINVAL, "%s: workspace too small", who);
  Batch bt{};
  bt.n = n_mats;
  for (int z = 0; z < n_mats; ++z) {
    if (!Q[z] || !workspace[z] || !status[z]) return set_error(HB_EINVAL, "%s: null pointer", who);
    if ((reinterpret_cast<uintptr_t>(workspace[z]) & 255) != 0) return set_error(HB_EINVAL, "%s: workspace must be 256-byte aligned", who);
    if ((reinterpret_cast<uintptr_t>(Q[z]) & 3) != 0) return set_error(HB_EINVAL, "%s: matrix must be 4-byte aligned", who);
    bt.dq[z] = (int64_t)(reinterpret_cast<intptr_t>(Q[z]) - reinterpret_cast<intptr_t>(Q[0]));
    bt.dws[z] = (int64_t)(reinterpret_cast<intptr_t>(workspace[z]) - reinterpret_cast<intptr_t>(workspace[0]));
    bt.status[z] = status[z];
  }
  // the 128-bit paths of the kernels test the alignment of problem 0's pointers: every matrix must agree with it
  for (int z = 1; z < n_mats; ++z)
    if ((bt.dq[z] & 15) != 0) return set_error(HB_EINVAL, "%s: the matrices of one call must share their alignment modulo 16 bytes", who);
  float* Q0 = Q[0];
  char* ws = static_cast<char*>(workspace[0]);
  float* Cb = reinterpret_cast<float*>(ws + p.off_c);
  float* G = reinterpret_cast<float*>(ws + p.off_g);
  float* part = reinterpret_cast<float*>(ws + p.off_part);
  constexpr int trsm_lds = kTrsmLds;
  static LdsReservation reserved;
  const void* trsm = reinterpret_cast<const void*>(trsm_right_upper_kernel);
  if (int rc = reserve_lds(reserved, &trsm, 1, trsm_lds, who)) return rc;
  set_status_kernel<<<1, 64, 0, s>>>(bt, 0);  // a kernel, not a memset node, so that callers may capture the call in a graph
  const int M = (int)m, LD = (int)ld;
  for (int j0 = 0; j0 < (int)n; j0 += kPanel) {
    const int w = (int)n - j0 < kPanel ? (int)n - j0 : kPanel;
    float* P = Q0 + j0;
    for (int pass = 0; pass < 2; ++pass) {  // everything twice: one round of Gram-Schmidt loses orthogonality in fp32
      if (j0 > 0) {
        // C = Qprev^T P ;  P -= Qprev C
        SgemmArgs a{Q0, P, Cb, j0, w, M, LD, LD, w, 0, 0.0f, 0.0f, 0, nullptr};
        sgemm_launch(a, true, false, part, p.part_elems, s, bt, kCInWs);
        SgemmArgs b{Q0, Cb, P, M, w, j0, LD, w, LD, 1, -1.0f, 1.0f, 0, nullptr};
        sgemm_launch(b, false, false, part, p.part_elems, s, bt, kBInWs);
      }
      // Cholesky QR of the panel: G = P^T P = R^T R ;  P <- P R^-1
      SgemmArgs c{P, P, G, w, w, M, LD, LD, w, 0, 0.0f, 0.0f, 0, nullptr};
      sgemm_launch(c, true, false, part, p.part_elems, s, bt, kCInWs);
      chol_kernel<<<n_mats, kCholThreads, 0, s>>>(G, w, bt);
      trsm_right_upper_kernel<<<dim3((M + kTrsmRows - 1) / kTrsmRows, n_mats), 256, trsm_lds, s>>>(P, LD, M, G, w, bt);
    }
  }
  return check_launch(who);
}

extern "C" int hb_orthonormalize_f32(float* Q, int64_t m, int64_t n, int64_t ld, void* workspace, int64_t workspace_bytes, int32_t* status,
                                     void* stream_) {
  return orthonormalize_impl("hb_orthonormalize_f32", 1, &Q, m, n, ld, &workspace, workspace_bytes, &status, static_cast<hipStream_t>(stream_));
}

extern "C" int hb_orthonormalize_f32_batched(int32_t n_mats, float* const* Q, int64_t m, int64_t n, int64_t ld, void* const* workspace,
                                             int64_t workspace_bytes, int32_t* const* status, void* stream_) {
  return orthonormalize_impl("hb_orthonormalize_f32_batched", n_mats, Q, m, n, ld, workspace, workspace_bytes, status,
                             static_cast<hipStream_t>(stream_));
}
