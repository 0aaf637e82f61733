// Newton-Schulz orthogonalisation for Muon on gfx950 (MI355X): bf16 MFMA GEMMs with fused epilogues.
//
// Reference: zeropower_via_newtonschulz5 (heavyball/utils.py:550-577), its legacy variant (:637-657) and the dispatcher
// with the max(1, rows/cols)^0.5 post-scale (:784-817).  Per iteration the reference runs
//     s = x @ x^T ;  y = c*s ; y.diag += b ;  y = y @ s ; y.diag += a ;  x = y @ x
// with every intermediate rounded to bf16.  Here each product is one launch of the same "NT" GEMM kernel
// (C[i,j] = sum_k A[i,k] * B[j,k], both operands K-contiguous):
//     S , Y  = gemm(X , X )      epilogue: S = bf16(acc); Y = bf16(c * S) (+ b on the diagonal, rounded again)
//     Y2     = gemm(Y , S )      S is symmetric bit for bit, so its rows serve as the K-contiguous operand
//     X', X't = gemm(Y2, X^T)    epilogue writes the result in both orientations, so the next iteration has X^T
// so no operand ever has to be transposed on its way into the matrix cores.
//
// S and Y2 (a polynomial in S) are symmetric: only the upper triangle of their tiles is computed, each off-diagonal tile
// is also written transposed.  Every product is ONE grouped launch over the tiles of all matrices of a batch, so the
// half-empty grids of the symmetric products and small matrices fill the GPU together.
//
// Kernel: workgroup tile BM x BN x BK, waves in a WGM x WGN grid, each wave accumulating (BM/WGM) x (BN/WGN) in
// 32x32x16 bf16 MFMA tiles (fp32 accumulators in AGPRs).  Operand tiles travel global -> LDS directly
// (global_load_lds, 16 bytes per lane) into a ring of STAGES slots, all of them in flight; LDS rows have their 16-byte
// chunks XOR-swizzled with the row index, which makes the 128-bit fragment reads (lane = row, 8 consecutive k)
// conflict free.  Fragment reads and loads are issued one per MFMA, in the shadow of the matrix instruction; one
// barrier per K-tile.
#include <algorithm>
#include <cstring>
#include <functional>
#include <vector>

#include "hb_device.h"
#include "hb_host.h"

namespace hb {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));


// kModePartial: raw fp32 product of one K chunk.  kModeFinalX: kModeFinal with the rarer epilogues (a float16 update buffer, the
// parameter step applied in place); they live in a kernel of their own so that the common last product stays as small as it was
// (with them inside, the 256-wide kernel's plain last product took 11 % longer).
enum { kModeS = 0, kModeY2 = 1, kModeX = 2, kModeFinal = 3, kModePartial = 4, kModeFinalX = 5 };

// One entry of a grouped launch: a run of consecutive tiles of one matrix, on one XCD (see locate_tile).  A launch multiplies
// any number of independent matrices.
struct Problem {
  const uint16_t* A;  // [M, K], row stride lda
  const uint16_t* B;  // [N, K], row stride ldb
  uint16_t* C;        // primary bf16 output [M, N] (S, Y2 or X)
  uint16_t* C2;       // ModeS: Y [M, N];  ModeX: X^T [N, M]
  float* F;           // ModeFinal: fp32 output, [M, N] or transposed [N, M]
  int K, lda, ldb, ldc, ldc2, ldf;
  int f_rows, f_cols, f_transposed;  // valid extent of F (the workspace is padded to tile multiples)
  float scale;                       // ModeFinal: post-scale
  float mul_c, diag;                 // ModeS: c and b; ModeY2: diag = a (per matrix: one launch may mix coefficient schedules)
  int tiles_m, tiles_n;              // tile grid of C
  int pos_begin;                     // where this run starts in the tile list of its XCD
  int t0, n_run;                     // the run: tiles t0 .. t0 + n_run - 1 of the matrix' tile list
  // ModeFinal.  Bits 0-1: the reference's update buffer is 16 bits wide (1 bf16, 2 fp16): cast and scaling round to it (to nearest).
  // kApplyToParam: F is the parameter and takes the step instead of receiving the update (mul_c, diag: its two factors).
  int round_out;
};
static_assert(sizeof(Problem) % 16 == 0, "tables of problems are moved in 16-byte pieces");
enum : int { kApplyToParam = 4, kCautiousWd = 8 };  // bits of Problem::round_out beside the update format

// A table: this header, then the entries of XCD 0, of XCD 1, ...; entries [first[x], first[x + 1]) are XCD x's, in list order
struct TableHeader {
  int first[9];
  int pad_[7];
};
static_assert(sizeof(TableHeader) == 64, "the entries start 16-byte aligned");

// LDS tile layout: one row of BK bf16 (BK*2 bytes) per matrix row, its 16-byte chunks XOR-swizzled so that the 128-bit
// fragment reads are conflict free.  A wavefront's ds_read_b128 is served 16 lanes (256 B, all 64 banks) per cycle and
// those 16 lanes read 16 consecutive rows at the same k-chunk; 256 B hold RP = 256/(BK*2) rows, so rotating the chunk
// index by (row / RP) spreads the 16 rows over all 16 chunk slots of the bank period.
template <int BK>
__device__ __forceinline__ uint32_t lds_off(int row, int chunk) {
  constexpr int CPR = BK / 8;         // 16-byte chunks per row
  constexpr int RP = 256 / (BK * 2);  // rows per 256-byte bank period
  return (uint32_t)(row * (BK * 2) + ((chunk ^ ((row / RP) & (CPR - 1))) << 4));
}

typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// Workgroup -> (matrix, tile).  Workgroup ids go round-robin over the 8 XCDs (each with its own L2), so XCD x runs the ids
// congruent to x, in order: id b is position b / 8 of XCD (b % 8)'s tile list.  The host fills these lists (gemm_stage):
//   * a matrix with many tiles hands XCD x the x-th eighth of its tile list, a contiguous run: consecutive tiles share an
//     operand panel, so the panels an XCD touches at a time stay few;
//   * a matrix with few tiles (the 128-wide class) goes to ONE XCD as a whole: its tiles start together and walk K in step, so
//     each panel comes into that XCD's L2 once and serves every tile that needs it.  Dealt out in eighths, every XCD fetches
//     nearly every panel (a 6 x 6 triangle touches 5 of its 6 panels per XCD) and the products of a GPT-2-sized bucket run at
//     the pace of the memory-side traffic instead of the matrix cores';
//   * every list is ordered longest K first (the hardware starts workgroups in id order, so the long tiles start first and
//     the short ones fill in behind them), and the lists carry equal work (longest-processing-time assignment).
// In the symmetric modes the tile list of a matrix is the upper triangle of the grid, in strips.
//
// The lists live in a table in device memory, written before the first product of a call (a bucket of a GPT-2-sized model
// has more matrices than a kernel argument holds, and one launch over all of them balances where two launches each end in a
// half-empty round).  The table is read-only while a product runs, so it is read through the constant address space, i.e.
// with scalar loads; the entry of a workgroup is found by bisection.
typedef const __attribute__((address_space(4))) Problem* table_ptr_t;
typedef const __attribute__((address_space(4))) TableHeader* header_ptr_t;

template <bool SYMMETRIC>
__device__ __forceinline__ bool locate_tile(const void* table, int bid, table_ptr_t& g, int& pi, int& bi, int& bj) {
  const header_ptr_t hdr = (header_ptr_t) reinterpret_cast<uintptr_t>(table);
  g = (table_ptr_t)(reinterpret_cast<uintptr_t>(table) + sizeof(TableHeader));
  const int x = bid & 7, pos = bid >> 3;
  int lo = hdr->first[x], hi = hdr->first[x + 1] - 1;
  if (lo > hi) return false;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (pos >= g[mid].pos_begin) lo = mid;
    else hi = mid - 1;
  }
  pi = lo;
  const int local = pos - g[pi].pos_begin;
  if (local >= g[pi].n_run) return false;  // past the end of a list that is shorter than the longest one
  const int t = g[pi].t0 + local;
#ifndef HB_NS_STRIP
#define HB_NS_STRIP 4
#endif
  constexpr int kStrip = HB_NS_STRIP;
  if (SYMMETRIC) {
    // upper triangle in strips of kStrip tile rows; inside a strip column by column (the first columns of a strip are
    // cut by the diagonal), so that a run of consecutive tiles is a compact block here too
    const int T = g[pi].tiles_n;
    int first = 0, rem = t;
    for (;;) {
      const int h = T - first < kStrip ? T - first : kStrip;
      const int count = h * (h + 1) / 2 + (T - first - h) * h;
      if (rem < count) break;
      rem -= count;
      first += kStrip;
    }
    const int h = T - first < kStrip ? T - first : kStrip;
    int col = first, in_col = 1;  // column `first + k` of the strip holds min(k + 1, h) tiles
    while (rem >= in_col) {
      rem -= in_col;
      ++col;
      if (in_col < h) ++in_col;
    }
    bi = first + rem;
    bj = col;
  } else {
    // strips of kStrip tile rows, walked column by column: a run of consecutive tiles then covers a compact block
    // (kStrip rows x run/kStrip columns) and shares few operand panels
    const int tiles_m = g[pi].tiles_m, tiles_n = g[pi].tiles_n;
    const int strip = t / (kStrip * tiles_n), in_strip = t % (kStrip * tiles_n);
    const int first = strip * kStrip;
    const int height = tiles_m - first < kStrip ? tiles_m - first : kStrip;
    bi = first + in_strip % height;
    bj = in_strip / height;
  }
  return true;
}

// s_waitcnt lgkmcnt(N) only.  The fragment reads below are issued through inline assembly, so the compiler neither
// tracks them nor inserts waits for them: without that it waits for *all* outstanding LDS reads (lgkmcnt(0)) before
// every group of MFMAs, which serialises the next step's fragment traffic with this step's matrix work.
template <int N>
__device__ __forceinline__ void wait_lgkmcnt() {
  static_assert(N >= 0 && N <= 15, "4-bit counter");
  __builtin_amdgcn_s_waitcnt(0xC07F | (N << 8));
}

__device__ __forceinline__ bf16x8 lds_read_b128(uint32_t addr) {
  bf16x8 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr));
  return v;
}

__device__ __forceinline__ void wait_vmcnt(int n) {  // s_waitcnt vmcnt(n) only (expcnt, lgkmcnt left alone)
  switch (n) {
    case 0: __builtin_amdgcn_s_waitcnt(0x0F70); break;
    case 4: __builtin_amdgcn_s_waitcnt(0x0F74); break;
    case 8: __builtin_amdgcn_s_waitcnt(0x0F78); break;
    case 12: __builtin_amdgcn_s_waitcnt(0x0F7C); break;
    case 16: __builtin_amdgcn_s_waitcnt(0x4F70); break;
    case 20: __builtin_amdgcn_s_waitcnt(0x4F74); break;
    case 24: __builtin_amdgcn_s_waitcnt(0x4F78); break;
    case 32: __builtin_amdgcn_s_waitcnt(0x8F70); break;
    default: __builtin_amdgcn_s_waitcnt(0x0F70); break;
  }
}

// The epilogue of both product kernels.  Accumulator register r of tile (i, j) of a wavefront holds row
// (r/4)*8 + (lane/32)*4 + r%4, column lane%32 of the 32 x 32 block.
//
// VIA_LDS (the 128-wide class): the row-major bf16 outputs go through a wavefront-private piece of LDS (`stage`, WTM rows of
// WTN * 2 + 16 bytes) and leave as 16-byte stores, 4 per wavefront and output instead of 32 two-byte ones.  With k-loops of a
// few hundred the epilogue is a third of a tile's time, and what it costs is the number of store instructions in the queue that
// the co-resident workgroup's loads share, not their addresses.  The caller has passed a barrier since the last fragment read.
template <int MODE, int TM, int TN, int WTM, int WTN, bool VIA_LDS = false>
__device__ __forceinline__ void ns_epilogue(floatx16 (&acc)[TM][TN], const Problem& g, const int row0, const int col0,
                                            const int wm, const int wn, const int lane, const int bi, const int bj, char* stage = nullptr) {
  constexpr bool SYMMETRIC = MODE == kModeS || MODE == kModeY2;
  constexpr bool BF16_OUT = MODE == kModeS || MODE == kModeY2 || MODE == kModeX;
  constexpr int PITCH = WTN * 2 + 16;
  const int erow = (lane >> 5) * 4, lcol = lane & 31;
  // the wavefront's WTM x WTN block from `stage` to row-major `base`: a lane moves 16 bytes, WTN / 8 lanes a row
  auto flush_rows = [&](uint16_t* base, int ld) {
    constexpr int PPR = WTN / 8;
    static_assert(WTM * PPR % 64 == 0, "whole wavefront passes");
#pragma unroll
    for (int k = 0; k < WTM * PPR / 64; ++k) {
      const int p = lane + 64 * k, r = p / PPR, part = p % PPR;
      const uint4 w = *reinterpret_cast<const uint4*>(stage + r * PITCH + part * 16);
      *reinterpret_cast<uint4*>(base + (size_t)(row0 + wm * WTM + r) * ld + col0 + wn * WTN + part * 8) = w;
    }
  };
  // Transposed copies (X^T, the mirror of a symmetric tile).  A lane holds 4 + 4 + 4 + 4 rows of one column, lane + 32 the
  // rows between them; v_permlane32_swap trades halves so that a lane below 32 ends up with rows 0..15 of its column and
  // its partner with rows 16..31, 32 contiguous bytes of the transposed matrix each (64 per column) instead of 8.
  auto store_transposed = [&](uint16_t* base, int ld, int col, int row_tile, const uint32_t (&v)[16]) {
    uint32_t pk[4][2], out[8];
#pragma unroll
    for (int rb4 = 0; rb4 < 4; ++rb4) {
      pk[rb4][0] = v[rb4 * 4 + 0] | (v[rb4 * 4 + 1] << 16);
      pk[rb4][1] = v[rb4 * 4 + 2] | (v[rb4 * 4 + 3] << 16);
    }
#pragma unroll
    for (int h = 0; h < 2; ++h)  // h = 0: rows 0-7 | 16-23, h = 1: rows 8-15 | 24-31
#pragma unroll
      for (int w = 0; w < 2; ++w) {
        const auto sw = __builtin_amdgcn_permlane32_swap(pk[h][w], pk[h + 2][w], false, false);
        out[h * 4 + w] = sw[0];      // rows +0..3 of the octet
        out[h * 4 + 2 + w] = sw[1];  // rows +4..7
      }
    uint4* dst = reinterpret_cast<uint4*>(base + (size_t)col * ld + row_tile + (lane >> 5) * 16);
    dst[0] = make_uint4(out[0], out[1], out[2], out[3]);
    dst[1] = make_uint4(out[4], out[5], out[6], out[7]);
  };
  // VIA_LDS in ModeS: two passes, S and then Y, through the one staging block
  constexpr int PASSES = VIA_LDS && MODE == kModeS ? 2 : 1;
#pragma unroll
  for (int pass = 0; pass < PASSES; ++pass) {
#pragma unroll
  for (int i = 0; i < TM; ++i) {
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int col = col0 + wn * WTN + j * 32 + lcol;
      const int row_tile = row0 + wm * WTM + i * 32;
      uint32_t prim[16], sec[16];
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int row = row_tile + (q >> 2) * 8 + erow + (q & 3);
        uint32_t h = f32_to_bf16_rne(acc[i][j][q]);
        if (MODE == kModeS) {
          uint32_t y = f32_to_bf16_rne(bf16_to_f32(h) * g.mul_c);       // heavyball/utils.py:569
          if (row == col) y = f32_to_bf16_rne(bf16_to_f32(y) + g.diag);  // :570
          sec[q] = y;
        } else if (MODE == kModeY2) {
          if (row == col) h = f32_to_bf16_rne(bf16_to_f32(h) + g.diag);  // :572
        }
        prim[q] = h;
      }
      // kApplyToParam: F is the fp32 parameter and takes p <- p * (1 - decay * lr) + update * (-lr), the tail of the reference's
      // chain (heavyball/utils.py:2373-2390; the two factors travel in mul_c and diag, which this mode has no other use for), with
      // the decay factor 1 where update and parameter disagree in sign under kCautiousWd.  The sub-tile's 16 parameter values
      // are read before any of them is written, so that the loads are in flight together.
      const bool apply = MODE == kModeFinalX && (g.round_out & kApplyToParam) != 0;
      float pv[16];
      if (MODE == kModeFinalX && apply) {
#pragma unroll
        for (int rb4 = 0; rb4 < 4; ++rb4) {
          const int row = row_tile + rb4 * 8 + erow;
          if (g.f_transposed) {
            const float* src = g.F + (size_t)col * g.ldf + row;
            if (col < g.f_rows && row + 3 < g.f_cols && (reinterpret_cast<uintptr_t>(src) & 15) == 0) {
              const float4 p4 = *reinterpret_cast<const float4*>(src);
              pv[rb4 * 4 + 0] = p4.x; pv[rb4 * 4 + 1] = p4.y; pv[rb4 * 4 + 2] = p4.z; pv[rb4 * 4 + 3] = p4.w;
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r) pv[rb4 * 4 + r] = col < g.f_rows && row + r < g.f_cols ? src[r] : 0.0f;
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) pv[rb4 * 4 + r] = row + r < g.f_rows && col < g.f_cols ? g.F[(size_t)(row + r) * g.ldf + col] : 0.0f;
          }
        }
      }
      auto stepped = [&](float p, float u) {
        float om = g.mul_c;
        if ((g.round_out & kCautiousWd) && ((f2u(p) ^ f2u(u)) >> 31)) om = 1.0f;
        return p * om + u * g.diag;
      };
#pragma unroll
      for (int rb4 = 0; rb4 < 4; ++rb4) {
        const int row = row_tile + rb4 * 8 + erow;
        if (MODE == kModeFinal || MODE == kModeFinalX || MODE == kModePartial) {
          float o[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            if (MODE == kModePartial) {
              o[r] = acc[i][j][rb4 * 4 + r];  // one K chunk of a split product: summed and rounded by ns_split_reduce_kernel
            } else {
              o[r] = bf16_to_f32(prim[rb4 * 4 + r]) * g.scale;  // x.to(G.dtype) then y *= scale (heavyball/utils.py:577, :808-809)
              if ((g.round_out & 3) == 1) o[r] = bf16_to_f32(f32_to_bf16_rne(o[r]));  // ... in bf16 when G is bf16
              else if (MODE == kModeFinalX && (g.round_out & 3) == 2)  // fp16: the cast leaves bf16's range (subnormals, overflow), then the product rounds again
                o[r] = f16_to_f32(f32_to_f16_rne(f16_to_f32(f32_to_f16_rne_plain(bf16_to_f32(prim[rb4 * 4 + r]))) * g.scale));
            }
          }
          if (MODE == kModeFinalX && apply) {
#pragma unroll
            for (int r = 0; r < 4; ++r) o[r] = stepped(pv[rb4 * 4 + r], o[r]);
          }
          if (g.f_transposed) {
            // the 4 consecutive rows of X are 16 contiguous bytes of the output's row `col`
            float* dst = g.F + (size_t)col * g.ldf + row;
            if (col < g.f_rows && row + 3 < g.f_cols && (reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
              *reinterpret_cast<float4*>(dst) = make_float4(o[0], o[1], o[2], o[3]);
            } else {
#pragma unroll
              for (int r = 0; r < 4; ++r)
                if (col < g.f_rows && row + r < g.f_cols) dst[r] = o[r];
            }
          } else {
#pragma unroll
            for (int r = 0; r < 4; ++r)
              if (row + r < g.f_rows && col < g.f_cols) g.F[(size_t)(row + r) * g.ldf + col] = o[r];
          }
        } else if (VIA_LDS) {
#pragma unroll
          for (int r = 0; r < 4; ++r)
            *reinterpret_cast<uint16_t*>(stage + (i * 32 + rb4 * 8 + erow + r) * PITCH + (j * 32 + lcol) * 2) =
                (uint16_t)(pass == 0 ? prim[rb4 * 4 + r] : sec[rb4 * 4 + r]);
        } else {
#pragma unroll
          for (int r = 0; r < 4; ++r) g.C[(size_t)(row + r) * g.ldc + col] = (uint16_t)prim[rb4 * 4 + r];
          if (MODE == kModeS) {
#pragma unroll
            for (int r = 0; r < 4; ++r) g.C2[(size_t)(row + r) * g.ldc2 + col] = (uint16_t)sec[rb4 * 4 + r];
          }
        }
      }
      if (pass == 0) {
        if constexpr (MODE == kModeX) store_transposed(g.C2, g.ldc2, col, row_tile, prim);  // X^T, the B operand of the next iteration
        // Symmetric modes: a tile above the diagonal is also written transposed to its place below it.  Diagonal tiles
        // are computed in full, so a matrix that fits one tile gets the plain product.
        if (SYMMETRIC && bi != bj) {
          store_transposed(g.C, g.ldc, col, row_tile, prim);
          if constexpr (MODE == kModeS) store_transposed(g.C2, g.ldc2, col, row_tile, sec);
        }
      }
    }
  }
  if constexpr (VIA_LDS && BF16_OUT) flush_rows(pass == 0 ? g.C : g.C2, pass == 0 ? g.ldc : g.ldc2);
  }
}

template <int BM, int BN, int BK, int STAGES, int WGM, int WGN, int MODE>
__global__ __launch_bounds__(WGM* WGN * 64) void ns_gemm_kernel(const void* table) {
  constexpr int NW = WGM * WGN;
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  constexpr int ROWB = BK * 2;                   // bytes per LDS row
  constexpr int CPR = BK / 8;                    // 16-byte chunks per row
  constexpr int RPL = 1024 / ROWB;               // rows moved by one direct-to-LDS load (64 lanes x 16 B)
  constexpr int STAGE = (BM + BN) * ROWB;
  constexpr int LOADS = (BM + BN) / RPL / NW;    // loads per wave per K-tile
  constexpr int KS = BK / 16;                    // MFMA k-steps per K-tile
  static_assert((BM + BN) % (RPL * NW) == 0 && BM % RPL == 0, "tile rows must split evenly over the waves");
  static_assert(STAGES >= 2 && STAGES <= 4 && (STAGES == 2 || LOADS % 4 == 0) && 2 * LOADS <= 32 && KS % 2 == 0 && TM + TN <= 15, "pipeline bookkeeping");
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  constexpr bool SYMMETRIC = MODE == kModeS || MODE == kModeY2 || MODE == kModePartial;  // the tile list is the upper triangle
  int pi, bi, bj;
  table_ptr_t ka;
  if (!locate_tile<SYMMETRIC>(table, blockIdx.x, ka, pi, bi, bj)) return;  // an id past the end of its XCD's list: the whole workgroup leaves
  Problem g;
  g.A = ka[pi].A; g.B = ka[pi].B; g.C = ka[pi].C; g.C2 = ka[pi].C2; g.F = ka[pi].F;
  g.K = ka[pi].K; g.lda = ka[pi].lda; g.ldb = ka[pi].ldb; g.ldc = ka[pi].ldc; g.ldc2 = ka[pi].ldc2; g.ldf = ka[pi].ldf;
  g.f_rows = ka[pi].f_rows; g.f_cols = ka[pi].f_cols; g.f_transposed = ka[pi].f_transposed; g.scale = ka[pi].scale;
  g.mul_c = ka[pi].mul_c; g.diag = ka[pi].diag; g.round_out = ka[pi].round_out;
  const int row0 = bi * BM, col0 = bj * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WGN, wn = wave % WGN;

  // Direct global -> LDS loads: one instruction moves 64 x 16 B into 1 KiB of consecutive LDS, i.e. RPL rows.
  // Lane l lands in row l/CPR, slot l%CPR, so it fetches the k-chunk that the swizzle keeps in that slot.
  // Rows [0, BM) are A's, rows [BM, BM+BN) are B's; wave w owns row groups w*LOADS .. w*LOADS+LOADS-1.
  const int lrow = lane / CPR, lslot = lane % CPR;
  const uint16_t* gsrc[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int r = (wave * LOADS + i) * RPL + lrow;  // row in the combined A||B tile
    const int chunk = lslot ^ ((r / (256 / ROWB)) & (CPR - 1));
    gsrc[i] = r < BM ? g.A + (size_t)(row0 + r) * g.lda + chunk * 8 : g.B + (size_t)(col0 + r - BM) * g.ldb + chunk * 8;
  }
  auto issue_loads = [&](int kt) {
    char* dst = smem + (kt % STAGES) * STAGE + (wave * LOADS) * 1024;
#pragma unroll
    for (int i = 0; i < LOADS; ++i) __builtin_amdgcn_global_load_lds((gptr_t)(gsrc[i] + kt * BK), (lptr_t)(dst + i * 1024), 16, 0, 0);
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int KT = g.K / BK;
  const int frag_row = lane & 31, frag_k = lane >> 5;
  bf16x8 af[2][TM], bfr[2][TN];
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lptr_t)smem;
  auto read_frags = [&](int kt, int ks, int set) {
    const uint32_t sa = smem_base + (kt % STAGES) * STAGE + (wm * WTM) * ROWB;
    const uint32_t sb = smem_base + (kt % STAGES) * STAGE + BM * ROWB + (wn * WTN) * ROWB;
#pragma unroll
    for (int i = 0; i < TM; ++i) af[set][i] = lds_read_b128(sa + lds_off<BK>(i * 32 + frag_row, ks * 2 + frag_k));
#pragma unroll
    for (int j = 0; j < TN; ++j) bfr[set][j] = lds_read_b128(sb + lds_off<BK>(j * 32 + frag_row, ks * 2 + frag_k));
  };
  auto mfma_step = [&](int set) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[set][i], bfr[set][j], acc[i][j], 0, 0, 0);
      }
  };
  // wait until tile t has landed: loads complete in order, so it has once at most `ahead` younger tiles (those issued
  // after it, capped by what exists) are still in flight
  auto wait_tile = [&](int t, int ahead) {
    const int younger = KT - 1 - t < ahead ? KT - 1 - t : ahead;
    if (younger <= 0) wait_vmcnt(0);
    else if (younger == 1) wait_vmcnt(LOADS);
    else if (younger == 2) wait_vmcnt(2 * LOADS);
    else if (younger == 3) wait_vmcnt(3 * LOADS);
    else wait_vmcnt(0);
  };

  // Main loop.  The LDS ring holds STAGES K-tiles: one being multiplied, the others in flight from L2/HBM.  One barrier
  // per K-tile: once through it, tile kt is in LDS for everyone and everyone has finished reading tile kt-1, whose slot
  // then takes tile kt+STAGES-1.  Inside a tile the fragments of k-step s+1 are fetched while step s is multiplied.
  // With eight wavefronts per workgroup (two per SIMD) the hardware interleaves one wavefront's waits with the other's
  // matrix instructions.  This kernel serves the 128 x 128 tile class; the 256 x 256 class runs on ns_gemm4_kernel below.
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s)
    if (s < KT) issue_loads(s);
  for (int kt = 0; kt < KT; ++kt) {
    wait_tile(kt, STAGES - 2);  // tiles up to kt+STAGES-2 have been issued so far
    __syncthreads();
    if (kt + STAGES - 1 < KT) issue_loads(kt + STAGES - 1);
    read_frags(kt, 0, 0);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < KS) {
        read_frags(kt, ks + 1, nxt);
        wait_lgkmcnt<TM + TN>();
      } else {
        wait_lgkmcnt<0>();
      }
      __builtin_amdgcn_sched_barrier(0);
      mfma_step(cur);
      __builtin_amdgcn_sched_barrier(0);
    }
  }

#ifndef HB_NS_EPILOGUE_LDS
#define HB_NS_EPILOGUE_LDS 1
#endif
  constexpr bool kStaged = HB_NS_EPILOGUE_LDS && (MODE == kModeS || MODE == kModeY2 || MODE == kModeX);
  static_assert(!kStaged || NW * WTM * (WTN * 2 + 16) <= STAGES * STAGE, "the staging blocks reuse the ring");
  if (kStaged) __syncthreads();  // everyone has read its last fragments: the ring is free
  ns_epilogue<MODE, TM, TN, WTM, WTN, kStaged>(acc, g, row0, col0, wm, wn, lane, bi, bj, smem + wave * (WTM * (WTN * 2 + 16)));
}

// The 256 x 256 tile class: four wavefronts of 128 x 128 (one per SIMD, accumulators in the accumulation registers),
// K-tiles of 32 in a ring of four.  A wavefront per SIMD has nobody to hide its waits behind, so the instruction stream
// is laid out by hand: every fragment read and every direct-to-LDS load is issued in the shadow of one matrix
// instruction (a 32 x 32 x 16 MFMA occupies the pipe for eight issue slots of the wavefront; at most three other
// instructions follow each one here), and the steady-state loop carries no conditions: the first and the last tiles run
// a conditional copy of the same body.  Per tile and compute unit this moves 64 KB of fragments out of LDS and 32 KB
// into it, against 256 KB + 64 KB per 64 of K for eight wavefronts of 64 x 128, which kept LDS busier than the matrix
// pipes.  One barrier per tile, in its middle: past it, tile kt + 1 has landed for everyone and nobody reads tile kt any more
// (the fragments of its second k-step are in registers), so its slot is refilled while that k-step is multiplied.
// The order of the additions into an accumulator is that of ns_gemm_kernel: the two kernels return the same bits.
template <int V>
using ns_ic = std::integral_constant<int, V>;

template <int OFF>
__device__ __forceinline__ bf16x8 lds_read_b128_off(uint32_t addr) {
  static_assert(OFF >= 0 && OFF < 65536, "16-bit offset field");
  bf16x8 v;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "i"(OFF));
  return v;
}

template <int MODE>
__global__ __launch_bounds__(256) void ns_gemm4_kernel(const void* table) {
  constexpr int BM = 256, BN = 256, BK = 32, STAGES = 4, WGN = 2;
  constexpr int WTM = 128, WTN = 128, TM = 4, TN = 4;
  constexpr int ROWB = BK * 2;                  // bytes per LDS row
  constexpr int STAGE = (BM + BN) * ROWB;       // 32 KB: A's 256 rows, then B's
  constexpr int LOADS = 8;                      // direct-to-LDS loads (16 rows each) per wavefront and K-tile: 128 rows of one operand
  extern __shared__ __attribute__((aligned(1024))) char smem[];

  constexpr bool SYMMETRIC = MODE == kModeS || MODE == kModeY2 || MODE == kModePartial;  // the tile list is the upper triangle
  int pi, bi, bj;
  table_ptr_t ka;
  if (!locate_tile<SYMMETRIC>(table, blockIdx.x, ka, pi, bi, bj)) return;
  Problem g;
  g.A = ka[pi].A; g.B = ka[pi].B; g.C = ka[pi].C; g.C2 = ka[pi].C2; g.F = ka[pi].F;
  g.K = ka[pi].K; g.lda = ka[pi].lda; g.ldb = ka[pi].ldb; g.ldc = ka[pi].ldc; g.ldc2 = ka[pi].ldc2; g.ldf = ka[pi].ldf;
  g.f_rows = ka[pi].f_rows; g.f_cols = ka[pi].f_cols; g.f_transposed = ka[pi].f_transposed; g.scale = ka[pi].scale;
  g.mul_c = ka[pi].mul_c; g.diag = ka[pi].diag; g.round_out = ka[pi].round_out;
  const int row0 = bi * BM, col0 = bj * BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WGN, wn = wave % WGN;
  const int KT = g.K / BK;

  // Loads: wavefronts 0 and 1 bring A's rows 0..127 and 128..255, wavefronts 2 and 3 B's.  One instruction moves 16 rows
  // of 64 B: lane l lands in row l / 4, slot l % 4 and fetches the k-chunk that the swizzle keeps in that slot.  The source
  // is a wavefront-uniform base (operand, first row, K-tile) plus a 32-bit lane offset.
  const int half = wave & 1;
  const int ld = wave < 2 ? g.lda : g.ldb;
  const char* base = wave < 2 ? reinterpret_cast<const char*>(g.A + (size_t)(row0 + half * 128) * g.lda)
                              : reinterpret_cast<const char*>(g.B + (size_t)(col0 + half * 128) * g.ldb);
  const int lrow = lane >> 2, lslot = lane & 3;
  uint32_t voff[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int r = i * 16 + lrow;  // row inside the wavefront's 128 (a multiple of 128 further in the tile: the swizzle does not see it)
    voff[i] = (uint32_t)(r * ld * 2 + ((lslot ^ ((r >> 2) & 3)) << 4));
  }
  auto issue_one = [&](int kt, auto i_c) {
    constexpr int i = decltype(i_c)::value;
    char* dst = smem + (kt % STAGES) * STAGE + (wave * LOADS + i) * 1024;
    const char* src = base + (size_t)kt * (BK * 2);
    __builtin_amdgcn_global_load_lds((gptr_t)(src + voff[i]), (lptr_t)dst, 16, 0, 0);
  };

  floatx16 acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  // Fragment addresses: row i * 32 + frag_row of the wavefront's 128, chunk ks * 2 + frag_k, swizzled by (row / 4) & 3, which
  // depends on the lane alone; k-step 1 sits at the address of k-step 0 with bit 5 flipped.  Slots 2 and 3 lie beyond the
  // 16-bit offset field, so they get base registers of their own.
  const int frag_row = lane & 31, frag_k = lane >> 5;
  const uint32_t smem_base = (uint32_t)(uintptr_t)(lptr_t)smem;
  const uint32_t swz = (uint32_t)((frag_k ^ ((frag_row >> 2) & 3)) << 4);
  uint32_t fa[2][2], fb[2][2];  // [k-step][slot / 2]
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      fa[ks][h] = smem_base + h * 2 * STAGE + (wm * WTM + frag_row) * ROWB + (swz ^ (ks << 5));
      fb[ks][h] = smem_base + h * 2 * STAGE + (BM + wn * WTN + frag_row) * ROWB + (swz ^ (ks << 5));
    }
  bf16x8 afr[2][TM], bfr[2][TN];
  // fragment r (0..3: A's, 4..7: B's) of k-step ks of the tile in slot sl, into set
  auto read_one = [&](auto sl_c, auto ks_c, auto set_c, auto r_c) {
    constexpr int sl = decltype(sl_c)::value, ks = decltype(ks_c)::value, set = decltype(set_c)::value, r = decltype(r_c)::value;
    constexpr int off = (sl & 1) * STAGE + (r & 3) * 32 * ROWB;
    if constexpr (r < 4) afr[set][r] = lds_read_b128_off<off>(fa[ks][sl >> 1]);
    else bfr[set][r - 4] = lds_read_b128_off<off>(fb[ks][sl >> 1]);
  };
  // the 16 MFMAs of one k-step on fragment set `cur`; extra(m) is issued right behind MFMA m
  auto mfmas = [&](auto cur_c, auto&& extra) {
    constexpr int cur = decltype(cur_c)::value;
    auto one = [&](auto m_c) {
      constexpr int m = decltype(m_c)::value, i = m / TN, j = m % TN;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(afr[cur][i], bfr[cur][j], acc[i][j], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
      extra(m_c);
      __builtin_amdgcn_sched_barrier(0);
    };
    // nothing moves across this point: the compiler does not know that the wait in front of the k-step is what makes the
    // fragments (read through inline assembly) valid, and would hoist the first MFMA above it
    __builtin_amdgcn_sched_barrier(0);
    one(ns_ic<0>{}); one(ns_ic<1>{}); one(ns_ic<2>{}); one(ns_ic<3>{}); one(ns_ic<4>{}); one(ns_ic<5>{}); one(ns_ic<6>{}); one(ns_ic<7>{});
    one(ns_ic<8>{}); one(ns_ic<9>{}); one(ns_ic<10>{}); one(ns_ic<11>{}); one(ns_ic<12>{}); one(ns_ic<13>{}); one(ns_ic<14>{}); one(ns_ic<15>{});
  };
  // Tile kt, in slot kt % STAGES, its first fragments already in set 0.  STEADY: tiles kt + 1 and kt + STAGES exist, and
  // kt >= 1; otherwise the same body with its conditions.
  auto tile = [&](int kt, auto slot_c, auto steady_c) {
    constexpr int slot = decltype(slot_c)::value;
    constexpr bool STEADY = decltype(steady_c)::value;
    constexpr int nslot = (slot + 1) % STAGES;
    // k-step 0: behind the first eight MFMAs the fragments of k-step 1 (they then have the other eight to arrive in), behind
    // four of the rest the second half of the refill that the tile before began (into the slot that tile left at its barrier)
    wait_lgkmcnt<0>();
    const bool refill0 = kt >= 1 && kt - 1 + STAGES < KT;
    mfmas(ns_ic<0>{}, [&](auto m_c) {
      constexpr int m = decltype(m_c)::value;
      if constexpr (m < 8) read_one(slot_c, ns_ic<1>{}, ns_ic<1>{}, ns_ic<m>{});
      else if constexpr (m % 2 == 1) {
        if (STEADY || refill0) issue_one(kt - 1 + STAGES, ns_ic<4 + (m - 8) / 2>{});
      }
    });
    wait_lgkmcnt<0>();  // every read of tile kt is done
    const bool more = kt + 1 < KT;
    if (STEADY || more) {
      // tile kt + 1 must have landed.  Issued so far: the tiles up to kt - 1 + STAGES; still allowed in flight: those
      // younger than kt + 1 (loads complete in order)
      if constexpr (STEADY) {
        wait_vmcnt((STAGES - 2) * LOADS);
      } else {
        const int last_issued = KT - 1 < kt - 1 + STAGES ? KT - 1 : kt - 1 + STAGES;
        const int younger = last_issued - (kt + 1);
        if (younger <= 0) wait_vmcnt(0);
        else if (younger == 1) wait_vmcnt(LOADS);
        else if (younger == 2) wait_vmcnt(2 * LOADS);
        else wait_vmcnt(0);
      }
      __builtin_amdgcn_s_barrier();
    }
    // k-step 1: behind the first eight MFMAs the first fragments of tile kt + 1, behind four of the rest the first half of
    // the refill of this tile's slot with tile kt + STAGES
    const bool refill = kt + STAGES < KT;
    mfmas(ns_ic<1>{}, [&](auto m_c) {
      constexpr int m = decltype(m_c)::value;
      if constexpr (m < 8) {
        if (STEADY || more) read_one(ns_ic<nslot>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<m>{});
      } else if constexpr (m % 2 == 1) {
        if (STEADY || refill) issue_one(kt + STAGES, ns_ic<(m - 8) / 2>{});
      }
    });
  };
  // prologue: the ring is filled, tile 0 has landed for everyone, its first fragments are on their way
  for (int s = 0; s < STAGES && s < KT; ++s) {
    issue_one(s, ns_ic<0>{}); issue_one(s, ns_ic<1>{}); issue_one(s, ns_ic<2>{}); issue_one(s, ns_ic<3>{});
    issue_one(s, ns_ic<4>{}); issue_one(s, ns_ic<5>{}); issue_one(s, ns_ic<6>{}); issue_one(s, ns_ic<7>{});
  }
  {
    const int younger = (KT < STAGES ? KT : STAGES) - 1;
    if (younger <= 0) wait_vmcnt(0);
    else if (younger == 1) wait_vmcnt(LOADS);
    else if (younger == 2) wait_vmcnt(2 * LOADS);
    else wait_vmcnt(3 * LOADS);
  }
  __builtin_amdgcn_s_barrier();
  read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}); read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<1>{});
  read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<2>{}); read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<3>{});
  read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<4>{}); read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<5>{});
  read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<6>{}); read_one(ns_ic<0>{}, ns_ic<0>{}, ns_ic<0>{}, ns_ic<7>{});
  // the first group conditionally (tile 0 has no refill half behind it), the steady groups while the last tile of a group
  // still has its tile kt + STAGES, the rest conditionally again
  int kt = 0;
  tile(0, ns_ic<0>{}, std::false_type{});
  if (1 < KT) tile(1, ns_ic<1>{}, std::false_type{});
  if (2 < KT) tile(2, ns_ic<2>{}, std::false_type{});
  if (3 < KT) tile(3, ns_ic<3>{}, std::false_type{});
  for (kt = STAGES; kt + 2 * STAGES - 1 < KT; kt += STAGES) {
    tile(kt, ns_ic<0>{}, std::true_type{});
    tile(kt + 1, ns_ic<1>{}, std::true_type{});
    tile(kt + 2, ns_ic<2>{}, std::true_type{});
    tile(kt + 3, ns_ic<3>{}, std::true_type{});
  }
  for (; kt < KT; kt += STAGES) {
    tile(kt, ns_ic<0>{}, std::false_type{});
    if (kt + 1 < KT) tile(kt + 1, ns_ic<1>{}, std::false_type{});
    if (kt + 2 < KT) tile(kt + 2, ns_ic<2>{}, std::false_type{});
    if (kt + 3 < KT) tile(kt + 3, ns_ic<3>{}, std::false_type{});
  }

  ns_epilogue<MODE, TM, TN, WTM, WTN>(acc, g, row0, col0, wm, wn, lane, bi, bj);
}

// ---------------------------------------------------------------------------------------------------------------
// preparation: Frobenius norm, normalise + stochastic round to bf16 into X and X^T (zero padded)
// ---------------------------------------------------------------------------------------------------------------
// One matrix of a grouped preparation launch (the three kernels below share the descriptor).
struct PrepItem {
  const float* g;     // the gradient [rows, cols]
  uint16_t* X;        // [m, n] padded, m <= n
  uint16_t* Xt;       // [n, m] padded
  const double* partial;  // n_blocks partial sums of squares (the call's own scratch, or the caller's)
  float* norm;        // max(||g||_F, eps)
  int64_t flat_base;  // Philox flat index of g[0, 0]
  int rows, cols, ldx, ldxt, transpose;
  int n_blocks, block_begin;  // sum of squares: n_blocks partial sums; this matrix owns workgroups [block_begin, block_begin + sum_blocks)
  int sum_blocks;             // ... n_blocks of them, or none when the caller brought the partial sums
  int tiles_c, tile_begin;    // conversion: 64 x 64 tiles, tiles_c per tile row, first workgroup id
  int legacy;                 // two stochastic rounds (legacy_zeropower_via_newtonschulz5) instead of one
  // the reference's update buffer is 16 bits wide.  1 (bf16): norm and quotient are bf16 values (to nearest), no stochastic round.
  // 2 (fp16): norm and quotient are fp16 values (to nearest), the quotient is then rounded stochastically to bf16.
  int narrow_update;
};
constexpr int kMaxPrep = 28;
struct PrepGroup {
  PrepItem it[kMaxPrep];
  int n_items;
  float eps;
  Rng rng;
};
static_assert(sizeof(PrepGroup) <= 4096, "the group travels as a kernel argument");
typedef const __attribute__((address_space(4))) PrepGroup* prep_ptr_t;

__global__ __launch_bounds__(256) void ns_sumsq_kernel(const PrepGroup grp) {
  const prep_ptr_t ka = (prep_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
  int pi = 0;
  const int n_items = ka->n_items;
  while (pi + 1 < n_items && (int)blockIdx.x >= ka->it[pi + 1].block_begin) ++pi;
  const float* __restrict__ g = ka->it[pi].g;
  const int64_t n = (int64_t)ka->it[pi].rows * ka->it[pi].cols;
  const int nb = ka->it[pi].sum_blocks, b = blockIdx.x - ka->it[pi].block_begin;
  double* __restrict__ partial = const_cast<double*>(ka->it[pi].partial);
  __shared__ double lds[4];
  double acc = 0.0;
  const int64_t n4 = (reinterpret_cast<uintptr_t>(g) & 15) == 0 ? n >> 2 : 0;  // 128-bit loads when the buffer allows
  const float4* g4 = reinterpret_cast<const float4*>(g);
  for (int64_t i = (int64_t)b * 256 + threadIdx.x; i < n4; i += (int64_t)nb * 256) {
    const float4 v = g4[i];
    acc += (double)v.x * (double)v.x + (double)v.y * (double)v.y + (double)v.z * (double)v.z + (double)v.w * (double)v.w;
  }
  for (int64_t i = n4 * 4 + (int64_t)b * 256 + threadIdx.x; i < n; i += (int64_t)nb * 256) {
    const float v = g[i];
    acc += (double)v * (double)v;
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) partial[b] = lds[0] + lds[1] + lds[2] + lds[3];
}

// One workgroup per matrix adds the partial sums in a fixed order.  A caller's partial sums come a few per chunk of 4096
// elements (150 thousand for an embedding of 38 M elements), so the workgroup is 1024 lanes wide and every lane keeps eight loads
// in flight; a lane's terms and the order of the final additions depend on nothing but the count.
constexpr int kNormThreads = 1024;
__global__ __launch_bounds__(kNormThreads) void ns_norm_final_kernel(const PrepGroup grp) {
  const prep_ptr_t ka = (prep_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
  const int pi = blockIdx.x;
  const double* __restrict__ partial = ka->it[pi].partial;
  const int n = ka->it[pi].n_blocks;
  __shared__ double lds[kNormThreads / 64];
  double acc = 0.0;
  for (int i0 = threadIdx.x; i0 < n; i0 += kNormThreads * 8) {
    double v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = i0 + u * kNormThreads < n ? partial[i0 + u * kNormThreads] : 0.0;
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  acc = wave_sum(acc);
  if ((threadIdx.x & 63) == 0) lds[threadIdx.x >> 6] = acc;
  __syncthreads();
  if (threadIdx.x == 0) {
    double total = 0.0;
    for (int k = 0; k < kNormThreads / 64; ++k) total += lds[k];
    float nrm = __builtin_sqrtf((float)total);
    float eps = grp.eps;
    // a 16-bit tensor's norm is a value of its dtype; so is the clamp bound, except under the legacy schedule, whose division
    // promotes both sides to fp32 first (heavyball/utils.py:1174-1179, :1190)
    if (ka->it[pi].narrow_update == 1) {
      nrm = bf16_to_f32(f32_to_bf16_rne(nrm));
      if (!ka->it[pi].legacy) eps = bf16_to_f32(f32_to_bf16_rne(eps));
    } else if (ka->it[pi].narrow_update == 2) {
      nrm = f16_to_f32(f32_to_f16_rne(nrm));  // infinite past 65504: the quotient is then zero, as in the reference
      if (!ka->it[pi].legacy) eps = f16_to_f32(f32_to_f16_rne(eps));
    }
    ka->it[pi].norm[0] = __builtin_fmaxf(nrm, eps);  // G.norm().clamp(min=eps), heavyball/utils.py:555
  }
}

__global__ void ns_zero_kernel(uint4* __restrict__ p, int64_t n16) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n16; i += (int64_t)gridDim.x * blockDim.x) p[i] = make_uint4(0, 0, 0, 0);
}

// x = SR_bf16(g / norm) (default) or SR_bf16(float(SR_bf16(g)) / norm) (legacy, heavyball/utils.py:641-645), written as
// X [m, n] (G itself when rows <= cols, else G^T) and as X^T.  A workgroup converts a 64 x 64 tile of G: each lane
// takes 8 consecutive elements of two rows (two 128-bit loads and one Philox call each when the octet is aligned),
// writes them to the row-major copy as 128-bit stores, and the tile goes through LDS to reach the other copy with
// 128-bit stores too (eight lanes fill one 128-byte line).
__device__ __forceinline__ uint32_t ns_round_one(float v, float nrm, int legacy, const Rng& rng, int64_t flat, const Rand8* aligned) {
  if (legacy == 2) return f32_to_bf16_rne(v / nrm);  // bf16 update buffer: the quotient is a bf16 value already (heavyball/utils.py:2348-2349)
  Rand8 r, r2;
  const int lane8 = (int)(flat & 7);
  if (legacy != 3) {
    if (aligned) r = aligned[0];
    else r = rng.octet(flat & ~int64_t(7), HB_STREAM_NS_INPUT);
    if (legacy == 0) return sr_bf16(v / nrm, r.bits16(lane8));
    if (legacy == 4) return sr_bf16(f16_to_f32(f32_to_f16_rne_plain(v / nrm)), r.bits16(lane8));  // fp16 update buffer: an fp16 quotient
  }
  if (aligned) r2 = aligned[1];
  else r2 = rng.octet(flat & ~int64_t(7), HB_STREAM_NS_INPUT + 1);
  // legacy on a bf16 update buffer (3): its first round is the identity, the fp32 quotient is rounded stochastically
  const uint32_t h = legacy == 3 ? f32_to_bf16_rne(v) : sr_bf16(v, r.bits16(lane8));
  return sr_bf16(bf16_to_f32(h) / nrm, r2.bits16(lane8));
}

__global__ __launch_bounds__(256) void ns_prep_kernel(const PrepGroup grp) {
  const prep_ptr_t ka = (prep_ptr_t)__builtin_amdgcn_kernarg_segment_ptr();
  int pi = 0;
  const int n_items = ka->n_items;
  while (pi + 1 < n_items && (int)blockIdx.x >= ka->it[pi + 1].tile_begin) ++pi;
  const float* __restrict__ g = ka->it[pi].g;
  const int rows = ka->it[pi].rows, cols = ka->it[pi].cols, transpose = ka->it[pi].transpose;
  const int64_t flat_base = ka->it[pi].flat_base;
  // 0: one stochastic round, 1: two (legacy), 2: none (bf16 input), 3: bf16 input under the legacy schedule (one, after the division),
  // 4: fp16 input, one round of the fp16 quotient (under the legacy schedule fp16 input takes 1: only its norm differs)
  const int nu = ka->it[pi].narrow_update;
  const int legacy = nu == 1 ? (ka->it[pi].legacy ? 3 : 2) : nu == 2 && !ka->it[pi].legacy ? 4 : ka->it[pi].legacy;
  const Rng rng = grp.rng;
  __shared__ uint16_t tile[64][64 + 8];  // +8: rows 144 B apart, so the column reads below spread over the banks
  const float nrm = ka->it[pi].norm[0];
  const int tiles_c = ka->it[pi].tiles_c, local = blockIdx.x - ka->it[pi].tile_begin;
  const int ti = local / tiles_c, tj = local % tiles_c;
  // the copy whose rows run along G's rows gets the direct store; the other one the transposed store
  uint16_t* direct = transpose ? ka->it[pi].Xt : ka->it[pi].X;
  const int ldd = transpose ? ka->it[pi].ldxt : ka->it[pi].ldx;
  uint16_t* other = transpose ? ka->it[pi].X : ka->it[pi].Xt;
  const int ldo = transpose ? ka->it[pi].ldx : ka->it[pi].ldxt;
  const int oc = (threadIdx.x & 7) * 8;
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int r = (threadIdx.x >> 3) + 32 * half;
    const int i = ti * 64 + r, j0 = tj * 64 + oc;
    uint32_t h[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) h[e] = 0;
    if (i < rows && j0 < cols) {
      const int64_t f0 = (int64_t)i * cols + j0;
      const bool fast = j0 + 8 <= cols && ((flat_base + f0) & 7) == 0 && (f0 & 3) == 0 && (reinterpret_cast<uintptr_t>(g) & 15) == 0;
      if (fast) {
        const float4 a = *reinterpret_cast<const float4*>(g + f0), b = *reinterpret_cast<const float4*>(g + f0 + 4);
        const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        Rand8 rr[2];
        if (legacy < 2 || legacy == 4) rr[0] = rng.octet(flat_base + f0, HB_STREAM_NS_INPUT);
        if (legacy & 1) rr[1] = rng.octet(flat_base + f0, HB_STREAM_NS_INPUT + 1);
#pragma unroll
        for (int e = 0; e < 8; ++e) h[e] = ns_round_one(v[e], nrm, legacy, rng, flat_base + f0 + e, rr);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (j0 + e < cols) h[e] = ns_round_one(g[f0 + e], nrm, legacy, rng, flat_base + f0 + e, nullptr);
      }
      // direct copy: row i, columns j0 .. j0+7 (the padded leading dimension is a multiple of 128, so this stays in the row)
      *reinterpret_cast<uint4*>(direct + (size_t)i * ldd + j0) =
          make_uint4(h[0] | (h[1] << 16), h[2] | (h[3] << 16), h[4] | (h[5] << 16), h[6] | (h[7] << 16));
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) tile[r][oc + e] = (uint16_t)h[e];
  }
  __syncthreads();
  // transposed copy: a lane handles one column of the tile and 8 consecutive rows; 8 lanes make a full 128-byte line
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    const int jc = (threadIdx.x >> 3) + 32 * half, rc = (threadIdx.x & 7) * 8;
    const int jj = tj * 64 + jc, ii = ti * 64 + rc;
    if (jj < cols && ii < rows) {
      uint32_t t[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) t[e] = tile[rc + e][jc];
      *reinterpret_cast<uint4*>(other + (size_t)jj * ldo + ii) =
          make_uint4(t[0] | (t[1] << 16), t[2] | (t[3] << 16), t[4] | (t[5] << 16), t[6] | (t[7] << 16));
    }
  }
}

// ---------------------------------------------------------------------------------------------------------------
// host
// ---------------------------------------------------------------------------------------------------------------
static inline int64_t round_up(int64_t x, int64_t m) { return (x + m - 1) / m * m; }

// S = X X^T from its K chunks (added in chunk order) with the epilogue of the one-piece product: S rounded to bf16,
// Y = c S + b I with one bf16 rounding per operation (heavyball/utils.py:568-570).  The chunks hold the tiles on and above
// the diagonal; an element below takes the sum of its mirror image, which has the same terms in the same order.
__global__ __launch_bounds__(256) void ns_split_reduce_kernel(const float* __restrict__ part, int chunks, int mp, int tile, uint16_t* __restrict__ S,
                                                              uint16_t* __restrict__ Y, float mul_c, float diag) {
  // one workgroup per 32 x 32 block of a tile on or above the diagonal; a block of a tile above it is also written mirrored,
  // through LDS, so that both copies leave as runs of 32 elements
  const int nb = mp / 32;
  const int br = blockIdx.x / nb, bc = blockIdx.x % nb;
  const int tr = br * 32 / tile, tc = bc * 32 / tile;
  if (tr > tc) return;
  __shared__ uint32_t lds[32][33];
  const int64_t n = (int64_t)mp * mp;
  const int lc = threadIdx.x & 31, lr0 = (threadIdx.x >> 5) * 4;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int r = br * 32 + lr0 + k, col = bc * 32 + lc;
    const int64_t i = (int64_t)r * mp + col;
    float v = 0.0f;
    for (int c = 0; c < chunks; ++c) v += part[(size_t)c * n + i];
    const uint32_t h = f32_to_bf16_rne(v);
    uint32_t y = f32_to_bf16_rne(bf16_to_f32(h) * mul_c);
    if (r == col) y = f32_to_bf16_rne(bf16_to_f32(y) + diag);
    S[i] = (uint16_t)h;
    Y[i] = (uint16_t)y;
    lds[lr0 + k][lc] = h | (y << 16);
  }
  if (tr == tc) return;  // wave-uniform: the whole workgroup leaves
  __syncthreads();
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int col = lr0 + k, r = lc;  // element (r, col) of the block goes to (col, r) of the mirrored block
    const uint32_t w = lds[r][col];
    const int64_t i = (int64_t)(bc * 32 + col) * mp + br * 32 + r;
    S[i] = (uint16_t)(w & 0xFFFFu);
    Y[i] = (uint16_t)(w >> 16);
  }
}

struct NsPlan {
  int64_t rows, cols;    // the gradient as given
  int64_t m, n, mp, np;  // logical and padded dims of X (m <= n)
  int tile;              // 256 or 128
  size_t off_x[2], off_xt[2], off_s, off_y, off_y2, off_partial, off_norm, off_split, total;
  int split, split_chunk;  // S = X X^T in `split` chunks of K (0: in one piece), each `split_chunk` long but the last
};

// Tile class of each matrix: 256 x 256 tiles when the short side is >= 1024, else 128 x 128.  It depends on the shape
// alone (the mirrored tiles of the symmetric products make the rounding depend on the tile size), so a matrix gets the
// same result bit for bit in any batch.
static void choose_tiles(int n_mats, const int64_t* rows, const int64_t* cols, std::vector<int>& tile) {
  tile.resize(n_mats);
#ifndef HB_TILE256_MIN
#define HB_TILE256_MIN 1024
#endif
  for (int i = 0; i < n_mats; ++i) tile[i] = std::min(rows[i], cols[i]) >= HB_TILE256_MIN ? 256 : 128;
}

static NsPlan make_plan(int64_t rows, int64_t cols, int tile) {
  NsPlan p;
  p.rows = rows;
  p.cols = cols;
  p.m = rows <= cols ? rows : cols;
  p.n = rows <= cols ? cols : rows;
  p.tile = tile;
  p.mp = round_up(p.m, p.tile);
  p.np = round_up(p.n, p.tile);
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o += (bytes + 255) & ~size_t(255); return at; };
  for (int k = 0; k < 2; ++k) {  // X and X^T ping-pong: the product that makes the new X still reads the old X^T
    p.off_x[k] = take((size_t)p.mp * p.np * 2);
    p.off_xt[k] = take((size_t)p.np * p.mp * 2);
  }
  p.off_s = take((size_t)p.mp * p.mp * 2);
  p.off_y = take((size_t)p.mp * p.mp * 2);
  p.off_y2 = take((size_t)p.mp * p.mp * 2);
  p.off_partial = take(1024 * sizeof(double));
  p.off_norm = take(256);
  // A short, very wide X (an embedding matrix under a small hidden size) gives S = X X^T a handful of tiles with a k-loop
  // of hundreds of steps each: a few workgroups work for a long time while the rest of the chip idles.  Such a product is
  // cut along K into enough chunks for about two workgroups per compute unit (a multiple of 8 chunks where that many fit:
  // on the 128-wide tiles a chunk stays on one XCD); the chunks leave raw fp32 partial products of the tiles on and above
  // the diagonal and ns_split_reduce_kernel adds them up, mirrors them and applies the epilogue of the one-piece product.
  // The choice depends on the shape alone, so a matrix gets the same bits in any batch.
  p.split = 0;
  p.split_chunk = 0;
  p.off_split = o;
  const int64_t T = p.mp / p.tile;
  if (T * (T + 1) / 2 <= 40 && p.np >= 8192) {
    int64_t sk = 512 / (T * (T + 1) / 2);  // at most two workgroups per compute unit: one more chunk would start a second, almost empty round
    if (sk > p.np / 2048) sk = p.np / 2048;
    if (sk > 64) sk = 64;
    if (sk > 8) sk &= ~int64_t(7);
    if (sk >= 2) {
      p.split_chunk = (int)round_up((p.np + sk - 1) / sk, 64);
      p.split = (int)((p.np + p.split_chunk - 1) / p.split_chunk);
      p.off_split = take((size_t)p.split * p.mp * p.mp * sizeof(float));
    }
  }
  p.total = o;
  return p;
}

template <int BM, int BN, int BK, int STAGES, int WGM, int WGN, int MODE>
static int launch_group(const void* table, int n_blocks, hipStream_t s) {
  constexpr int smem = STAGES * (BM + BN) * BK * 2;
  static LdsReservation reserved;
  auto kern = ns_gemm_kernel<BM, BN, BK, STAGES, WGM, WGN, MODE>;
  const void* kp = reinterpret_cast<const void*>(kern);
  if (int rc = reserve_lds(reserved, &kp, 1, smem, "hb_ns5")) return rc;
  kern<<<n_blocks, WGM * WGN * 64, smem, s>>>(table);
  return HB_OK;
}

template <int MODE>
static int launch_group4(const void* table, int n_blocks, hipStream_t s) {
  constexpr int smem = 4 * (256 + 256) * 32 * 2;
  static LdsReservation reserved;
  auto kern = ns_gemm4_kernel<MODE>;
  const void* kp = reinterpret_cast<const void*>(kern);
  if (int rc = reserve_lds(reserved, &kp, 1, smem, "hb_ns5")) return rc;
  kern<<<n_blocks, 256, smem, s>>>(table);
  return HB_OK;
}

// A piece of the tables on its way to device memory: it travels as the argument of a one-workgroup kernel, which is the one
// way to bring host data to the device from a call that may neither allocate nor copy from pageable memory.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
constexpr int kUploadPieces = 248;
struct UploadArgs {
  u32x4 data[kUploadPieces];
  u32x4* dst;
  int n;
};
static_assert(sizeof(UploadArgs) <= 4096, "the piece travels as a kernel argument");

__global__ __launch_bounds__(256) void ns_upload_kernel(const UploadArgs a) {
  const auto* ka = (const __attribute__((address_space(4))) UploadArgs*)__builtin_amdgcn_kernarg_segment_ptr();
  const int t = threadIdx.x;
  if (t < ka->n) ka->dst[t] = ka->data[t];
}

// The launches of one Newton-Schulz call, collected first and issued after their tables are on the device: `host` holds
// every table of the call (each 256-byte aligned), `ops` the launches in order (an op is handed the tables' device address).
struct Stager {
  std::vector<char> host;
  std::vector<std::function<int(const char*)>> ops;
};

// One product of the iteration for every matrix of one tile class, in one launch.  Fills the tile lists of the eight XCDs as
// described at locate_tile.
#ifndef HB_NS_WHOLE_MAX
#define HB_NS_WHOLE_MAX 256  // a matrix of the 128-wide class with at most this many tiles stays on one XCD
#endif
template <int MODE>
static void gemm_stage(Stager& st, std::vector<Problem> probs, int tile, hipStream_t s) {
  constexpr bool symmetric = MODE == kModeS || MODE == kModeY2 || MODE == kModePartial;
  auto tiles_of = [](const Problem& q) { return symmetric ? q.tiles_m * (q.tiles_m + 1) / 2 : q.tiles_m * q.tiles_n; };
  std::stable_sort(probs.begin(), probs.end(), [&](const Problem& a, const Problem& b) { return (int64_t)a.K * tiles_of(a) > (int64_t)b.K * tiles_of(b); });
  std::vector<Problem> lists[8];
  int64_t load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  for (const Problem& q : probs) {
    const int n = tiles_of(q);
    if (tile == 128 && n <= HB_NS_WHOLE_MAX) {
      const int x = (int)(std::min_element(load, load + 8) - load);
      Problem e = q;
      e.t0 = 0;
      e.n_run = n;
      lists[x].push_back(e);
      load[x] += (int64_t)n * q.K;
      continue;
    }
    const int per = (n + 7) / 8;
    for (int x = 0; x < 8 && x * per < n; ++x) {
      Problem e = q;
      e.t0 = x * per;
      e.n_run = std::min(per, n - e.t0);
      lists[x].push_back(e);
      load[x] += (int64_t)e.n_run * q.K;
    }
  }
  TableHeader hdr{};
  int longest = 0, entries = 0;
  for (int x = 0; x < 8; ++x) {
    std::stable_sort(lists[x].begin(), lists[x].end(), [](const Problem& a, const Problem& b) { return a.K > b.K; });
    int pos = 0;
    for (Problem& e : lists[x]) {
      e.pos_begin = pos;
      pos += e.n_run;
    }
    longest = std::max(longest, pos);
    hdr.first[x] = entries;
    entries += (int)lists[x].size();
  }
  hdr.first[8] = entries;
  const size_t at = (st.host.size() + 255) & ~size_t(255);
  st.host.resize(at + sizeof(TableHeader) + (size_t)entries * sizeof(Problem));
  std::memcpy(st.host.data() + at, &hdr, sizeof(TableHeader));
  size_t o = at + sizeof(TableHeader);
  for (int x = 0; x < 8; ++x) {
    if (lists[x].empty()) continue;
    std::memcpy(st.host.data() + o, lists[x].data(), lists[x].size() * sizeof(Problem));
    o += lists[x].size() * sizeof(Problem);
  }
  const int blocks = 8 * longest;
#ifndef HB_GEMM_CFG_SMALL
#define HB_GEMM_CFG_SMALL 128, 128, 64, 2, 2, 4
#endif
  st.ops.push_back([=](const char* dev) {
    return tile == 256 ? launch_group4<MODE>(dev + at, blocks, s) : launch_group<HB_GEMM_CFG_SMALL, MODE>(dev + at, blocks, s);
  });
}

// The tables go to the device in pieces of a kernel argument each, then the launches run in order.
static int run_staged(Stager& st, char* dev_tables, size_t room, hipStream_t s, const char* who) {
  if (st.host.size() > room) return set_error(HB_EINVAL, "%s: internal error: tables outgrew their room", who);
  st.host.resize((st.host.size() + 15) & ~size_t(15));
  for (size_t at = 0; at < st.host.size(); at += sizeof(UploadArgs::data)) {
    UploadArgs u;
    const size_t bytes = std::min(sizeof(UploadArgs::data), st.host.size() - at);
    std::memcpy(u.data, st.host.data() + at, bytes);
    u.dst = reinterpret_cast<u32x4*>(dev_tables + at);
    u.n = (int)(bytes / 16);
    ns_upload_kernel<<<1, 256, 0, s>>>(u);
  }
  for (auto& op : st.ops)
    if (int rc = op(dev_tables)) return rc;
  return check_launch(who);
}

// Room for the tables of one call: 15 products, each listing every matrix once, or once per K chunk of a split product
static size_t table_bytes(const std::vector<NsPlan>& plans) {
  size_t entries = 0;
  for (const NsPlan& p : plans) entries += p.split > 1 ? p.split : 1;
  // 5 iterations x (S, split chunks, Y2, X) in two tile classes; a matrix is listed up to eight times (a run per XCD); each
  // table has a header and is 256-byte aligned
  return 20 * (8 * entries * sizeof(Problem) + 2 * (256 + sizeof(TableHeader)));
}

// coeffs_host: 3 * n_steps floats per matrix when per_matrix, else one table of that many; flags likewise
static int ns5_batched_impl(int n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols, int n_steps,
                            const float* coeffs_host, const int32_t* flags, bool per_matrix, float eps, const float* post_scale,
                            const float* param_step, const double* const* sumsq_parts, const int32_t* n_sumsq_parts, int32_t rng_mode,
                            uint64_t seed, uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes,
                            hipStream_t s, const char* who) {
  if (n_mats <= 0 || !g || !out || !rows || !cols || !coeffs_host || !flags || !post_scale || !flat_base || !workspace)
    return set_error(HB_EINVAL, "%s: null pointer or empty batch", who);
  if (rng_mode != HB_RNG_HALF && rng_mode != HB_RNG_PHILOX) return set_error(HB_EINVAL, "%s: bad rng_mode", who);
  if (n_steps < 1 || n_steps > 64) return set_error(HB_EINVAL, "%s: 1 to 64 iterations", who);
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0) return set_error(HB_EINVAL, "%s: workspace must be 256-byte aligned", who);
  auto flag_of = [&](int i) { return flags[per_matrix ? i : 0]; };
  auto coeff_of = [&](int i, int k) { return coeffs_host[(per_matrix ? (size_t)i * 3 * n_steps : 0) + k]; };
  for (int i = 0; i < n_mats; ++i) {
    const int f = flag_of(i);
    if ((f & ~(HB_NS_LEGACY | HB_NS_BF16_UPDATE | HB_NS_F16_UPDATE | HB_NS_APPLY_TO_PARAM | HB_NS_CAUTIOUS_WD)) ||
        (f & (HB_NS_BF16_UPDATE | HB_NS_F16_UPDATE)) == (HB_NS_BF16_UPDATE | HB_NS_F16_UPDATE))
      return set_error(HB_EINVAL, "%s: unknown flag bits, or both update formats at once", who);
    if ((f & HB_NS_APPLY_TO_PARAM) && (!param_step || g[i] == out[i]))
      return set_error(HB_EINVAL, "%s: HB_NS_APPLY_TO_PARAM needs param_step and an output that is not the input", who);
    if ((f & HB_NS_CAUTIOUS_WD) && !(f & HB_NS_APPLY_TO_PARAM)) return set_error(HB_EINVAL, "%s: HB_NS_CAUTIOUS_WD goes with HB_NS_APPLY_TO_PARAM", who);
  }
  if ((sumsq_parts == nullptr) != (n_sumsq_parts == nullptr)) return set_error(HB_EINVAL, "%s: sumsq_parts and n_sumsq_parts go together", who);
  for (int i = 0; i < n_mats; ++i) {
    if (sumsq_parts && sumsq_parts[i] && n_sumsq_parts[i] <= 0) return set_error(HB_EINVAL, "%s: no partial sums for matrix %d", who, i);
    if (!g[i] || !out[i]) return set_error(HB_EINVAL, "%s: null matrix pointer at %d", who, i);
    if (rows[i] <= 0 || cols[i] <= 0 || rows[i] > (1 << 20) || cols[i] > (1 << 20)) return set_error(HB_EINVAL, "%s: bad shape at %d", who, i);
  }
  std::vector<int> tile;
  choose_tiles(n_mats, rows, cols, tile);
  std::vector<NsPlan> plans(n_mats);
  std::vector<char*> base(n_mats);
  size_t total = 0;
  for (int i = 0; i < n_mats; ++i) {
    plans[i] = make_plan(rows[i], cols[i], tile[i]);
    base[i] = static_cast<char*>(workspace) + total;
    total += plans[i].total;
  }
  const size_t table_room = table_bytes(plans);
  char* const dev_tables = static_cast<char*>(workspace) + total;  // every plan's size is a multiple of 256
  total += table_room;
  if ((int64_t)total > workspace_bytes)
    return set_error(HB_EINVAL, "%s: workspace too small (%lld < %lld)", who, (long long)workspace_bytes, (long long)total);
  Stager st;
  auto X = [&](int i, int k) { return reinterpret_cast<uint16_t*>(base[i] + plans[i].off_x[k]); };
  auto Xt = [&](int i, int k) { return reinterpret_cast<uint16_t*>(base[i] + plans[i].off_xt[k]); };
  auto S = [&](int i) { return reinterpret_cast<uint16_t*>(base[i] + plans[i].off_s); };
  auto Y = [&](int i) { return reinterpret_cast<uint16_t*>(base[i] + plans[i].off_y); };
  auto Y2 = [&](int i) { return reinterpret_cast<uint16_t*>(base[i] + plans[i].off_y2); };

  // normalise + round every input into its X / X^T pair: three grouped launches per kMaxPrep matrices
  Rng rng{(uint32_t)seed, (uint32_t)(seed >> 32), step, rng_mode};
  for (int first = 0; first < n_mats; first += kMaxPrep) {
    PrepGroup pg{};
    pg.n_items = std::min(kMaxPrep, n_mats - first);
    pg.eps = eps;
    pg.rng = rng;
    int blocks = 0, tiles = 0;
    for (int k = 0; k < pg.n_items; ++k) {
      const int i = first + k;
      const NsPlan& p = plans[i];
      PrepItem& q = pg.it[k];
      q.g = g[i];
      q.X = X(i, 0);
      q.Xt = Xt(i, 0);
      q.partial = reinterpret_cast<double*>(base[i] + p.off_partial);
      q.norm = reinterpret_cast<float*>(base[i] + p.off_norm);
      q.flat_base = flat_base[i];
      q.rows = (int)p.rows;
      q.cols = (int)p.cols;
      q.ldx = (int)p.np;
      q.ldxt = (int)p.mp;
      q.transpose = p.rows > p.cols;
      q.legacy = (flag_of(i) & HB_NS_LEGACY) != 0;
      q.narrow_update = (flag_of(i) & HB_NS_BF16_UPDATE) ? 1 : (flag_of(i) & HB_NS_F16_UPDATE) ? 2 : 0;
      const int64_t n = p.rows * p.cols;
      q.block_begin = blocks;
      if (sumsq_parts && sumsq_parts[i]) {  // the caller's partial sums: nothing to launch for this matrix
        q.partial = sumsq_parts[i];
        q.n_blocks = n_sumsq_parts[i];
        q.sum_blocks = 0;
      } else {
        q.n_blocks = q.sum_blocks = (int)std::min<int64_t>(1024, (n + 4095) / 4096);
      }
      blocks += q.sum_blocks;
      q.tiles_c = (int)((p.cols + 63) / 64);
      q.tile_begin = tiles;
      tiles += (int)((p.rows + 63) / 64) * q.tiles_c;
      if (p.mp != p.m || p.np != p.n) {  // padding must be zero: it enters the products
        const int64_t n16 = (int64_t)(p.off_x[1] - p.off_x[0]) / 16;  // the first X / X^T pair; the products keep padding zero
        ns_zero_kernel<<<1024, 256, 0, s>>>(reinterpret_cast<uint4*>(base[i] + p.off_x[0]), n16);
      }
    }
    if (blocks > 0) ns_sumsq_kernel<<<blocks, 256, 0, s>>>(pg);
    ns_norm_final_kernel<<<pg.n_items, kNormThreads, 0, s>>>(pg);
    ns_prep_kernel<<<tiles, 256, 0, s>>>(pg);
  }

  // the tables in the workspace have room for five iterations: longer schedules run in groups of five, each group's tables
  // written over the last one's (in stream order, behind the products that read those)
  for (int it0 = 0; it0 < n_steps; it0 += 5) {
    st = Stager();
    for (int cls = 0; cls < 2; ++cls) {
      const int t = cls == 0 ? 256 : 128;
      std::vector<int> idx;
      for (int i = 0; i < n_mats; ++i)
        if (tile[i] == t) idx.push_back(i);
      if (idx.empty()) continue;
      std::vector<Problem> probs(idx.size());
      for (int it = it0; it < std::min(it0 + 5, n_steps); ++it) {
        const int cur = it & 1, nxt = cur ^ 1;
        auto ca = [&](int i) { return coeff_of(i, 3 * it); };      // the iteration's (a, b, c) of matrix i
        auto cb = [&](int i) { return coeff_of(i, 3 * it + 1); };
        auto cc = [&](int i) { return coeff_of(i, 3 * it + 2); };
        // S = X X^T, Y = c S + b I   (S is symmetric bit for bit: only the upper triangle of tiles is computed; a product
        // that is split along K goes through raw partial products and ns_split_reduce_kernel instead)
        std::vector<Problem> whole, chunks;
        for (size_t k = 0; k < idx.size(); ++k) {
          const int i = idx[k];
          const NsPlan& p = plans[i];
          Problem q{};
          q.tiles_m = q.tiles_n = (int)(p.mp / t);
          q.lda = (int)p.np; q.ldb = (int)p.np;
          q.mul_c = cc(i); q.diag = cb(i);
          if (p.split == 0) {
            q.A = X(i, cur); q.B = X(i, cur); q.K = (int)p.np;
            q.C = S(i); q.ldc = (int)p.mp; q.C2 = Y(i); q.ldc2 = (int)p.mp;
            whole.push_back(q);
            continue;
          }
          for (int c = 0; c < p.split; ++c) {
            const int64_t k0 = (int64_t)c * p.split_chunk;
            q.A = X(i, cur) + k0; q.B = X(i, cur) + k0;
            q.K = (int)(p.np - k0 < p.split_chunk ? p.np - k0 : p.split_chunk);
            q.F = reinterpret_cast<float*>(base[i] + p.off_split) + (size_t)c * p.mp * p.mp;
            q.ldf = (int)p.mp; q.f_rows = (int)p.mp; q.f_cols = (int)p.mp; q.f_transposed = 0; q.scale = 1.0f;
            chunks.push_back(q);
          }
        }
        if (!whole.empty()) gemm_stage<kModeS>(st, whole, t, s);
        if (!chunks.empty()) {
          gemm_stage<kModePartial>(st, chunks, t, s);
          for (size_t k = 0; k < idx.size(); ++k) {
            const int i = idx[k];
            const NsPlan& p = plans[i];
            if (p.split == 0) continue;
            const float* parts = reinterpret_cast<const float*>(base[i] + p.off_split);
            uint16_t *s_out = S(i), *y_out = Y(i);
            const float mul_c = cc(i), diag = cb(i);
            const int split = p.split, mp = (int)p.mp;
            st.ops.push_back([=](const char*) {
              ns_split_reduce_kernel<<<(unsigned)((mp / 32) * (mp / 32)), 256, 0, s>>>(parts, split, mp, t, s_out, y_out, mul_c, diag);
              return (int)HB_OK;
            });
          }
        }
        // Y2 = Y S + a I  (S symmetric: its rows are the K-contiguous operand; Y2 is a polynomial in S, so only the
        // upper triangle of tiles is computed and mirrored)
        for (size_t k = 0; k < idx.size(); ++k) {
          const int i = idx[k];
          const NsPlan& p = plans[i];
          Problem q{};
          q.A = Y(i); q.B = S(i); q.K = (int)p.mp; q.lda = (int)p.mp; q.ldb = (int)p.mp;
          q.C = Y2(i); q.ldc = (int)p.mp;
          q.tiles_m = q.tiles_n = (int)(p.mp / t);
          q.diag = ca(i);
          probs[k] = q;
        }
        gemm_stage<kModeY2>(st, probs, t, s);
        // X = Y2 X  ==  gemm(Y2, X^T)
        for (size_t k = 0; k < idx.size(); ++k) {
          const int i = idx[k];
          const NsPlan& p = plans[i];
          Problem q{};
          q.A = Y2(i); q.B = Xt(i, cur); q.K = (int)p.mp; q.lda = (int)p.mp; q.ldb = (int)p.mp;
          q.tiles_m = (int)(p.mp / t);
          q.tiles_n = (int)(p.np / t);
          if (it < n_steps - 1) {
            q.C = X(i, nxt); q.ldc = (int)p.np; q.C2 = Xt(i, nxt); q.ldc2 = (int)p.mp;
          } else {
            q.F = out[i]; q.f_transposed = p.rows > p.cols; q.ldf = (int)p.cols; q.f_rows = (int)p.rows; q.f_cols = (int)p.cols;
            q.scale = post_scale[i];
            q.round_out = (flag_of(i) & HB_NS_BF16_UPDATE) ? 1 : (flag_of(i) & HB_NS_F16_UPDATE) ? 2 : 0;
            if (flag_of(i) & HB_NS_APPLY_TO_PARAM) {
              q.round_out |= kApplyToParam | ((flag_of(i) & HB_NS_CAUTIOUS_WD) ? kCautiousWd : 0);
              q.mul_c = param_step[0];
              q.diag = param_step[1];
            }
          }
          probs[k] = q;
        }
        if (it < n_steps - 1) gemm_stage<kModeX>(st, probs, t, s);
        else {
          bool extras = false;  // anything the plain last product does not do: see kModeFinalX
          for (const Problem& q : probs) extras = extras || (q.round_out & ~1) != 0;
          if (extras) gemm_stage<kModeFinalX>(st, probs, t, s);
          else gemm_stage<kModeFinal>(st, probs, t, s);
        }
      }
    }
    if (int rc = run_staged(st, dev_tables, table_room, s, who)) return rc;
  }
  return HB_OK;
}

}  // namespace hb

extern "C" int hb_ns5_batched_workspace_bytes(int32_t n_mats, const int64_t* rows, const int64_t* cols, int64_t* bytes) {
  using namespace hb;
  if (n_mats <= 0 || !rows || !cols || !bytes) return set_error(HB_EINVAL, "hb_ns5_batched_workspace_bytes: bad arguments");
  for (int i = 0; i < n_mats; ++i)
    if (rows[i] <= 0 || cols[i] <= 0) return set_error(HB_EINVAL, "hb_ns5_batched_workspace_bytes: bad shape at %d", i);
  std::vector<int> tile;
  choose_tiles(n_mats, rows, cols, tile);
  int64_t total = 0;
  std::vector<NsPlan> plans(n_mats);
  for (int i = 0; i < n_mats; ++i) {
    plans[i] = make_plan(rows[i], cols[i], tile[i]);
    total += (int64_t)plans[i].total;
  }
  *bytes = total + (int64_t)table_bytes(plans);
  return HB_OK;
}

extern "C" int hb_ns_product(int32_t tile, int32_t mode, const void* A, const void* B, void* C, void* C2, int64_t M, int64_t N, int64_t K, float mul_c,
                             float diag, void* workspace, int64_t workspace_bytes, void* stream_) {
  using namespace hb;
  if (tile != 128 && tile != 256) return set_error(HB_EINVAL, "hb_ns_product: tile is 128 or 256");
  if (mode != kModeS && mode != kModeY2 && mode != kModeX) return set_error(HB_EINVAL, "hb_ns_product: mode is 0 (S), 1 (Y2) or 2 (X)");
  if (!A || !B || !C || !workspace || (mode != kModeY2 && !C2)) return set_error(HB_EINVAL, "hb_ns_product: null pointer");
  if (M <= 0 || N <= 0 || K <= 0 || M % tile || N % tile || K % 64 || M > (1 << 20) || N > (1 << 20) || K > (1 << 20))
    return set_error(HB_EINVAL, "hb_ns_product: M and N must be multiples of the tile, K of 64");
  if (mode != kModeX && M != N) return set_error(HB_EINVAL, "hb_ns_product: the symmetric products are square");
  if (workspace_bytes < 4096 || (reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
    return set_error(HB_EINVAL, "hb_ns_product: the workspace is 4096 bytes, 256-byte aligned");
  Problem q{};
  q.A = static_cast<const uint16_t*>(A); q.B = static_cast<const uint16_t*>(B);
  q.C = static_cast<uint16_t*>(C); q.C2 = static_cast<uint16_t*>(C2);
  q.K = (int)K; q.lda = (int)K; q.ldb = (int)K; q.ldc = (int)N; q.ldc2 = mode == kModeX ? (int)M : (int)N;
  q.mul_c = mul_c; q.diag = diag;
  q.tiles_m = (int)(M / tile); q.tiles_n = (int)(N / tile);
  hipStream_t s = static_cast<hipStream_t>(stream_);
  Stager st;
  if (mode == kModeS) gemm_stage<kModeS>(st, {q}, tile, s);
  else if (mode == kModeY2) gemm_stage<kModeY2>(st, {q}, tile, s);
  else gemm_stage<kModeX>(st, {q}, tile, s);
  return run_staged(st, static_cast<char*>(workspace), 4096, s, "hb_ns_product");
}

extern "C" int hb_ns_tile(int64_t rows, int64_t cols) {
  std::vector<int> tile;
  hb::choose_tiles(1, &rows, &cols, tile);
  return tile[0];
}

extern "C" int hb_ns5_workspace_bytes(int64_t rows, int64_t cols, int64_t* bytes) {
  return hb_ns5_batched_workspace_bytes(1, &rows, &cols, bytes);
}

extern "C" int hb_ns5_batched(int32_t n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols,
                              const float* coeffs_host, int32_t legacy, float eps, const float* post_scale, int32_t rng_mode,
                              uint64_t seed, uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes,
                              void* stream_) {
  return hb::ns5_batched_impl(n_mats, g, out, rows, cols, 5, coeffs_host, &legacy, false, eps, post_scale, nullptr, nullptr, nullptr, rng_mode, seed, step, flat_base,
                              workspace, workspace_bytes, static_cast<hipStream_t>(stream_), "hb_ns5_batched");
}

extern "C" int hb_ns5_batched_mixed(int32_t n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols,
                                    const float* coeffs_host, const int32_t* flags, float eps, const float* post_scale, int32_t rng_mode,
                                    uint64_t seed, uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes,
                                    void* stream_) {
  return hb::ns5_batched_impl(n_mats, g, out, rows, cols, 5, coeffs_host, flags, true, eps, post_scale, nullptr, nullptr, nullptr, rng_mode, seed, step, flat_base,
                              workspace, workspace_bytes, static_cast<hipStream_t>(stream_), "hb_ns5_batched_mixed");
}

extern "C" int hb_ns_batched_steps(int32_t n_mats, const float* const* g, float* const* out, const int64_t* rows, const int64_t* cols,
                                   int32_t n_steps, const float* coeffs_host, const int32_t* flags, float eps, const float* post_scale,
                                   const float* param_step, const double* const* sumsq_parts, const int32_t* n_sumsq_parts, int32_t rng_mode,
                                   uint64_t seed, uint32_t step, const int64_t* flat_base, void* workspace, int64_t workspace_bytes,
                                   void* stream_) {
  return hb::ns5_batched_impl(n_mats, g, out, rows, cols, n_steps, coeffs_host, flags, true, eps, post_scale, param_step, sumsq_parts,
                              n_sumsq_parts, rng_mode, seed, step, flat_base, workspace, workspace_bytes, static_cast<hipStream_t>(stream_),
                              "hb_ns_batched_steps");
}

extern "C" int hb_ns5(const float* g, float* out, int64_t rows, int64_t cols, const float* coeffs_host, int32_t legacy, float eps,
                      float post_scale, int32_t rng_mode, uint64_t seed, uint32_t step, int64_t flat_base, void* workspace,
                      int64_t workspace_bytes, void* stream_) {
  return hb::ns5_batched_impl(1, &g, &out, &rows, &cols, 5, coeffs_host, &legacy, false, eps, &post_scale, nullptr, nullptr, nullptr, rng_mode, seed, step, &flat_base, workspace,
                              workspace_bytes, static_cast<hipStream_t>(stream_), "hb_ns5");
}
