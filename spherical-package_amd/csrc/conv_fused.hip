// Fused mapped-convolution kernels for gfx950 (float32 tensors).
//
// The im2col column matrix never exists in HBM.  Three kernels cover the six
// contractions of mapped / mapped-transposed convolution (see ConvGeom):
//
//   gather_gemm   pix[b][n,m]  = sum_{c,k} Wm[n,(c,k)] * gather(img[b,c], tap(m,k)) + bias[n]
//   gemm_scatter  img[b,c]    += scatter_{tap(m,k)}( sum_n Wm[n,(c,k)] * pix[b][n,m] )
//   gather_wgrad  gW[n,(c,k)]  = sum_{b,m} pix[b][n,m] * gather(img[b,c], tap(m,k))
//
// Common structure: a 256-thread workgroup (4 wavefronts) owns a tile of
// pixels.  For one kernel sample k at a time it turns the tile's sample-map
// entries into a compact per-pixel tap list in LDS (offset + coefficient; the
// interpolation weight and the per-point weight are folded into one
// coefficient, zero-weight taps are dropped), which is then reused for every
// channel.  Column values are produced straight into an LDS operand tile (or
// consumed straight from MFMA accumulators) and contracted with
// v_mfma_f32_32x32x2_f32; each wavefront owns a 64 x 64 block of the 128 x 128
// (or 64 x 256) workgroup tile as 2 x 2 MFMA accumulators.
//
// These kernels read their operands from global memory.  For a map that has a tap plan
// (conv_plan.hpp) the drivers at the end of this file run them only on the tiles that the
// plan's LDS-window kernels (conv_window_gemm.hip, conv_window_wgrad.hip) leave over, and as
// the device-side fallback of the inverse plan.
//
// MFMA 32x32x2 f32 register layout used below (wave64, lane l):
//   A operand: A[i = l % 32][k = l / 32]        B operand: B[k = l / 32][j = l % 32]
//   D, 16 registers v: D[i = 8*(v/4) + 4*(l/32) + v%4][j = l % 32]
#include "conv_fused.hpp"
#include "conv_small.hpp"
#include "conv_product.hpp"
#include "conv_plan.hpp"

#include <hip/hip_runtime.h>

#include "sdk_host.hpp"
#include "sdk_mfma.hpp"
#include "sdk_taps.hpp"

namespace sdk {

constexpr int kThreads = 256;
constexpr int kKC = 32;         // reduction rows staged per step
constexpr int kMaxSlots = 32;   // tap slots per pixel and kernel sample (points * taps); LDS: 2 KB per slot at 256 pixels

__host__ __device__ constexpr int round_up(int v, int m) { return (v + m - 1) / m * m; }

// Row of D held in accumulator register v of lane l (see layout above).
__device__ __forceinline__ int mfma_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
}

// XCD-aware tile order: hardware workgroup ids go round-robin over the 8 XCDs
// (each with its own L2); give every XCD a contiguous band of tiles so that
// neighbouring pixel tiles, which share input rows, meet in one L2.
__device__ __forceinline__ int xcd_band_tile(int bid, int ntiles) {
  constexpr int X = 8;
  const int per = ntiles / X;           // full bands
  if (bid >= per * X) return bid;       // remainder keeps its natural order
  return (bid % X) * per + bid / X;
}

// ---------------------------------------------------------------------------
// Tap table of one kernel sample k for the TP pixels of a tile; thread tid < TP owns pixel
// `pix` (-1: no pixel).
// Layout tap_off[slot][TP], tap_co[slot][TP] (slot-major, so lanes that own
// consecutive pixels hit consecutive LDS banks).  Every pixel's active taps are
// packed to the front; slots up to the tile-wide maximum *smax are padded with
// coefficient 0.  Must be called by all threads of the workgroup.
// ---------------------------------------------------------------------------
template <int INTERP, bool WEIGHTED, int TP>
__device__ __forceinline__ void build_taps(const float* __restrict__ map,
                                           const float* __restrict__ wts, int pix, int K,
                                           int k, int P, int H, int W, int* __restrict__ tap_off,
                                           float* __restrict__ tap_co, int* __restrict__ smax) {
  const int tid = threadIdx.x;
  if (tid == 0) *smax = 0;
  __syncthreads();
  int cnt = 0;
  if (tid < TP) {
    if (pix >= 0) {
      const int q = WEIGHTED ? P : 1;
      const size_t s = ((size_t)pix * K + k) * q;
      PointTaps<float, INTERP> t;
      for (int p = 0; p < q; ++p) {
        t.set(map[(s + p) * 2], map[(s + p) * 2 + 1], H, W);
        const float wt = WEIGHTED ? wts[s + p] : 1.0f;
#pragma unroll
        for (int i = 0; i < PointTaps<float, INTERP>::N; ++i) {
          const float co = WEIGHTED ? wt * t.w[i] : t.w[i];
          if (t.off[i] >= 0 && co != 0.0f) {
            tap_off[cnt * TP + tid] = t.off[i];
            tap_co[cnt * TP + tid] = co;
            ++cnt;
          }
        }
      }
    }
    atomicMax(smax, cnt);
  }
  __syncthreads();
  if (tid < TP) {
    const int top = *smax;
    for (int sidx = cnt; sidx < top; ++sidx) {
      tap_off[sidx * TP + tid] = 0;
      tap_co[sidx * TP + tid] = 0.0f;
    }
  }
  __syncthreads();
}

// One reduction chunk of kKC rows: D(64 x 64 per wave) += A^T-tile x B-tile.
// As[r][lda] holds the A operand r-major (row index i contiguous), Bs[r][ldb]
// the B operand r-major (column index j contiguous).
__device__ __forceinline__ void mfma_chunk(const float* __restrict__ As, int lda, int a_base,
                                           const float* __restrict__ Bs, int ldb, int b_base,
                                           int rows, floatx16 (&acc)[2][2]) {
  const int lane = threadIdx.x & 63;
  const int lk = lane >> 5, lj = lane & 31;
#pragma unroll 4
  for (int r = 0; r < rows; r += 2) {
    const float a0 = As[(r + lk) * lda + a_base + lj];
    const float a1 = As[(r + lk) * lda + a_base + 32 + lj];
    const float b0 = Bs[(r + lk) * ldb + b_base + lj];
    const float b1 = Bs[(r + lk) * ldb + b_base + 32 + lj];
    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
  }
}

// Same contraction with operands rounded to bf16 (fp32 accumulate): the LDS tiles stay
// fp32 and are converted while the fragments are read; rows must be a multiple of 16.
__device__ __forceinline__ void mfma_chunk_bf16(const float* __restrict__ As, int lda, int a_base,
                                                const float* __restrict__ Bs, int ldb, int b_base,
                                                int rows, floatx16 (&acc)[2][2]) {
  const int lane = threadIdx.x & 63;
  const int lk = lane >> 5, lj = lane & 31;
  for (int r = 0; r < rows; r += 16) {
    Bf16Frag a[2], b[2];
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      float fa[8], fb[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        fa[j] = As[(r + 8 * lk + j) * lda + a_base + 32 * blk + lj];
        fb[j] = Bs[(r + 8 * lk + j) * ldb + b_base + 32 * blk + lj];
      }
      a[blk] = pack_bf16x8(fa);
      b[blk] = pack_bf16x8(fb);
    }
    acc[0][0] = mfma_bf16(a[0], b[0], acc[0][0]);
    acc[0][1] = mfma_bf16(a[0], b[1], acc[0][1]);
    acc[1][0] = mfma_bf16(a[1], b[0], acc[1][0]);
    acc[1][1] = mfma_bf16(a[1], b[1], acc[1][1]);
  }
}

template <bool BF16>
__device__ __forceinline__ void mfma_chunk_any(const float* __restrict__ As, int lda, int a_base,
                                               const float* __restrict__ Bs, int ldb, int b_base,
                                               int rows, floatx16 (&acc)[2][2]) {
  if constexpr (BF16)
    mfma_chunk_bf16(As, lda, a_base, Bs, ldb, b_base, rows, acc);
  else
    mfma_chunk(As, lda, a_base, Bs, ldb, b_base, rows, acc);
}

// The same contraction over operand tiles stored with the reduction index contiguous:
// At[i][kLdK], Bt[j][kLdK] (kKC values per row, 4 floats of skew).  Lane half h contracts
// rows 16h + 0..15 (fp32, four per 16-byte read) or 16t + 8h + 0..7 (bf16, instruction t),
// so every operand fragment arrives as a 16-byte LDS read: a quarter of the LDS
// instructions of mfma_chunk().
constexpr int kLdK = kKC + 4;

template <int MM>
__device__ __forceinline__ void mfma_chunk_kc(const float* __restrict__ At, int a_base,
                                              const float* __restrict__ Bt, int b_base,
                                              floatx16 (&acc)[2][2]) {
  const int lane = threadIdx.x & 63;
  const int lk = lane >> 5, lj = lane & 31;
  const float* a0p = At + (a_base + lj) * kLdK;
  const float* a1p = a0p + 32 * kLdK;
  const float* b0p = Bt + (b_base + lj) * kLdK;
  const float* b1p = b0p + 32 * kLdK;
  if constexpr (MM != kMmF32) {
#pragma unroll
    for (int t = 0; t < kKC / 16; ++t) {
      const int o = 16 * t + 8 * lk;
      auto read8 = [&](const float* p, float (&f)[8]) {
        const float4 lo = *reinterpret_cast<const float4*>(p + o);
        const float4 hi = *reinterpret_cast<const float4*>(p + o + 4);
        f[0] = lo.x; f[1] = lo.y; f[2] = lo.z; f[3] = lo.w;
        f[4] = hi.x; f[5] = hi.y; f[6] = hi.z; f[7] = hi.w;
      };
      float fa0[8], fa1[8], fb0[8], fb1[8];
      read8(a0p, fa0);
      read8(a1p, fa1);
      read8(b0p, fb0);
      read8(b1p, fb1);
      if constexpr (MM == kMmBf16) {
        const Bf16Frag a0 = pack_bf16x8(fa0), a1 = pack_bf16x8(fa1);
        const Bf16Frag b0 = pack_bf16x8(fb0), b1 = pack_bf16x8(fb1);
        acc[0][0] = mfma_bf16(a0, b0, acc[0][0]);
        acc[0][1] = mfma_bf16(a0, b1, acc[0][1]);
        acc[1][0] = mfma_bf16(a1, b0, acc[1][0]);
        acc[1][1] = mfma_bf16(a1, b1, acc[1][1]);
      } else {
        const Bf16Split a0 = split_bf16x8(fa0), a1 = split_bf16x8(fa1);
        const Bf16Split b0 = split_bf16x8(fb0), b1 = split_bf16x8(fb1);
        acc[0][0] = mfma_split(a0, b0, acc[0][0]);
        acc[0][1] = mfma_split(a0, b1, acc[0][1]);
        acc[1][0] = mfma_split(a1, b0, acc[1][0]);
        acc[1][1] = mfma_split(a1, b1, acc[1][1]);
      }
    }
  } else {
#pragma unroll
    for (int q = 0; q < kKC / 8; ++q) {
      const int o = (kKC / 2) * lk + 4 * q;
      const float4 a0 = *reinterpret_cast<const float4*>(a0p + o);
      const float4 a1 = *reinterpret_cast<const float4*>(a1p + o);
      const float4 b0 = *reinterpret_cast<const float4*>(b0p + o);
      const float4 b1 = *reinterpret_cast<const float4*>(b1p + o);
      const float av0[4] = {a0.x, a0.y, a0.z, a0.w}, av1[4] = {a1.x, a1.y, a1.z, a1.w};
      const float bv0[4] = {b0.x, b0.y, b0.z, b0.w}, bv1[4] = {b1.x, b1.y, b1.z, b1.w};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[i], bv0[i], acc[0][0], 0, 0, 0);
        acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av0[i], bv1[i], acc[0][1], 0, 0, 0);
        acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[i], bv0[i], acc[1][0], 0, 0, 0);
        acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(av1[i], bv1[i], acc[1][1], 0, 0, 0);
      }
    }
  }
}

__device__ __forceinline__ void zero_acc(floatx16 (&acc)[2][2]) {
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;
}

// ---------------------------------------------------------------------------
// Weight re-layout (once per call, a few hundred KB): from Wm[Cp][Cg*K] to
//   Wg[k][c][n]  (n contiguous, padded to CgP x CpP)   (n_fastest = 1)
//   Ws[k][n][c]  (c contiguous, padded to CpP x CgP)   for gemm_scatter (n_fastest = 0)
//   Wk[k][c / kKC][n][c % kKC]  (rows of kKC reduction values)  for gather_gemm (n_fastest = 2)
//   Wt[k][n / kKC][c][n % kKC]  (the same with the roles of n and c exchanged: CpP pads c,
//                                CgP pads n)                for the inverse gather (n_fastest = 3)
// Padding is zero so the hot loops need no channel guards on the weight side.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void relayout_weight_kernel(
    const float* __restrict__ Wm, float* __restrict__ out, int Cp, int Cg, int K, int CpP, int CgP,
    int n_fastest) {
  const size_t total = (size_t)K * CpP * CgP;
  for (size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x; e < total;
       e += (size_t)gridDim.x * kThreads) {
    int n, c, k;
    if (n_fastest >= 2) {
      int red = (int)(e % kKC);
      const int row = (int)((e / kKC) % CpP);
      const size_t rest = e / ((size_t)kKC * CpP);   // k * (CgP / kKC) + chunk
      red += (int)(rest % (CgP / kKC)) * kKC;
      k = (int)(rest / (CgP / kKC));
      if (n_fastest == 2) {
        n = row;
        c = red;
      } else {
        n = red;
        c = row;
      }
    } else if (n_fastest) {
      n = (int)(e % CpP);
      c = (int)((e / CpP) % CgP);
      k = (int)(e / ((size_t)CpP * CgP));
    } else {
      c = (int)(e % CgP);
      n = (int)((e / CgP) % CpP);
      k = (int)(e / ((size_t)CpP * CgP));
    }
    out[e] = (n < Cp && c < Cg) ? Wm[(size_t)n * Cg * K + (size_t)c * K + k] : 0.0f;
  }
}

// ---------------------------------------------------------------------------
// gather_gemm.  Workgroup tile: TN pixel-side channels x TM pixels, TN*TM = 16384.
// grid.x = pixel tiles * n tiles, grid.y = batch.
// LDS: Bs[kKC][TM] column tile, As[kKC][TN] weight tile, tap table.
//
// INV: the tap lists do not come from the sample map but from an inverse map
// (conv_inverse.hip): rows inv_off / inv_co [(pixel tile * K + k) * slots + s][TM] and
// their count inv_ns[pixel tile * K + k].  The kernel does nothing unless *gate == 0.
//
// TILED (TM = 128): the workgroup's pixels are not TM consecutive ones but a 2-D tile of the
// tiling pt, taken from a device-side list (tile_list[i], i < *tile_count): the tiles a
// plan-driven kernel leaves to this one.
// ---------------------------------------------------------------------------
template <int INTERP, bool WEIGHTED, int TN, int TM, int MM, bool INV = false, bool TILED = false>
__global__ __launch_bounds__(kThreads) void gather_gemm_kernel(
    const float* __restrict__ img, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ Wg, const float* __restrict__ bias, float* __restrict__ pix, int Cg,
    int H, int W, int Cp, int M, int K, int P, int CgP, int CpP, int slots, int m_tiles,
    const int* __restrict__ inv_off = nullptr, const float* __restrict__ inv_co = nullptr,
    const int* __restrict__ inv_ns = nullptr, const int* __restrict__ gate = nullptr,
    PixelTiling pt = PixelTiling(), const int* __restrict__ tile_list = nullptr,
    const int* __restrict__ tile_count = nullptr) {
  static_assert(!TILED || TM % 128 == 0, "tiled pixel order: 128-pixel tiles");
  constexpr int TPW = TILED ? TM / 128 : 1;   // listed tiles per workgroup
  if constexpr (INV) {
    if (*gate != 0) return;
  }
  extern __shared__ __align__(16) unsigned char smem[];
  float* Bs = reinterpret_cast<float*>(smem);             // [TM][kLdK] columns, reduction index contiguous
  float* As = Bs + TM * kLdK;                              // [TN][kLdK] weights
  int* tap_off = reinterpret_cast<int*>(As + TN * kLdK);   // [slots][TM]
  float* tap_co = reinterpret_cast<float*>(tap_off + slots * TM);
  int* smax = reinterpret_cast<int*>(tap_co + slots * TM);

  constexpr int WAVES_N = TN / 64;           // waves along n
  constexpr int SPLIT = kThreads / TM;       // threads sharing one pixel in the gather
  constexpr int RPT = kKC / SPLIT;           // column rows per thread and chunk
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n_tiles = CpP / TN;
  int tile = TILED ? 0 : xcd_band_tile(blockIdx.x, m_tiles * n_tiles);
  // pixel (index into the pixel grid, -1: none) of tile-local pixel p
  int lt[TPW];       // TILED: the listed pixel tiles of this workgroup (-1: none)
  int ptile = 0;     // otherwise: the run of TM pixels whose inverse rows are read
#pragma unroll
  for (int i = 0; i < TPW; ++i) lt[i] = -1;
  if constexpr (TILED) {
    // XCD x (workgroup ids go round-robin over the 8 XCDs) takes an eighth of the list,
    // however long the list is; a workgroup takes TPW consecutive entries
    const int cnt = *tile_count, units = (cnt + TPW - 1) / TPW, per = (units + 7) >> 3;
    const int wg = blockIdx.x / n_tiles, slot = (wg & 7) * per + (wg >> 3);
    if ((wg >> 3) >= per || slot >= units) return;
    tile = blockIdx.x % n_tiles;   // (only the n tile is taken from `tile` below)
#pragma unroll
    for (int i = 0; i < TPW; ++i)
      lt[i] = slot * TPW + i < cnt ? tile_list[slot * TPW + i] : -1;
  } else {
    ptile = tile / n_tiles;
  }
  const int m0 = (tile / n_tiles) * TM, n0 = (tile % n_tiles) * TN;
  auto pixel_of = [&](int p) -> int {
    if constexpr (TILED) {
      const int t2 = TPW == 1 ? lt[0] : (p < 128 ? lt[0] : lt[TPW - 1]);
      if (t2 < 0) return -1;
      const int pl = p & 127;
      const int oy = (t2 / pt.tiles_x) * pt.TY() + (pl >> pt.tx_shift);
      const int ox = ((t2 % pt.tiles_x) << pt.tx_shift) + (pl & (pt.TX() - 1));
      return (oy < pt.OH && ox < pt.OW) ? oy * pt.OW + ox : -1;
    } else {
      return m0 + p < M ? m0 + p : -1;
    }
  };
  const int a_base = (wave % WAVES_N) * 64, b_base = (wave / WAVES_N) * 64;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const int gm = tid % TM, gpart = tid / TM;

  // The accumulators start at the bias of their rows, so the epilogue is stores alone (a bias
  // read behind each store would wait for that store too: 64 round trips per workgroup).
  floatx16 acc[2][2];
  zero_acc(acc);
  if (bias != nullptr) {
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + a_base + 32 * a + mfma_row(v, lane);
        const float bv = bias[n < Cp ? n : Cp - 1];
#pragma unroll
        for (int b = 0; b < 2; ++b) acc[a][b][v] = n < Cp ? bv : 0.0f;
      }
  }

  for (int k = 0; k < K; ++k) {
    if constexpr (INV && TILED) {
      // rows of the listed image tiles: ((tile * K + k) * slots + s) * 128 + pixel
      if (tid == 0) {
        int top = 0;
#pragma unroll
        for (int i = 0; i < TPW; ++i)
          if (lt[i] >= 0) top = max(top, inv_ns[(size_t)lt[i] * K + k]);
        *smax = min(top, slots);
      }
      __syncthreads();
      for (int e = tid; e < *smax * TM; e += kThreads) {
        const int s = e / TM, p = e - s * TM;
        const int t2 = TPW == 1 ? lt[0] : (p < 128 ? lt[0] : lt[TPW - 1]);
        float co = 0.0f;
        int off = 0;
        if (t2 >= 0) {
          const size_t at = (((size_t)t2 * K + k) * slots + s) * 128 + (p & 127);
          co = s < inv_ns[(size_t)t2 * K + k] ? inv_co[at] : 0.0f;
          off = co != 0.0f ? inv_off[at] : 0;
        }
        tap_co[e] = co;
        tap_off[e] = off;
      }
      __syncthreads();
    } else if constexpr (INV) {
      const size_t rows = ((size_t)ptile * K + k) * slots * TM;
      if (tid == 0) *smax = min(inv_ns[(size_t)ptile * K + k], slots);
      __syncthreads();
      for (int e = tid; e < *smax * TM; e += kThreads) {
        const float co = inv_co[rows + e];
        tap_co[e] = co;
        tap_off[e] = co != 0.0f ? inv_off[rows + e] : 0;
      }
      __syncthreads();
    } else {
      build_taps<INTERP, WEIGHTED, TM>(map, wts, tid < TM ? pixel_of(tid) : -1, K, k, P, H, W,
                                       tap_off, tap_co, smax);
    }
    const int ns = *smax;
    for (int c0 = 0; c0 < CgP; c0 += kKC) {
      // ---- gather kKC column rows (channels c0.., sample k) for TM pixels
      float col[RPT];
#pragma unroll
      for (int j = 0; j < RPT; ++j) col[j] = 0.0f;
      // gpart is the same for all lanes of a wave when TM >= 64: keep the channel
      // base in scalar registers so each load needs only a 32-bit lane offset
      const int cfirst = c0 + (TM >= 64 ? __builtin_amdgcn_readfirstlane(gpart) : gpart) * RPT;
      for (int s0 = 0; s0 < ns; s0 += 4) {
        int off[4];
        float co[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const bool on = s0 + u < ns;
          off[u] = on ? tap_off[(s0 + u) * TM + gm] : 0;
          co[u] = on ? tap_co[(s0 + u) * TM + gm] : 0.0f;
        }
        // one scalar base for the chunk; every load adds a 32-bit lane offset
        const char* base = reinterpret_cast<const char*>(img_b + (size_t)min(cfirst, Cg - 1) * HW);
        const unsigned plane_bytes = (unsigned)HW * 4u;
#pragma unroll
        for (int j = 0; j < RPT; ++j) {
          // padded rows re-read the last channel and meet zero weights
          const unsigned cj = (unsigned)(min(cfirst + j, Cg - 1) - min(cfirst, Cg - 1)) * plane_bytes;
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const float d = *reinterpret_cast<const float*>(base + ((unsigned)off[u] * 4u + cj));
            col[j] = __builtin_fmaf(co[u], co[u] != 0.0f ? d : 0.0f, col[j]);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < RPT; j += 4)
        *reinterpret_cast<float4*>(Bs + gm * kLdK + gpart * RPT + j) =
            make_float4(col[j], col[j + 1], col[j + 2], col[j + 3]);
      // ---- weight tile As[n][r] = Wk[k][c0 / kKC][n0 + n][r]
      const float4* src = reinterpret_cast<const float4*>(
          Wg + (((size_t)k * (CgP / kKC) + c0 / kKC) * CpP + n0) * kKC);
      for (int e = tid; e < TN * kKC / 4; e += kThreads) {
        const int n = e / (kKC / 4), r4 = e % (kKC / 4);
        *reinterpret_cast<float4*>(As + n * kLdK + 4 * r4) = src[e];
      }
      __syncthreads();
      mfma_chunk_kc<MM>(As, a_base, Bs, b_base, acc);
      __syncthreads();
    }
  }

  // ---- epilogue: store (lanes along pixels: 128-byte rows)
  float* pix_b = pix + (size_t)blockIdx.y * Cp * M;
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int m = pixel_of(b_base + 32 * b + (lane & 31));
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + a_base + 32 * a + mfma_row(v, lane);
        if (n < Cp && m >= 0) pix_b[(size_t)n * M + m] = acc[a][b][v];
      }
    }
}

// ---------------------------------------------------------------------------
// gemm_scatter.  Workgroup tile: TC gather-side channels x TM pixels.  For every
// kernel sample k and channel tile: D[c][m] = sum_n Ws[k][n][c] * pix[b][n][m],
// then each accumulator is splatted through the pixel's taps with hardware
// float atomics (lanes own consecutive pixels, so a wave's atomics fall on
// neighbouring addresses).  img must be pre-filled (zeros or bias).
// grid.x = pixel tiles, grid.y = batch.
// ---------------------------------------------------------------------------
template <int INTERP, bool WEIGHTED, int TC, int TM, bool BF16>
__global__ __launch_bounds__(kThreads) void gemm_scatter_kernel(
    const float* __restrict__ pix, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ Wsc, float* __restrict__ img, int Cg, int H, int W, int Cp, int M,
    int K, int P, int CgP, int CpP, int slots, int m_tiles, const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;   // another kernel has done the work
  extern __shared__ __align__(16) unsigned char smem[];
  float* Bs = reinterpret_cast<float*>(smem);             // [kKC][TM]  pix chunk
  float* As = Bs + kKC * TM;                               // [kKC][TC]  weight chunk
  int* tap_off = reinterpret_cast<int*>(As + kKC * TC);
  float* tap_co = reinterpret_cast<float*>(tap_off + slots * TM);
  int* smax = reinterpret_cast<int*>(tap_co + slots * TM);

  constexpr int WAVES_C = TC / 64;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int tile = xcd_band_tile(blockIdx.x, m_tiles);
  const int m0 = tile * TM;
  const int a_base = (wave % WAVES_C) * 64, b_base = (wave / WAVES_C) * 64;
  const size_t HW = (size_t)H * W;
  const float* pix_b = pix + (size_t)blockIdx.y * Cp * M;
  float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  const bool vec_ok = (M % 4 == 0);

  for (int k = 0; k < K; ++k) {
    build_taps<INTERP, WEIGHTED, TM>(map, wts, m0 + tid < M ? m0 + tid : -1, K, k, P, H, W,
                                     tap_off, tap_co, smax);
    const int ns = *smax;
    for (int c0 = 0; c0 < CgP; c0 += TC) {
      floatx16 acc[2][2];
      zero_acc(acc);
      for (int nn0 = 0; nn0 < CpP; nn0 += kKC) {
        // pix chunk Bs[r][m] = pix[b][nn0 + r][m0 + m]
        if (vec_ok) {
          for (int e = tid; e < kKC * TM / 4; e += kThreads) {
            const int r = e / (TM / 4), m4 = (e % (TM / 4)) * 4;
            float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
            if (nn0 + r < Cp && m0 + m4 < M)
              v = *reinterpret_cast<const float4*>(pix_b + (size_t)(nn0 + r) * M + m0 + m4);
            reinterpret_cast<float4*>(Bs)[e] = v;
          }
        } else {
          for (int e = tid; e < kKC * TM; e += kThreads) {
            const int r = e / TM, m = e % TM;
            Bs[e] = (nn0 + r < Cp && m0 + m < M) ? pix_b[(size_t)(nn0 + r) * M + m0 + m] : 0.0f;
          }
        }
        // weight chunk As[r][c] = Ws[k][nn0 + r][c0 + c]
        const float4* src =
            reinterpret_cast<const float4*>(Wsc + ((size_t)k * CpP + nn0) * CgP + c0);
        for (int e = tid; e < kKC * TC / 4; e += kThreads) {
          const int r = e / (TC / 4), c4 = e % (TC / 4);
          reinterpret_cast<float4*>(As)[e] = src[(size_t)r * (CgP / 4) + c4];
        }
        __syncthreads();
        mfma_chunk_any<BF16>(As, TC, a_base, Bs, TM, b_base, kKC, acc);
        __syncthreads();
      }
      // ---- scatter the 64 x 64 block of this wave
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int ml = b_base + 32 * b + (lane & 31);
        for (int s = 0; s < ns; ++s) {
          const int off = tap_off[s * TM + ml];
          const float co = tap_co[s * TM + ml];
          if (co != 0.0f) {
#pragma unroll
            for (int a = 0; a < 2; ++a)
#pragma unroll
              for (int v = 0; v < 16; ++v) {
                const int c = c0 + a_base + 32 * a + mfma_row(v, lane);
                if (c < Cg) atomic_add_noret(img_b + (size_t)c * HW + off, co * acc[a][b][v]);
              }
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// gather_wgrad.  Workgroup: one kernel sample k, one TC x TN tile of gW, one
// batch element and one range of pixels; D[n][c] = sum_m pix[b][n][m] * col[(c,k)][m]
// accumulated over the range in chunks of KM pixels, then added atomically to gW.
// grid.x = 8 * ceil(ranges * batch / 8) * K * c tiles * n tiles; ids past the last range exit.
// LDS: As[KM][TN+1] (pix, transposed), Bs[KM][TC+1] (columns, transposed), taps.
// ---------------------------------------------------------------------------
template <int INTERP, bool WEIGHTED, int KM, bool BF16>
__global__ __launch_bounds__(kThreads) void gather_wgrad_kernel(
    const float* __restrict__ pix, const float* __restrict__ map, const float* __restrict__ wts,
    const float* __restrict__ img, float* __restrict__ gW, int Cg, int H, int W, int Cp, int M,
    int K, int P, int slots, int c_tiles, int n_tiles, int chunks_per_range, int ranges,
    int batches) {
  constexpr int TN = 128, TC = 128, LDA = TN + 1, LDB = TC + 1;
  extern __shared__ __align__(16) unsigned char smem[];
  float* As = reinterpret_cast<float*>(smem);              // [KM][LDA]
  float* Bs = As + KM * LDA;                               // [KM][LDB]
  int* tap_off = reinterpret_cast<int*>(Bs + KM * LDB);    // [slots][KM]
  float* tap_co = reinterpret_cast<float*>(tap_off + slots * KM);
  int* smax = reinterpret_cast<int*>(tap_co + slots * KM);

  constexpr int GROUPS = kThreads / KM;   // channel groups in the gather
  constexpr int CPT = TC / GROUPS;        // channels per thread
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  // 1-D grid.  Workgroup ids go round-robin over the 8 XCDs; all K * c_tiles * n_tiles
  // output tiles of one pixel range read the same pixels of img and pix, so they are
  // given consecutive slots of one XCD and meet in its L2.
  const int kinds = K * c_tiles * n_tiles;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int kind = slot % kinds, range_id = (slot / kinds) * 8 + xcd;
  if (range_id >= ranges * batches) return;
  const int range = range_id % ranges, batch = range_id / ranges;
  const int k = kind / (c_tiles * n_tiles);
  const int c0 = ((kind / n_tiles) % c_tiles) * TC;
  const int n0 = (kind % n_tiles) * TN;
  const int a_base = (wave & 1) * 64, b_base = (wave >> 1) * 64;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)batch * Cg * HW;
  const float* pix_b = pix + (size_t)batch * Cp * M;
  const int gm = tid % KM, grp = tid / KM;

  floatx16 acc[2][2];
  zero_acc(acc);

  const int chunk_beg = range * chunks_per_range;
  const int chunk_end = min(chunk_beg + chunks_per_range, (M + KM - 1) / KM);
  for (int ch = chunk_beg; ch < chunk_end; ++ch) {
    const int m0 = ch * KM;
    build_taps<INTERP, WEIGHTED, KM>(map, wts, m0 + tid < M ? m0 + tid : -1, K, k, P, H, W,
                                     tap_off, tap_co, smax);
    const int ns = *smax;
    // ---- gather columns for KM pixels x TC channels -> Bs[m][c]
    float col[CPT];
#pragma unroll
    for (int j = 0; j < CPT; ++j) col[j] = 0.0f;
    const int cfirst = c0 + (KM >= 64 ? __builtin_amdgcn_readfirstlane(grp) : grp) * CPT;
    for (int s0 = 0; s0 < ns; s0 += 4) {
      int off[4];
      float co[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const bool on = s0 + u < ns;
        off[u] = on ? tap_off[(s0 + u) * KM + gm] : 0;
        co[u] = on ? tap_co[(s0 + u) * KM + gm] : 0.0f;
      }
      const char* base = reinterpret_cast<const char*>(img_b + (size_t)min(cfirst, Cg - 1) * HW);
      const unsigned plane_bytes = (unsigned)HW * 4u;
#pragma unroll
      for (int j = 0; j < CPT; ++j) {
        const unsigned cj = (unsigned)(min(cfirst + j, Cg - 1) - min(cfirst, Cg - 1)) * plane_bytes;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float d = *reinterpret_cast<const float*>(base + ((unsigned)off[u] * 4u + cj));
          col[j] = __builtin_fmaf(co[u], co[u] != 0.0f ? d : 0.0f, col[j]);
        }
      }
    }
#pragma unroll
    for (int j = 0; j < CPT; ++j)
      Bs[gm * LDB + grp * CPT + j] = (cfirst + j < Cg) ? col[j] : 0.0f;
    // ---- pix tile As[m][n] = pix[b][n0 + n][m0 + m]
    {
      constexpr int NPT = TN / GROUPS;
      const bool mok = m0 + gm < M;
#pragma unroll
      for (int j = 0; j < NPT; ++j) {
        const int n = grp * NPT + j;
        As[gm * LDA + n] = (mok && n0 + n < Cp) ? pix_b[(size_t)(n0 + n) * M + m0 + gm] : 0.0f;
      }
    }
    __syncthreads();
    mfma_chunk_any<BF16>(As, LDA, a_base, Bs, LDB, b_base, KM, acc);
    // the next build_taps() starts with a barrier, which also protects As / Bs
  }

  // ---- epilogue: gW[n][c*K + k] += D[n][c]
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const int c = c0 + b_base + 32 * b + (lane & 31);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + a_base + 32 * a + mfma_row(v, lane);
        if (n < Cp && c < Cg)
          atomic_add_noret(gW + (size_t)n * Cg * K + (size_t)c * K + k, acc[a][b][v]);
      }
    }
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------
static int slots_for(const ConvGeom& g) {
  const int nt = (g.interp == 1 || g.interp == 2) ? 4 : 1;
  return pts(g.P) * nt;
}

bool fused_supported(const ConvGeom& g) {
  if (slots_for(g) > kMaxSlots) return false;
  if ((int64_t)g.H * g.W > ((int64_t)1 << 24)) return false;  // 32-bit byte offsets over 32 planes
  if (g.B > 65535) return false;
  return true;
}

static bool inverse_candidate(const ConvGeom& g);
static size_t inverse_bytes(const ConvGeom& g);
static bool scatter_tries_inverse(const ConvGeom& g);
static size_t inverse_ws_offset(const ConvGeom& g);
// Tail of the workspace used by the weight gradient: partial sums of the plan-driven kernel,
// those of the window kernel, the tile lists.
struct WgradTail {
  size_t partial, window_partial, lists, total;
};
static WgradTail wgrad_tail(const ConvGeom& g) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  WgradTail t;
  t.partial = 0;
  t.window_partial = up(planned_wgrad_partial_bytes(g));
  t.lists = t.window_partial + up(window_wgrad_partial_bytes(g));
  t.total = t.lists + (window_wgrad_partial_bytes(g) != 0 ? up(tile_lists_bytes(g)) : 0);
  return t;
}

// Scratch of the forward-style contraction when it runs from the plan: the weight copy of the
// global-gather kernel, the plan, the tile lists and the weight copy of the window kernel.
struct GatherLayout {
  size_t plan, lists, window_weights, total;
};
static GatherLayout gather_layout(const ConvGeom& g) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  GatherLayout l;
  l.plan = up((size_t)g.K * round_up(g.Cp, 128) * round_up(g.Cg, 128) * sizeof(float));
  l.lists = l.plan + up(plan_bytes(g));
  l.window_weights = l.lists + up(tile_lists_bytes(g));
  l.total = l.window_weights + up(window_gemm_weight_bytes(g));
  return l;
}
static bool gather_from_window(const ConvGeom& g) { return window_gemm_supported(g); }

size_t fused_workspace_bytes(const ConvGeom& g) {
  const int CpP = round_up(g.Cp, 128), CgP = round_up(g.Cg, 128);
  size_t need = std::max((size_t)g.K * CpP * CgP * sizeof(float), staged_workspace_bytes(g));
  if (gather_from_window(g)) need = std::max(need, gather_layout(g).total);
  if (plan_supported(g)) need = ((need + 255) & ~(size_t)255) + plan_bytes(g);
  if (scatter_tries_inverse(g)) need = std::max(need, inverse_ws_offset(g) + inverse_bytes(g));
  need = std::max(need, product_workspace_bytes(g));
  // last: the weight gradient's tile lists and partial sums (the plan and, in a combined
  // backward call, everything before it are still in use when they are written)
  return ((need + 255) & ~(size_t)255) + wgrad_tail(g).total;
}

static char* wgrad_tail_base(const ConvGeom& g, float* workspace) {
  return reinterpret_cast<char*>(workspace) + (fused_workspace_bytes(g) - wgrad_tail(g).total);
}
static float* wgrad_partial(const ConvGeom& g, float* workspace) {
  if (planned_wgrad_partial_bytes(g) == 0) return nullptr;
  return reinterpret_cast<float*>(wgrad_tail_base(g, workspace) + wgrad_tail(g).partial);
}

// gW += the sums of a plan: tiles that fit the window kernel there, the others (and every
// tile when that kernel does not cover the call) in the plan-driven kernel.
static int wgrad_from_plan(const ConvGeom& g, int mm, const Plan& plan, const float* pix,
                           const float* img, float* gW, float* workspace, hipStream_t stream,
                           const TileLists* lists4 = nullptr) {
  if (window_wgrad_supported(g, mm) && window_wgrad_partial_bytes(g) != 0) {
    const WgradTail t = wgrad_tail(g);
    char* base = wgrad_tail_base(g, workspace);
    TileLists tl;
    int rc = SDK_OK;
    if (lists4 != nullptr) tl = *lists4;
    else rc = build_tile_lists(plan, base + t.lists, stream, &tl, 4);
    if (rc) return rc;
    float* wp = reinterpret_cast<float*>(base + t.window_partial);
    rc = window_wgrad(g, mm, plan, tl, pix, img, gW, wp, stream);
    if (rc) return rc;
    if (plan.big_lut != nullptr) {
      // big tiles from their big windows (the partial sums of the first launch have been added
      // up by then), what is left from global memory
      rc = window_wgrad(g, mm, plan, tl, pix, img, gW, wp, stream, true);
      if (rc) return rc;
      return planned_wgrad(g, mm, plan, pix, img, gW, wgrad_partial(g, workspace), stream,
                           tl.rest_small, tl.count + 3);
    }
    return planned_wgrad(g, mm, plan, pix, img, gW, wgrad_partial(g, workspace), stream, tl.rest,
                         tl.count + 1);
  }
  if (window_wgrad_narrow_supported(g, mm) && window_wgrad_partial_bytes(g) != 0) {
    // narrow layers with one plan row per sample: the tiles inside their window from the
    // window, the others from global memory
    const WgradTail t = wgrad_tail(g);
    char* base = wgrad_tail_base(g, workspace);
    TileLists tl;
    int rc = SDK_OK;
    if (lists4 != nullptr) tl = *lists4;
    else rc = build_tile_lists(plan, base + t.lists, stream, &tl, 4);
    if (rc) return rc;
    float* wp = reinterpret_cast<float*>(base + t.window_partial);
    rc = window_wgrad_narrow(g, mm, plan, tl, pix, img, gW, wp, stream);
    if (rc) return rc;
    if (window_wgrad_big_supported(g, mm) && plan.big_lut != nullptr) {
      rc = window_wgrad(g, mm, plan, tl, pix, img, gW, wp, stream, true);
      if (rc) return rc;
      return planned_wgrad(g, mm, plan, pix, img, gW, wgrad_partial(g, workspace), stream,
                           tl.rest_small, tl.count + 3);
    }
    return planned_wgrad(g, mm, plan, pix, img, gW, wgrad_partial(g, workspace), stream, tl.rest,
                         tl.count + 1);
  }
  if (window_wgrad_big_supported(g, mm) && window_wgrad_partial_bytes(g) != 0 &&
      plan.big_lut != nullptr) {
    // at most 64 pixel-side channels: the big tiles from their big windows, every other tile
    // in the plan-driven kernel
    const WgradTail t = wgrad_tail(g);
    char* base = wgrad_tail_base(g, workspace);
    TileLists tl;
    int rc = SDK_OK;
    if (lists4 != nullptr) tl = *lists4;
    else rc = build_tile_lists(plan, base + t.lists, stream, &tl, 4);
    if (rc) return rc;
    rc = window_wgrad(g, mm, plan, tl, pix, img, gW,
                      reinterpret_cast<float*>(base + t.window_partial), stream, true);
    if (rc) return rc;
    return planned_wgrad(g, mm, plan, pix, img, gW, wgrad_partial(g, workspace), stream,
                         tl.not_big, tl.count + 6);
  }
  return planned_wgrad(g, mm, plan, pix, img, gW, wgrad_partial(g, workspace), stream);
}

static int relayout(const ConvGeom& g, const float* Wm, float* out, int CpP, int CgP,
                    int n_fastest, hipStream_t stream) {
  const size_t total = (size_t)g.K * CpP * CgP;
  const int blocks = (int)std::min<size_t>((total + kThreads - 1) / kThreads, 2048);
  launch(relayout_weight_kernel, dim3(blocks), dim3(kThreads), stream, Wm, out, g.Cp, g.Cg, g.K,
         CpP, CgP, n_fastest);
  SDK_LAUNCH_CHECK("relayout_weight");
  return SDK_OK;
}

template <typename Kern, typename... Args>
static int launch_smem(const char* what, Kern kern, dim3 grid, size_t smem, hipStream_t stream,
                       Args... args) {
  if (smem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    if (e != hipSuccess)
      return fail(SDK_ERR_DEVICE, "%s: cannot reserve %zu bytes of LDS: %s", what, smem,
                  hipGetErrorString(e));
  }
  kern<<<grid, dim3(kThreads), smem, stream>>>(args...);
  SDK_LAUNCH_CHECK(what);
  return SDK_OK;
}

int fused_gather_gemm(const ConvGeom& g, int compute, const float* img, const float* map,
                      const float* wts, const float* Wm, const float* bias, float* pix,
                      float* workspace, hipStream_t stream, const CachedPlan* cached) {
  // images of a few channels: the packed kernel (a 32-channel chunk would be mostly padding)
  if (small_conv_supported(g)) return small_forward(g, img, map, wts, Wm, bias, pix, stream);
  const int mm = matrix_mode(compute);
  const int slots = slots_for(g);
  const bool narrow = g.Cp <= 64;
  const int TN = narrow ? 64 : 128, TM = narrow ? 256 : 128;
  const int CpP = round_up(g.Cp, TN), CgP = round_up(g.Cg, kKC);
  int rc = relayout(g, Wm, workspace, CpP, CgP, 2, stream);
  if (rc) return rc;
  const size_t smem = sizeof(float) * kLdK * (TM + TN) + (size_t)slots * TM * 8 + 16;
  if (gather_from_window(g)) {
    // Tiles whose taps stay inside an LDS-sized window of the image are gathered from that
    // window (window_gemm), the others (polar rows of a spherical map, incoherent maps) from
    // global memory by the kernel below, which takes their list.
    const GatherLayout l = gather_layout(g);
    char* ws = reinterpret_cast<char*>(workspace);
    Plan plan;
    TileLists tl;
    if (cached != nullptr) {
      plan = cached->plan;
      tl = cached->lists;
    } else {
      rc = build_plan(g, map, wts, ws + l.plan, stream, &plan);
      if (rc) return rc;
      rc = build_tile_lists(plan, ws + l.lists, stream, &tl);
      if (rc) return rc;
    }
    rc = window_gemm(g, mm, plan, tl, img, Wm, false, bias, pix,
                     reinterpret_cast<float*>(ws + l.window_weights), nullptr, stream);
    if (rc) return rc;
    // big tiles from their big windows; the rest list below is then what neither kernel took
    const bool with_big = plan.big_lut != nullptr;
    if (with_big) {
      rc = window_gemm(g, mm, plan, tl, img, Wm, false, bias, pix,
                       reinterpret_cast<float*>(ws + l.window_weights), nullptr, stream, kListBig);
      if (rc) return rc;
    }
    const int* rest_list = with_big ? tl.rest_small : tl.rest;
    const int* rest_count = with_big ? tl.count + 3 : tl.count + 1;
    // the listed rest: 128 x 128 tiles, or 64 channels x two listed tiles for narrow layers
    const int units = (int)ceil_div(plan.tiles, TM / 128);
    const dim3 grid_t((unsigned)((units + 7) / 8 * 8 * (CpP / TN)), (unsigned)g.B);
#define GT2(TNv, TMv, BFv)                                                                        \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                              \
                      (rc = launch_smem("gather_gemm(tiles)",                                     \
                                        gather_gemm_kernel<INTERP, WEIGHTED, TNv, TMv, BFv, false, true>, \
                                        grid_t, smem, stream, img, map, wts,                      \
                                        (const float*)workspace, bias, pix, g.Cg, g.H, g.W, g.Cp, \
                                        g.M, g.K, g.P, CgP, CpP, slots, plan.tiles,               \
                                        (const int*)nullptr, (const float*)nullptr,               \
                                        (const int*)nullptr, (const int*)nullptr, plan.pt,        \
                                        rest_list, rest_count)))
#define GT(BFv)                                                  \
  do {                                                           \
    if (narrow) GT2(64, 256, BFv); else GT2(128, 128, BFv);      \
  } while (0)
    if (mm == kMmBf16) GT(kMmBf16); else if (mm == kMmSplit) GT(kMmSplit); else GT(kMmF32);
#undef GT2
#undef GT
    return rc;
  }
  const int m_tiles = (int)ceil_div(g.M, TM), n_tiles = CpP / TN;
  const dim3 grid((unsigned)(m_tiles * n_tiles), (unsigned)g.B);
#define GG(TNv, TMv, BFv)                                                                          \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                          \
                      (rc = launch_smem("gather_gemm",                                        \
                                        gather_gemm_kernel<INTERP, WEIGHTED, TNv, TMv, BFv>, grid, \
                                        smem, stream, img, map, wts, (const float*)workspace, \
                                        bias, pix, g.Cg, g.H, g.W, g.Cp, g.M, g.K, g.P, CgP,  \
                                        CpP, slots, m_tiles, (const int*)nullptr,             \
                                        (const float*)nullptr, (const int*)nullptr,           \
                                        (const int*)nullptr, PixelTiling(), (const int*)nullptr, \
                                        (const int*)nullptr)))
  if (mm == kMmBf16) { if (narrow) GG(64, 256, kMmBf16); else GG(128, 128, kMmBf16); }
  else if (mm == kMmSplit) { if (narrow) GG(64, 256, kMmSplit); else GG(128, 128, kMmSplit); }
  else { if (narrow) GG(64, 256, kMmF32); else GG(128, 128, kMmF32); }
#undef GG
  return rc;
}


// ---------------------------------------------------------------------------
// Inverse map: the scatter  img[u] += co * v[m, k]  over all taps (m, k) -> u, regrouped by
// target u, so that gemm_scatter can run as gather_gemm over the pixel-side tensor with no
// atomics.  Rows: for target tile t (TM consecutive image elements), sample k, slot s < kInvSlots:
// source pixel inv_off[((t*K + k)*kInvSlots + s)*TM + u % TM] and coefficient inv_co[...] (0 = empty).
// cnt[u*K + k] counts the sources of (u, k); *gate counts taps that found no free slot: the
// inverse is usable only if it stays 0.
// ---------------------------------------------------------------------------
constexpr int kInvSlots = 16;

template <int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kThreads) void inverse_fill_kernel(
    const float* __restrict__ map, const float* __restrict__ wts, int M, int K, int P, int H, int W,
    int TM, int* __restrict__ cnt, int* __restrict__ inv_off, float* __restrict__ inv_co,
    int* __restrict__ gate) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= (size_t)M * K) return;
  const int m = (int)(i / K), k = (int)(i % K);
  const int q = WEIGHTED ? P : 1;
  PointTaps<float, INTERP> t;
  for (int p = 0; p < q; ++p) {
    const size_t s = i * q + p;
    t.set(map[s * 2], map[s * 2 + 1], H, W);
    const float wt = WEIGHTED ? wts[s] : 1.0f;
#pragma unroll
    for (int j = 0; j < PointTaps<float, INTERP>::N; ++j) {
      const float co = WEIGHTED ? wt * t.w[j] : t.w[j];
      if (t.off[j] >= 0 && co != 0.0f) {
        const int u = t.off[j];
        const int slot = atomicAdd(&cnt[(size_t)u * K + k], 1);
        if (slot < kInvSlots) {
          const size_t e = (((size_t)(u / TM) * K + k) * kInvSlots + slot) * TM + u % TM;
          inv_off[e] = m;
          inv_co[e] = co;
        } else {
          atomicAdd(gate, 1);
        }
      }
    }
  }
}

// ns[t*K + k] = largest source count of any target of tile t for sample k (capped at the slots)
__global__ __launch_bounds__(kThreads) void inverse_rows_kernel(const int* __restrict__ cnt, int HW,
                                                                int K, int TM,
                                                                int* __restrict__ ns) {
  __shared__ int mx[256];
  const int t = blockIdx.x, tid = threadIdx.x;
  for (int k = tid; k < K; k += kThreads) mx[k] = 0;
  __syncthreads();
  for (int e = tid; e < TM * K; e += kThreads) {
    const int u = t * TM + e / K, k = e % K;   // cnt rows of a tile are contiguous: coalesced
    if (u < HW) {
      const int c = cnt[(size_t)u * K + k];
      if (c > 0) atomicMax(&mx[k], min(c, kInvSlots));
    }
  }
  __syncthreads();
  for (int k = tid; k < K; k += kThreads) ns[(size_t)t * K + k] = mx[k];
}

struct InverseMap {
  int TM, tiles;
  int* gate;
  int* cnt;
  int* ns;
  int* off;
  float* co;
  float* weights;   // Ws[k][n][c] copy for the gather kernel
};

static bool inverse_candidate(const ConvGeom& g) {
  // Inverse lists are as short as the map is injective per sample: one source per target for a
  // one-to-one map, about as many as a sample has taps for a map of unit scale.  K <= 256 for
  // the row-count kernel; the pixel side is gathered with 32-bit offsets.
  return g.K <= 256 && g.M <= (1 << 24);
}

static int inverse_tm(const ConvGeom& g) { return g.Cg <= 64 ? 256 : 128; }

static void inverse_layout(const ConvGeom& g, size_t (&off)[7]) {
  const size_t HW = (size_t)g.H * g.W, TM = inverse_tm(g), tiles = (HW + TM - 1) / TM;
  const size_t rows = tiles * g.K * kInvSlots * TM;
  const int TN = g.Cg <= 64 ? 64 : 128;
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  off[0] = 0;                                  // gate
  off[1] = 256;                                // cnt
  off[2] = off[1] + up(HW * g.K * 4);          // co   (gate, cnt, co are cleared together)
  off[3] = off[2] + up(rows * 4);              // off
  off[4] = off[3] + up(rows * 4);              // ns
  off[5] = off[4] + up(tiles * g.K * 4);       // weights
  off[6] = off[5] + up((size_t)g.K * round_up(g.Cp, kKC) * round_up(g.Cg, TN) * 4);
}

// The scatter's geometry seen as the gather it becomes over the inverse plan: the pixel-side
// tensor is gathered (planes of OH x OW), the image side is produced.
static ConvGeom inverse_geom(const ConvGeom& g) {
  ConvGeom r = g;
  r.Cg = g.Cp;
  r.H = g.M / g.OW;
  r.W = g.OW;
  r.Cp = g.Cg;
  r.M = g.H * g.W;
  r.OW = g.W;
  r.P = kInversePlanRows / 4;   // plan rows per sample: kInversePlanRows (bilinear slots x P)
  r.interp = 1;
  return r;
}
static bool scatter_from_window(const ConvGeom& g) {
  return g.M % g.OW == 0 && window_gemm_supported(inverse_geom(g)) &&
         (int64_t)g.H * g.W * g.K < ((int64_t)1 << 31);
}
// Scratch of the scatter run from the inverse plan (behind the forward plan's region).
struct ScatterLayout {
  size_t inverse, lists, window_weights, gather_weights, total;
};
static ScatterLayout scatter_layout(const ConvGeom& g) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const ConvGeom r = inverse_geom(g);
  ScatterLayout l;
  l.inverse = 0;
  l.lists = up(inverse_plan_bytes(g));
  l.window_weights = l.lists + up(tile_lists_bytes(r));
  l.gather_weights = l.window_weights + up(window_gemm_weight_bytes(r));
  l.total = l.gather_weights +
            up((size_t)g.K * round_up(g.Cp, kKC) * round_up(g.Cg, 128) * sizeof(float));
  return l;
}

static size_t inverse_bytes(const ConvGeom& g) {
  if (scatter_from_window(g)) return scatter_layout(g).total;
  size_t off[7];
  inverse_layout(g, off);
  return off[6];
}

// The scatter runs as a gather over an inverse map or plan whenever one can be built: always
// beside the plan-driven scatter kernel (its fallback when a target has too many sources), and
// through the window kernels also where that kernel does not reach (more than 128 pixel-side
// channels), with the atomic scatter kernel as the fallback.
static bool scatter_tries_inverse(const ConvGeom& g) {
  return inverse_candidate(g) && (planned_scatter_supported(g) || scatter_from_window(g));
}
// Where the inverse structures start in the workspace: behind the weight copies of the fallback
// kernels and the tap plan.
static size_t inverse_ws_offset(const ConvGeom& g) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const size_t weights = std::max((size_t)g.K * round_up(g.Cp, 128) * round_up(g.Cg, 128) * sizeof(float),
                                  staged_workspace_bytes(g));
  return up(up(weights) + (plan_supported(g) ? plan_bytes(g) : 0));
}

static int build_inverse(const ConvGeom& g, const float* map, const float* wts, char* ws,
                         hipStream_t stream, InverseMap* inv) {
  size_t off[7];
  inverse_layout(g, off);
  const int HW = g.H * g.W;
  inv->TM = inverse_tm(g);
  inv->tiles = (int)ceil_div(HW, inv->TM);
  inv->gate = reinterpret_cast<int*>(ws + off[0]);
  inv->cnt = reinterpret_cast<int*>(ws + off[1]);
  inv->co = reinterpret_cast<float*>(ws + off[2]);
  inv->off = reinterpret_cast<int*>(ws + off[3]);
  inv->ns = reinterpret_cast<int*>(ws + off[4]);
  inv->weights = reinterpret_cast<float*>(ws + off[5]);
  int rc = zero_fill(ws, off[3], stream);
  if (rc) return rc;
  const int64_t total = (int64_t)g.M * g.K;
  if (ceil_div(total, kThreads) >= ((int64_t)1 << 31))
    return fail(SDK_ERR_UNSUPPORTED, "inverse map: too many samples");
  SDK_DISPATCH_INTERP(g.interp, g.P,
                      (launch(inverse_fill_kernel<INTERP, WEIGHTED>,
                              dim3((unsigned)ceil_div(total, kThreads)), dim3(kThreads), stream, map,
                              wts, g.M, g.K, g.P, g.H, g.W, inv->TM, inv->cnt, inv->off, inv->co,
                              inv->gate)));
  SDK_LAUNCH_CHECK("inverse_fill");
  launch(inverse_rows_kernel, dim3((unsigned)inv->tiles), dim3(kThreads), stream,
         (const int*)inv->cnt, HW, g.K, inv->TM, inv->ns);
  SDK_LAUNCH_CHECK("inverse_rows");
  return SDK_OK;
}

// img[b] = Ws^T x gather(pix[b]) + bias over the inverse map; does nothing if *inv.gate != 0.
static int inverse_gather_gemm(const ConvGeom& g, int mm, const InverseMap& inv,
                               const float* pix, const float* Wm, const float* bias, float* img,
                               hipStream_t stream) {
  // roles in the gather kernel: gathered tensor = pix (Cp channels, planes of M elements),
  // output = img (Cg channels, H*W elements), weights Ws[k][n][c] with c contiguous
  const bool narrow = g.Cg <= 64;
  const int TN = narrow ? 64 : 128, TM = inv.TM;
  const int CoutP = round_up(g.Cg, TN), CinP = round_up(g.Cp, kKC);
  int rc = relayout(g, Wm, inv.weights, CoutP, CinP, 3, stream);
  if (rc) return rc;
  const int HW = g.H * g.W;
  const int m_tiles = inv.tiles, n_tiles = CoutP / TN;
  const dim3 grid((unsigned)(m_tiles * n_tiles), (unsigned)g.B);
  const size_t smem = sizeof(float) * kLdK * (TM + TN) + (size_t)kInvSlots * TM * 8 + 16;
#define IG(TNv, TMv, BFv)                                                                        \
  rc = launch_smem("inverse_gather_gemm", gather_gemm_kernel<0, false, TNv, TMv, BFv, true>, grid, \
                   smem, stream, pix, (const float*)nullptr, (const float*)nullptr,              \
                   (const float*)inv.weights, bias, img, g.Cp, 1, g.M, g.Cg, HW, g.K, 0, CinP,   \
                   CoutP, kInvSlots, m_tiles, (const int*)inv.off, (const float*)inv.co,         \
                   (const int*)inv.ns, (const int*)inv.gate, PixelTiling(), (const int*)nullptr, \
                   (const int*)nullptr)
  if (mm == kMmBf16) { if (narrow) IG(64, 256, kMmBf16); else IG(128, 128, kMmBf16); }
  else if (mm == kMmSplit) { if (narrow) IG(64, 256, kMmSplit); else IG(128, 128, kMmSplit); }
  else { if (narrow) IG(64, 256, kMmF32); else IG(128, 128, kMmF32); }
#undef IG
  return rc;
}

int fused_gemm_scatter(const ConvGeom& g, int compute, const float* pix, const float* map,
                       const float* wts, const float* Wm, const float* bias, float* img,
                       float* workspace, hipStream_t stream, SharedPlan* shared,
                       const CachedPlan* cached) {
  const bool bf16 = compute == SDK_COMPUTE_BF16;
  int rc = SDK_OK;
  if (small_conv_supported(g)) {
    // images of a few channels: fill, then the packed scatter kernel
    if (!(shared != nullptr && shared->cleared && bias == nullptr))
      rc = plane_fill<float>(img, bias, g.B * g.Cg, g.Cg, (size_t)g.H * g.W, stream);
    if (rc) return rc;
    if (shared != nullptr) shared->valid = false;
    return small_scatter(g, pix, map, wts, Wm, img, stream);
  }
  if (product_route(g)) {
    // the image is finer than the pixel grid: products at the grid's resolution, then their
    // splat as a gather (conv_product.hip)
    if (shared != nullptr) shared->valid = false;
    return product_gemm_scatter(g, pix, map, wts, Wm, bias, img, workspace, stream,
                                cached != nullptr ? cached->col2im_lists : nullptr);
  }
  const bool planned_fb = planned_scatter_supported(g);
  const int* generic_gate = nullptr;   // gate of the atomic scatter kernel at the end
  bool filled = false;
  if (scatter_tries_inverse(g)) {
    const int* gate = nullptr;
    {
      // Try the scatter as a gather over the inverse map.  The inverse is built on the device;
      // if a target collects more sources than its rows hold, the gather kernel exits at once
      // and the fill and the scatter kernel below run instead (and vice versa).
      char* inv_ws = reinterpret_cast<char*>(workspace) + inverse_ws_offset(g);
      if (scatter_from_window(g)) {
        // the inverse lists as a plan: image tiles whose sources stay inside a window of the
        // pixel grid gather from LDS, the others from global memory
        const int mm = matrix_mode(compute);
        const ScatterLayout l = scatter_layout(g);
        const ConvGeom r = inverse_geom(g);
        InversePlan ip;
        TileLists tl;
        if (cached != nullptr && cached->has_inverse) {
          ip = cached->inverse;
          tl = cached->inverse_lists;
        } else {
          rc = build_inverse_plan(g, map, wts, inv_ws + l.inverse, stream, &ip);
          if (rc) return rc;
          rc = build_tile_lists(ip.plan, inv_ws + l.lists, stream, &tl, 0, kProductCap);
          if (rc) return rc;
        }
        float* ww = reinterpret_cast<float*>(inv_ws + l.window_weights);
        // image tiles with few sources (the image finer than the pixel grid) in the product
        // form where it exists, all others inside their window in the gather form
        const bool product = window_product_supported(r, mm);
        rc = window_gemm(r, mm, ip.plan, tl, pix, Wm, true, bias, img, ww, ip.gate, stream,
                         product ? kListInsideLarge : kListInside);
        if (rc) return rc;
        if (product) {
          rc = window_product(r, ip.plan, tl, pix, bias, img, ww, ip.gate, stream);
          if (rc) return rc;
        }
        const bool with_big = ip.plan.big_lut != nullptr;
        if (with_big) {
          rc = window_gemm(r, mm, ip.plan, tl, pix, Wm, true, bias, img, ww, ip.gate, stream,
                           kListBig);
          if (rc) return rc;
        }
        const int* rest_list = with_big ? tl.rest_small : tl.rest;
        const int* rest_count = with_big ? tl.count + 3 : tl.count + 1;
        float* gw = reinterpret_cast<float*>(inv_ws + l.gather_weights);
        // the listed rest: 128 x 128 tiles, or 64 channels x two listed tiles for narrow images
        const bool narrow = g.Cg <= 64;
        const int TN = narrow ? 64 : 128, TM = narrow ? 256 : 128;
        const int CoutP = round_up(g.Cg, TN), CinP = round_up(g.Cp, kKC);
        rc = relayout(g, Wm, gw, CoutP, CinP, 3, stream);
        if (rc) return rc;
        const int units = (int)ceil_div(ip.plan.tiles, TM / 128);
        const dim3 grid_t((unsigned)((units + 7) / 8 * 8 * (CoutP / TN)), (unsigned)g.B);
        const size_t smem = sizeof(float) * kLdK * (TM + TN) + (size_t)kInversePlanRows * TM * 8 + 16;
#define IT2(TNv, TMv, BFv)                                                                       \
  rc = launch_smem("inverse_gather_gemm(tiles)",                                                 \
                   gather_gemm_kernel<0, false, TNv, TMv, BFv, true, true>, grid_t, smem, stream, \
                   pix, (const float*)nullptr, (const float*)nullptr, (const float*)gw, bias,    \
                   img, g.Cp, 1, g.M, g.Cg, g.H * g.W, g.K, 0, CinP, CoutP, kInversePlanRows,    \
                   ip.plan.tiles, (const int*)ip.raw_off, (const float*)ip.raw_co,               \
                   (const int*)ip.plan.ns, (const int*)ip.gate, ip.plan.pt, rest_list, rest_count)
#define IT(BFv)                                                  \
  do {                                                           \
    if (narrow) IT2(64, 256, BFv); else IT2(128, 128, BFv);      \
  } while (0)
        if (mm == kMmBf16) IT(kMmBf16); else if (mm == kMmSplit) IT(kMmSplit); else IT(kMmF32);
#undef IT2
#undef IT
        if (rc) return rc;
        gate = ip.gate;
      } else {
        InverseMap inv;
        rc = build_inverse(g, map, wts, inv_ws, stream, &inv);
        if (rc) return rc;
        rc = inverse_gather_gemm(g, matrix_mode(compute), inv, pix, Wm, bias, img, stream);
        if (rc) return rc;
        gate = inv.gate;
      }
    }
    rc = plane_fill<float>(img, bias, g.B * g.Cg, g.Cg, (size_t)g.H * g.W, stream, gate);
    if (rc) return rc;
    filled = true;
    generic_gate = gate;
  }
  if (planned_fb) {
    if (!filled) {
      rc = plane_fill<float>(img, bias, g.B * g.Cg, g.Cg, (size_t)g.H * g.W, stream);
      if (rc) return rc;
    }
    if (cached != nullptr && shared != nullptr) {
      // the weight gradient of this call takes the cached plan; the scatter kernel (which runs
      // only if the gate is raised) builds its own
      shared->plan = cached->plan;
      shared->valid = true;
      return planned_gemm_scatter(g, bf16, pix, map, wts, Wm, img, workspace, generic_gate, stream,
                                  nullptr);
    }
    return planned_gemm_scatter(g, bf16, pix, map, wts, Wm, img, workspace, generic_gate, stream,
                                shared);
  }
  if (!filled) {
    rc = plane_fill<float>(img, bias, g.B * g.Cg, g.Cg, (size_t)g.H * g.W, stream);
    if (rc) return rc;
  }
  const int slots = slots_for(g);
  const bool narrow = g.Cg <= 64;
  const int TC = narrow ? 64 : 128, TM = narrow ? 256 : 128;
  const int CgP = round_up(g.Cg, TC), CpP = round_up(g.Cp, kKC);
  rc = relayout(g, Wm, workspace, CpP, CgP, false, stream);
  if (rc) return rc;
  const int m_tiles = (int)ceil_div(g.M, TM);
  const dim3 grid((unsigned)m_tiles, (unsigned)g.B);
  const size_t smem = sizeof(float) * (kKC * TM + kKC * TC) + (size_t)slots * TM * 8 + 16;
#define GS(TCv, TMv, BFv)                                                                           \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                           \
                      (rc = launch_smem("gemm_scatter",                                        \
                                        gemm_scatter_kernel<INTERP, WEIGHTED, TCv, TMv, BFv>, grid, \
                                        smem, stream, pix, map, wts, (const float*)workspace,  \
                                        img, g.Cg, g.H, g.W, g.Cp, g.M, g.K, g.P, CgP, CpP,    \
                                        slots, m_tiles, generic_gate)))
  if (bf16) { if (narrow) GS(64, 256, true); else GS(128, 128, true); }
  else { if (narrow) GS(64, 256, false); else GS(128, 128, false); }
#undef GS
  return rc;
}

int fused_gather_wgrad(const ConvGeom& g, int compute, const float* pix, const float* map,
                       const float* wts, const float* img, float* gW, float* workspace,
                       hipStream_t stream, const SharedPlan* shared, const CachedPlan* cached) {
  const bool bf16 = compute == SDK_COMPUTE_BF16;
  const bool cleared = shared != nullptr && shared->cleared && small_wgrad_supported(g);
  int rc = cleared ? SDK_OK : zero_fill(gW, sizeof(float) * (size_t)g.Cp * g.Cg * g.K, stream);
  if (rc) return rc;
  if (g.B == 0) return SDK_OK;
  if (small_wgrad_supported(g))
    return small_wgrad(g, pix, map, wts, img, gW, stream, cleared ? shared->bias_sum : nullptr);
  if (planned_wgrad_supported(g)) {
    if (cached != nullptr)
      return wgrad_from_plan(g, matrix_mode(compute), cached->plan, pix, img, gW, workspace,
                             stream, &cached->lists4);
    if (shared != nullptr && shared->valid)
      return wgrad_from_plan(g, matrix_mode(compute), shared->plan, pix, img, gW, workspace,
                             stream);
    Plan plan;
    rc = build_plan(g, map, wts, workspace, stream, &plan);
    if (rc) return rc;
    return wgrad_from_plan(g, matrix_mode(compute), plan, pix, img, gW, workspace, stream);
  }
  constexpr int KM = 64;
  const int slots = slots_for(g);
  const int c_tiles = (int)ceil_div(g.Cg, 128), n_tiles = (int)ceil_div(g.Cp, 128);
  const int chunks = (int)ceil_div(g.M, KM);
  // enough pixel ranges for ~8 workgroups per CU overall, at least 8 chunks each
  const int64_t base = (int64_t)g.K * c_tiles * n_tiles * g.B;
  int ranges = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(2048, base), ceil_div(chunks, 8)));
  ranges = std::min(ranges, 65535);
  const int cpr = (int)ceil_div(chunks, ranges);
  ranges = (int)ceil_div(chunks, cpr);
  const int64_t slots_total = ceil_div((int64_t)ranges * g.B, 8) * 8 * g.K * c_tiles * n_tiles;
  if (slots_total >= ((int64_t)1 << 31))
    return fail(SDK_ERR_UNSUPPORTED, "gather_wgrad: grid too large");
  const dim3 grid((unsigned)slots_total, 1, 1);
  const size_t smem = sizeof(float) * (size_t)KM * (129 + 129) + (size_t)slots * KM * 8 + 16;
#define GW(BFv)                                                                                 \
  SDK_DISPATCH_INTERP(g.interp, g.P,                                                            \
                      (rc = launch_smem("gather_wgrad",                                         \
                                        gather_wgrad_kernel<INTERP, WEIGHTED, KM, BFv>, grid,   \
                                        smem, stream, pix, map, wts, img, gW, g.Cg, g.H, g.W,   \
                                        g.Cp, g.M, g.K, g.P, slots, c_tiles, n_tiles, cpr,      \
                                        ranges, (int)g.B)))
  if (bf16) GW(true); else GW(false);
#undef GW
  return rc;
}

// ---------------------------------------------------------------------------
// Cached plan: [tap plan][tile lists][tile lists, at most four rows][inverse plan][its lists]
// ---------------------------------------------------------------------------
namespace {
struct CachedLayout {
  size_t plan, lists, lists4, inverse, inverse_lists, col2im, total;
  bool has_inverse, has_col2im;
};
CachedLayout cached_layout(const ConvGeom& g) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  CachedLayout l;
  l.plan = 0;
  l.lists = up(plan_bytes(g));
  l.lists4 = l.lists + up(tile_lists_bytes(g));
  l.inverse = l.lists4 + up(tile_lists_bytes(g));
  // the inverse plan as scatter_from_window() needs it, whatever the channel counts
  l.has_inverse = g.K <= 256 && g.M <= (1 << 24) && g.M % g.OW == 0 &&
                  plan_supported(inverse_geom(g)) &&
                  (int64_t)g.H * g.W * g.K < ((int64_t)1 << 31);
  l.inverse_lists = l.inverse + (l.has_inverse ? up(inverse_plan_bytes(g)) : 0);
  l.col2im = l.inverse_lists + (l.has_inverse ? up(tile_lists_bytes(inverse_geom(g))) : 0);
  // the inverted map of the product route (conv_product.hpp), where the map may take it
  l.has_col2im = product_route_map(g);
  l.total = l.col2im + (l.has_col2im ? up(col2im_lists_bytes(g.H, g.W, g.M, g.K, g.P, g.interp)) : 0);
  return l;
}
}  // namespace

size_t cached_plan_bytes(const ConvGeom& g) {
  if (!plan_supported(g) || (int64_t)g.H * g.W > ((int64_t)1 << 24)) return 0;
  return cached_layout(g).total;
}

void load_cached_plan(const ConvGeom& g, void* buffer, CachedPlan* out) {
  const CachedLayout l = cached_layout(g);
  char* b = static_cast<char*>(buffer);
  load_plan(g, b + l.plan, &out->plan);
  load_tile_lists(out->plan, b + l.lists, &out->lists);
  load_tile_lists(out->plan, b + l.lists4, &out->lists4);
  out->has_inverse = l.has_inverse;
  if (l.has_inverse) {
    load_inverse_plan(g, b + l.inverse, &out->inverse);
    load_tile_lists(out->inverse.plan, b + l.inverse_lists, &out->inverse_lists);
  }
  out->col2im_lists = l.has_col2im ? b + l.col2im : nullptr;
}

int build_cached_plan(const ConvGeom& g, const float* map, const float* wts, void* buffer,
                      hipStream_t stream) {
  const CachedLayout l = cached_layout(g);
  char* b = static_cast<char*>(buffer);
  CachedPlan cp;
  int rc = build_plan(g, map, wts, b + l.plan, stream, &cp.plan);
  if (rc) return rc;
  rc = build_tile_lists(cp.plan, b + l.lists, stream, &cp.lists, 0);
  if (rc) return rc;
  rc = build_tile_lists(cp.plan, b + l.lists4, stream, &cp.lists4, 4);
  if (rc) return rc;
  if (l.has_inverse) {
    rc = build_inverse_plan(g, map, wts, b + l.inverse, stream, &cp.inverse);
    if (rc) return rc;
    rc = build_tile_lists(cp.inverse.plan, b + l.inverse_lists, stream, &cp.inverse_lists, 0,
                          kProductCap);
    if (rc) return rc;
  }
  if (l.has_col2im) {
    rc = col2im_lists_build(map, wts, b + l.col2im, g.H, g.W, g.M, g.K, g.P, g.interp, stream);
    if (rc) return rc;
  }
  return SDK_OK;
}

}  // namespace sdk
