// Gather -> MFMA contraction from an LDS window, driven by a tap plan (gfx950, float32 tensors):
//
//   pix[b][n, m] = sum_{c, k} Wm[n, (c, k)] * col[b][(c, k), m] + bias[n]
//   col[b][(c, k), m] = sum_r coefficient(m, k, r) * img[b][c][tap(m, k, r)]
//
// for the tiles of a plan (conv_plan.hpp) whose taps all fall into the tile's image window.
// Those tiles never gather from global memory: per chunk of 32 image channels the window
// (at most kRegionCap elements) is staged in LDS with the channels of one element side by
// side, and the column values are produced straight into MFMA B fragments:
//
//   workgroup  = one 2-D tile of 128 pixels x TN = 32 * NB pixel-side channels x one batch element
//   wave w     = pixels 32w .. 32w+31 of the tile x all TN channels (NB accumulators of 32 x 32)
//   lane l     = pixel j = l % 32, reduction half h = l / 32
//
// v_mfma_f32_32x32x2_f32 step s contracts channels 2s + h, so a lane needs the 16 channels
// {h, h+2, ...} of its pixel; v_mfma_f32_32x32x16_bf16 instruction t contracts channels
// 16t + 8h + 0..7.  The window and the weight tile keep the 32 channels of a chunk in that
// order (position 16h + s, or 16h + 8t + j), so a lane reads its 16 values of one tap, and its
// 16 weights of one row n, as four 16-byte LDS reads.  Per kernel sample and chunk a wave issues
// 16 NB MFMAs, 64 fused multiply-adds, about 16 + 4 NB LDS reads and no global gather; plan rows
// (window index, coefficient) are read from global memory one sample ahead, weights are staged
// through a double-buffered LDS tile, and there is one barrier per sample.
//
// Rows padded by the plan (coefficient 0) are pointed at a zero element behind the window, so
// a non-finite image value never meets a zero coefficient.
#include <hip/hip_runtime.h>

#include "conv_fused.hpp"
#include "conv_plan.hpp"
#include "conv_window.hpp"
#include "sdk_host.hpp"
#include "sdk_mfma.hpp"

namespace sdk {

namespace {

constexpr int kWgThreads = 256;
constexpr int kWE = 36;   // floats per window element / weight row: 32 channels + 4 of skew

// Position of channel c (0..31 inside its chunk) in a window element or weight row.
__host__ __device__ constexpr int chunk_pos(int c, bool bf16) {
  return bf16 ? 16 * ((c >> 3) & 1) + 8 * (c >> 4) + (c & 7) : 16 * (c & 1) + (c >> 1);
}

__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Wp[k][chunk][n][pos] (n padded to CpP, channels to whole chunks, zeros in the padding):
// one (k, chunk, 128-row block) is 16 KB of consecutive memory.
// swapped: the roles of the two channel indices of Wm are exchanged (Wm is [Cg, Cp * K]): the
// contraction over the inverse plan gathers the pixel side and produces the image side.
__global__ __launch_bounds__(kWgThreads) void window_weight_kernel(
    const float* __restrict__ Wm, float* __restrict__ out, int Cp, int Cg, int K, int CpP,
    int chunks, int bf16, int swapped) {
  const size_t total = (size_t)K * chunks * CpP * kCC;
  for (size_t e = (size_t)blockIdx.x * kWgThreads + threadIdx.x; e < total;
       e += (size_t)gridDim.x * kWgThreads) {
    const int pos = (int)(e % kCC);
    const int n = (int)((e / kCC) % CpP);
    const size_t rest = e / ((size_t)kCC * CpP);
    const int chunk = (int)(rest % chunks), k = (int)(rest / chunks);
    // inverse of chunk_pos
    const int hh = pos >> 4, lo = pos & 15;
    const int cl = bf16 ? 16 * (lo >> 3) + 8 * hh + (lo & 7) : 2 * lo + hh;
    const int c = chunk * kCC + cl;
    float v = 0.0f;
    if (n < Cp && c < Cg)
      v = swapped ? Wm[(size_t)c * Cp * K + (size_t)n * K + k]
                  : Wm[(size_t)n * Cg * K + (size_t)c * K + k];
    out[e] = v;
  }
}

// ---------------------------------------------------------------------------
// Inverse plan.  The scatter  img[u] += co * v[m, k]  over all taps (m, k) -> u, regrouped by
// target u, is a gather over the pixel-side tensor: per image pixel u and sample k a list of
// (source pixel m, coefficient) pairs.  The lists are collected with integer atomics
// (inverse_fill_tiled_kernel: at most kInvRows entries per list, *gate counts the taps that
// found theirs full) in tiles of the image grid, then turned into a plan whose windows lie
// in the pixel grid (inverse_plan_kernel), so the same window kernel runs the contraction.
// Lists are sorted by source pixel: the summation order does not depend on the order in
// which the atomics were served.
//   raw_off / raw_co [((tile * K + k) * kInvRows + slot) * 128 + p]   p: tile-local image pixel
//   cnt[u * K + k]                                                    entries of (u, k)
// ---------------------------------------------------------------------------
constexpr int kInvRows = kInversePlanRows;

template <int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kWgThreads) void inverse_fill_tiled_kernel(
    const float* __restrict__ map, const float* __restrict__ wts, int M, int K, int P, int H, int W,
    PixelTiling it, int* __restrict__ cnt, int* __restrict__ raw_off, float* __restrict__ raw_co,
    int* __restrict__ gate) {
  const size_t i = (size_t)blockIdx.x * kWgThreads + threadIdx.x;
  if (i >= (size_t)M * K) return;
  const int m = (int)(i / K), k = (int)(i % K);
  const int q = WEIGHTED ? P : 1;
  PointTaps<float, INTERP> t;
  for (int p = 0; p < q; ++p) {
    const size_t s = i * q + p;
    t.set(map[s * 2], map[s * 2 + 1], H, W);
    const float wt = WEIGHTED ? wts[s] : 1.0f;
#pragma unroll
    for (int jj = 0; jj < PointTaps<float, INTERP>::N; ++jj) {
      const float co = WEIGHTED ? wt * t.w[jj] : t.w[jj];
      if (t.off[jj] >= 0 && co != 0.0f) {
        const int u = t.off[jj], uy = t.ty[jj], ux = t.tx[jj];
        const int slot = atomicAdd(&cnt[(size_t)u * K + k], 1);
        if (slot < kInvRows) {
          const int tile = (uy / it.TY()) * it.tiles_x + (ux >> it.tx_shift);
          const int pl = (uy % it.TY()) * it.TX() + (ux & (it.TX() - 1));
          const size_t e = (((size_t)tile * K + k) * kInvRows + slot) * 128 + pl;
          raw_off[e] = m;
          raw_co[e] = co;
        } else {
          atomicAdd(gate, 1);
        }
      }
    }
  }
}

// One workgroup per image tile; thread = (tile pixel p, parity of the sample).  Writes the
// plan of the tile (conv_plan.hpp; windows in the OH x OW pixel grid, columns modulo OW) and
// sorts the tile's raw lists by source pixel in place.
__global__ __launch_bounds__(kWgThreads) void inverse_plan_kernel(
    const int* __restrict__ cnt, int* __restrict__ raw_off, float* __restrict__ raw_co,
    PixelTiling it, int K, int OH, int OW, int* __restrict__ hdr, int* __restrict__ ns_out,
    int2* __restrict__ taps, const int* __restrict__ gate, int* __restrict__ big_lut) {
  if (*gate != 0) return;
  __shared__ int bb[4];
  __shared__ int ns_l[kPlanKMax];
  __shared__ WindowSet wset;
  const int tid = threadIdx.x, lane = tid & 63;
  const int tile = blockIdx.x;
  const int ty0 = (tile / it.tiles_x) * it.TY(), tx0 = (tile % it.tiles_x) << it.tx_shift;
  const int p = tid & 127, kpar = tid >> 7;
  const int uy = ty0 + (p >> it.tx_shift), ux = tx0 + (p & (it.TX() - 1));
  const bool pix_ok = uy < it.OH && ux < it.OW;
  const int u = uy * it.OW + ux;
  // anchor: the tile's first pixel, scaled to the pixel grid
  const int ay = min((int)((long long)ty0 * OH / it.OH), OH - 1);
  const int ax = min((int)((long long)tx0 * OW / it.OW), OW - 1);
  for (int k = tid; k < K; k += kWgThreads) ns_l[k] = 0;
  if (tid == 0) {
    bb[0] = INT_MAX;
    bb[1] = INT_MIN;
    bb[2] = INT_MAX;
    bb[3] = INT_MIN;
  }
  __syncthreads();

  int dy0 = INT_MAX, dy1 = INT_MIN, dx0 = INT_MAX, dx1 = INT_MIN;
  for (int k = kpar; k < K; k += 2) {
    const int n = pix_ok ? min(cnt[(size_t)u * K + k], kInvRows) : 0;
    int* ro = raw_off + ((size_t)tile * K + k) * kInvRows * 128 + p;
    float* rc = raw_co + ((size_t)tile * K + k) * kInvRows * 128 + p;
    // insertion sort by source pixel (n <= 16)
    int so[kInvRows];
    float sc[kInvRows];
#pragma unroll
    for (int a = 0; a < kInvRows; ++a) {
      so[a] = a < n ? ro[a * 128] : INT_MAX;
      sc[a] = a < n ? rc[a * 128] : 0.0f;
    }
#pragma unroll
    for (int a = 1; a < kInvRows; ++a) {
#pragma unroll
      for (int b = a; b > 0; --b) {
        const bool sw = so[b] < so[b - 1];
        const int o1 = sw ? so[b] : so[b - 1], o2 = sw ? so[b - 1] : so[b];
        const float c1 = sw ? sc[b] : sc[b - 1], c2 = sw ? sc[b - 1] : sc[b];
        so[b - 1] = o1;
        so[b] = o2;
        sc[b - 1] = c1;
        sc[b] = c2;
      }
    }
#pragma unroll
    for (int a = 0; a < kInvRows; ++a) {
      if (a < n) {
        ro[a * 128] = so[a];
        rc[a * 128] = sc[a];
        const int my = so[a] / OW, mx = so[a] - my * OW;
        const int dy = my - ay;
        int dx = mx - ax;
        dx += (dx > OW / 2) ? -OW : ((dx < -(OW / 2)) ? OW : 0);
        dy0 = min(dy0, dy);
        dy1 = max(dy1, dy);
        dx0 = min(dx0, dx);
        dx1 = max(dx1, dx);
      }
    }
    const int nmax = wave_max(n);
    if (lane == 0) atomicMax(&ns_l[k], nmax);
  }
  dy0 = wave_min(dy0);
  dy1 = wave_max(dy1);
  dx0 = wave_min(dx0);
  dx1 = wave_max(dx1);
  if (lane == 0) {
    atomicMin(&bb[0], dy0);
    atomicMax(&bb[1], dy1);
    atomicMin(&bb[2], dx0);
    atomicMax(&bb[3], dx1);
  }
  __syncthreads();   // (also orders the sorted lists written above before they are re-read)
  Region rg = choose_region(bb[0], bb[1], bb[2], bb[3], ay, ax, it.TY(), it.TX(), OW);
  bool whole = bb[0] > bb[1] || (bb[1] - bb[0] + 1) * min(bb[3] - bb[2] + 1, OW) <= kRegionCap;
  int listed = -1;   // >= 0: elements of a listed window
  int big = -1;      // >= 0: elements of the tile's big window
  // A box that fits may still hold far more pixels than the tile has sources (the sources of an
  // up-sampling map on a mesh: 60 of them spread over a few hundred indices): the sorted list
  // of the distinct sources then makes the smaller window, small enough for the product form.
  const bool sparse_box = whole && bb[0] <= bb[1] && rg.RS > kProductCap;
  if (!whole || sparse_box) {
    // the distinct sources of the tile may still fit: try a listed window
    set_clear(wset);
    __syncthreads();
    for (int k = kpar; k < K; k += 2) {
      const int n = pix_ok ? min(cnt[(size_t)u * K + k], kInvRows) : 0;
      const int* ro = raw_off + ((size_t)tile * K + k) * kInvRows * 128 + p;
      for (int a = 0; a < n; ++a) set_insert(wset, ro[a * 128]);
    }
    __syncthreads();
    const int distinct = set_finish(wset);
    if (sparse_box && (distinct < 0 || distinct > kProductCap)) {
      // the box stays
    } else if (distinct >= 0 && distinct <= kRegionCap) {
      listed = distinct;
      rg.ry0 = 0;
      rg.rx0 = 0;
      rg.RH = 1;
      rg.RW = listed;
      rg.RS = listed;
      rg.RSp = listed | 1;
      whole = true;
    } else if (distinct > kRegionCap && big_lut != nullptr) {
      big = distinct;   // too many for a window, few enough for a big one
    }
  }
  int* tile_hdr = hdr + (size_t)tile * kHdrStride;
  if (tid == 0) {
    tile_hdr[0] = rg.ry0;
    tile_hdr[1] = rg.rx0;
    tile_hdr[2] = rg.RH;
    tile_hdr[3] = rg.RW;
    tile_hdr[4] = whole ? 1 : 0;
    int most = 0;
    for (int k = 0; k < K; ++k) most = max(most, ns_l[k]);
    tile_hdr[5] = most;
    tile_hdr[6] = listed >= 0 ? 1 : 0;
    tile_hdr[7] = big >= 0 ? 1 : 0;
  }
  if (listed >= 0) {
    for (int e = tid; e < listed; e += kWgThreads) tile_hdr[kHdrLut + e] = wset.list[e];
  } else {
    write_region_lut(rg, OH, OW, tile_hdr + kHdrLut);
  }
  if (big >= 0) {
    int* bl = big_lut + (size_t)tile * kBigStride;
    if (tid == 0) bl[0] = big;
    for (int e = tid; e < big; e += kWgThreads) {
      const int off = wset.list[e], y = off / OW;
      bl[kBigLut + e] = off;
      bl[kBigLut + kBigCap + e] = rg.encode(y, off - y * OW, OW);
    }
  }
  for (int k = tid; k < K; k += kWgThreads) ns_out[(size_t)tile * K + k] = ns_l[k];
  for (int k = kpar; k < K; k += 2) {
    const int n = pix_ok ? min(cnt[(size_t)u * K + k], kInvRows) : 0;
    const int top = ns_l[k];
    const int* ro = raw_off + ((size_t)tile * K + k) * kInvRows * 128 + p;
    const float* rc = raw_co + ((size_t)tile * K + k) * kInvRows * 128 + p;
    int2* row = taps + ((size_t)tile * K + k) * kInvRows * 128 + p;
    for (int a = 0; a < top; ++a) {
      int2 v = make_int2(0, 0);
      if (a < n) {
        const int mm = ro[a * 128];
        const int my = mm / OW, mx = mm - my * OW;
        const int at = listed >= 0 ? set_rank(wset, listed, mm)
                       : (big >= 0 ? set_rank(wset, big, mm) : rg.encode(my, mx, OW));
        v = make_int2(at, __float_as_int(rc[a * 128]));
      }
      row[(size_t)a * 128] = v;
    }
  }
}

// Splits the plan's tiles by class, each list in ascending tile order.  One workgroup.
//   lists[0 .. tiles)            tiles inside their window (header value 4 != 0), count[0] of them
//   lists[tiles .. 2 tiles)      the others, count[1]
//   lists[2 tiles .. 3 tiles)    those of the others that are big tiles (header value 7), count[2]
//   lists[3 tiles .. 4 tiles)    ... and those that are not, count[3]
//   lists[4 tiles .. 5 tiles)    small_cap > 0: the tiles of the first list whose window has at
//                                most small_cap elements, count[4]
//   lists[5 tiles .. 6 tiles)    ... and the others of the first list, count[5]
//   lists[6 tiles .. 7 tiles)    every tile that is not in the third list, count[6]
// max_rows > 0: a tile with a sample of more rows is neither inside nor big.
__global__ __launch_bounds__(1024) void tile_lists_kernel(const int* __restrict__ hdr, int tiles,
                                                          int* __restrict__ lists,
                                                          int* __restrict__ count, int max_rows,
                                                          int small_cap) {
  constexpr int NC = 7;
  __shared__ int wave_n[NC][16];
  __shared__ int base[NC];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid < NC) base[tid] = 0;
  __syncthreads();
  for (int t0 = 0; t0 < tiles; t0 += 1024) {
    const int t = t0 + tid;
    const bool live = t < tiles;
    const bool rows_ok = live && (max_rows <= 0 || hdr[t * kHdrStride + 5] <= max_rows);
    const bool fit = rows_ok && hdr[t * kHdrStride + 4] != 0;
    const bool small = fit && small_cap > 0 &&
                       hdr[t * kHdrStride + 2] * hdr[t * kHdrStride + 3] <= small_cap;
    bool cls[NC];
    cls[0] = fit;
    cls[1] = live && !fit;
    cls[2] = cls[1] && rows_ok && hdr[t * kHdrStride + 7] != 0;
    cls[3] = cls[1] && !cls[2];
    cls[4] = small;
    cls[5] = fit && !small;
    cls[6] = live && !cls[2];
    unsigned long long mask[NC];
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      mask[c] = __ballot(cls[c]);
      if (lane == 0) wave_n[c][wave] = __popcll(mask[c]);
    }
    __syncthreads();
    const unsigned long long below = (1ull << lane) - 1ull;
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      if (cls[c]) {
        int o = base[c];
        for (int w = 0; w < wave; ++w) o += wave_n[c][w];
        lists[(size_t)c * tiles + o + __popcll(mask[c] & below)] = t;
      }
    }
    __syncthreads();
    if (tid < NC) {
      int a = 0;
      for (int w = 0; w < 16; ++w) a += wave_n[tid][w];
      base[tid] += a;
    }
    __syncthreads();
  }
  if (tid < NC) count[tid] = base[tid];
}


// CAP: elements of the LDS window.  kRegionCap: the tiles of `list` lie inside their window,
// two workgroups share a CU.  kBigCap: `list` holds big tiles, whose window is their list in
// big_lut; it takes most of a CU's LDS and one workgroup runs per CU.
// XR: plan rows beyond the first four that are requested ahead as well (0 or 2).  The lists of
// an inverse plan are as long as targets have sources: at unit scale a third of the samples
// of a weighted bispherical map have six rows somewhere in a tile.
// RBT: plan rows requested and applied together: 4, or 1 for plans whose samples have a single
// row (nearest taps without interpolation weights; three rows of padding would cost three
// quarters of the gather's LDS reads and multiply-adds).
template <int MM, int NB, int CAP, int XR, int RBT = 4>
__global__ __launch_bounds__(kWgThreads, CAP > kRegionCap ? 1 : 2) void window_gemm_kernel(
    const float* __restrict__ img, const int* __restrict__ hdr, const int* __restrict__ ns,
    const int2* __restrict__ taps, const int* __restrict__ list, const int* __restrict__ count,
    const float* __restrict__ Wp, const float* __restrict__ bias, float* __restrict__ pix, int Cg,
    int H, int W, int Cp, int K, int S, int CpP, int chunks, PixelTiling pt, int tiles,
    int n_tiles, const int* __restrict__ gate, const int* __restrict__ big_lut) {
  if (gate != nullptr && *gate != 0) return;   // the plan is not valid: another kernel does the work
  constexpr bool BF16 = MM != kMmF32;
  constexpr bool BIG = CAP > kRegionCap;
  constexpr int TN = 32 * NB;
  __shared__ __align__(16) float region[(CAP + 1) * kWE];
  __shared__ __align__(16) float As[2][TN * kWE];
  __shared__ int src[CAP];
  __shared__ int ns_l[kPlanKMax];   // rows per sample (a scalar load here would sit in the LDS waits)

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int j = lane & 31, h = lane >> 5;
  // Workgroup ids go round-robin over the 8 XCDs (each with its own L2): XCD x takes the
  // list entries [x * per, (x + 1) * per), so neighbouring tiles meet in one L2 and every XCD
  // gets the same share of the list however long it is.
  const int cnt = *count;
  const int per = (cnt + 7) >> 3;
  const int wg = blockIdx.x / n_tiles;
  const int slot = (wg & 7) * per + (wg >> 3);
  if ((wg >> 3) >= per || slot >= cnt) return;
  const int tile = list[slot];
  const int n0 = (blockIdx.x % n_tiles) * TN;
  const int ty0 = (tile / pt.tiles_x) * pt.TY(), tx0 = (tile % pt.tiles_x) << pt.tx_shift;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)blockIdx.y * Cg * HW;

  // this lane's pixel and its plan rows: row r of sample k at rows_p[(k * S + r) * 128]
  const int p_local = 32 * wave + j;
  int RS;
  const int2* rows_p = taps + (size_t)tile * K * S * 128 + p_local;
  if constexpr (BIG) {
    const int* bl = big_lut + (size_t)tile * kBigStride;
    RS = min(bl[0], CAP);
    for (int e = tid; e < RS; e += kWgThreads) src[e] = bl[kBigLut + e];
  } else {
    RS = hdr[tile * kHdrStride + 2] * hdr[tile * kHdrStride + 3];
    load_region_lut(hdr + (size_t)tile * kHdrStride, RS, src);
  }
  if (tid < kWE) region[RS * kWE + tid] = 0.0f;   // the zero element padded rows point at
  for (int k = tid; k < K; k += kWgThreads) ns_l[k] = ns[(size_t)tile * K + k];

  // The accumulators start at the bias of their rows (register v of lane l: row
  // 8 (v / 4) + 4 (l / 32) + v % 4): the reads are issued here, with the window's, and the
  // epilogue is stores alone.  (Read behind each store they serialise: on this part a wait
  // for the load also waits for the store before it, 64 round trips per tile and wave.)
  floatx16 acc[NB];
  if (bias != nullptr) {
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
        const float bv = bias[n < Cp ? n : Cp - 1];
        acc[a][v] = n < Cp ? bv : 0.0f;
      }
  } else {
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][v] = 0.0f;
  }

  // weight tile of (k, chunk): TN rows of 32 values, 16-byte pieces e = tid + 256 i
  constexpr int WPT = TN * kCC / 4 / kWgThreads;   // float4 per thread: 4 (TN = 128), 2 or 1
  static_assert(WPT == 4 || WPT == 2 || WPT == 1, "weight tile of 128, 64 or 32 rows");
  float4 w0, w1, w2, w3;   // (named registers: an array here ends up in scratch memory)
  w0 = w1 = w2 = w3 = make_float4(0.f, 0.f, 0.f, 0.f);
#define SDK_LOAD_WEIGHTS(kv, chunkv)                                              \
  do {                                                                            \
    const float4* srcw = reinterpret_cast<const float4*>(                         \
        Wp + (((size_t)(kv) * chunks + (chunkv)) * CpP + n0) * kCC) + tid;        \
    w0 = srcw[0];                                                                 \
    if constexpr (WPT >= 2) w1 = srcw[kWgThreads];                                \
    if constexpr (WPT == 4) {                                                     \
      w2 = srcw[2 * kWgThreads];                                                  \
      w3 = srcw[3 * kWgThreads];                                                  \
    }                                                                             \
  } while (0)
#define SDK_STORE_WEIGHTS(bufv)                                                   \
  do {                                                                            \
    float* dstw = &As[bufv][(tid >> 3) * kWE + 4 * (tid & 7)];                    \
    *reinterpret_cast<float4*>(dstw) = w0;                                        \
    if constexpr (WPT >= 2) *reinterpret_cast<float4*>(dstw + 32 * kWE) = w1;     \
    if constexpr (WPT == 4) {                                                     \
      *reinterpret_cast<float4*>(dstw + 64 * kWE) = w2;                           \
      *reinterpret_cast<float4*>(dstw + 96 * kWE) = w3;                           \
    }                                                                             \
  } while (0)

  // Plan rows of one sample: the first four are requested a whole sample ahead, without
  // conditions (rows past the sample's count re-read its last slot and are masked when they
  // are used), so that no branch and no wait sits between a request and the MFMAs that cover
  // its latency.  Samples with more than four rows fetch the others when they need them.
  constexpr int RB = RBT;
  int2 rows[RB], rows_next[RB];
  int2 xrows[XR > 0 ? XR : 1], xrows_next[XR > 0 ? XR : 1];
#define SDK_LOAD_ROWS_N(dst, kv, r0v, NR)                                         \
  do {                                                                            \
    _Pragma("unroll") for (int u = 0; u < (NR); ++u)                              \
      dst[u] = rows_p[((size_t)(kv) * S + min((r0v) + u, S - 1)) * 128];          \
  } while (0)
#define SDK_LOAD_ROWS(dst, kv, r0v) SDK_LOAD_ROWS_N(dst, kv, r0v, RB)
  // col[] += the taps of up to four rows (FIRST: col[] = ..., the product of the first row
  // instead of a register clear and a multiply-add)
#define SDK_GATHER_ROWS(src, r0v, FIRST) SDK_GATHER_ROWS_N(src, r0v, FIRST, RB)
#define SDK_GATHER_ROWS_N(src, r0v, FIRST, NR)                                    \
  do {                                                                            \
    int e[RB];                                                                    \
    float co[RB];                                                                 \
    _Pragma("unroll") for (int u = 0; u < (NR); ++u) {                            \
      co[u] = (r0v) + u < n_rows ? __int_as_float(src[u].y) : 0.0f;               \
      e[u] = co[u] != 0.0f ? src[u].x : RS;                                       \
    }                                                                             \
    _Pragma("unroll") for (int u = 0; u < (NR); ++u) {                            \
      const float4* rp = reinterpret_cast<const float4*>(region + e[u] * kWE + 16 * h); \
      const float4 d0 = rp[0], d1 = rp[1], d2 = rp[2], d3 = rp[3];                \
      const float d[16] = {d0.x, d0.y, d0.z, d0.w, d1.x, d1.y, d1.z, d1.w,        \
                           d2.x, d2.y, d2.z, d2.w, d3.x, d3.y, d3.z, d3.w};       \
      _Pragma("unroll") for (int i = 0; i < 16; ++i)                              \
        colv[i] = (FIRST) && u == 0 ? co[u] * d[i] : __builtin_fmaf(co[u], d[i], colv[i]); \
    }                                                                             \
  } while (0)

  int buf = 0;
  SDK_LOAD_WEIGHTS(0, 0);
  int n_rows = ns[(size_t)tile * K];
  SDK_LOAD_ROWS(rows, 0, 0);
  if constexpr (XR > 0) SDK_LOAD_ROWS_N(xrows, 0, RB, XR);
  for (int chunk = 0; chunk < chunks; ++chunk) {
    const int c0 = chunk * kCC;
    __syncthreads();   // every wave is done with the previous chunk's window (and src is built)
    {
      // wave w stages channels 8w .. 8w+7 of every window element; a lane owns elements
      // lane, lane + 64, ... and has all its loads in flight before the first LDS write
      constexpr int ITER = (CAP + 63) / 64;
      const int cw = c0 + 8 * wave;
      const char* cbase = reinterpret_cast<const char*>(img_b + (size_t)min(cw, Cg - 1) * HW);
      const unsigned plane = (unsigned)HW * 4u;
      float v[ITER][8];
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int e = lane + 64 * it;
        const int o = e < RS ? src[e] : -1;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const bool ok = o >= 0 && cw + i < Cg;
          const float d = *reinterpret_cast<const float*>(
              cbase + (ok ? (unsigned)i * plane + (unsigned)o * 4u : 0u));
          v[it][i] = ok ? d : 0.0f;
        }
      }
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int e = lane + 64 * it;
        if (e < RS) {
          float* dst = region + e * kWE;
          if constexpr (BF16) {
            float4* d4 = reinterpret_cast<float4*>(dst + 16 * (wave & 1) + 8 * (wave >> 1));
            d4[0] = make_float4(v[it][0], v[it][1], v[it][2], v[it][3]);
            d4[1] = make_float4(v[it][4], v[it][5], v[it][6], v[it][7]);
          } else {
            *reinterpret_cast<float4*>(dst + 4 * wave) =
                make_float4(v[it][0], v[it][2], v[it][4], v[it][6]);
            *reinterpret_cast<float4*>(dst + 16 + 4 * wave) =
                make_float4(v[it][1], v[it][3], v[it][5], v[it][7]);
          }
        }
      }
    }
    if (chunk == 0) SDK_STORE_WEIGHTS(buf);   // (later chunks: stored behind the previous chunk's last sample)
    __syncthreads();

    for (int k = 0; k < K; ++k) {
      // ---- request the next sample's weights and first rows (after the last sample of the
      // last chunk: the first ones again, unused)
      const bool last_k = k + 1 == K;
      const int kn = last_k ? 0 : k + 1;
      const int chunk_n = last_k ? (chunk + 1 < chunks ? chunk + 1 : 0) : chunk;
      SDK_LOAD_WEIGHTS(kn, chunk_n);
      SDK_LOAD_ROWS(rows_next, kn, 0);
      if constexpr (XR > 0) SDK_LOAD_ROWS_N(xrows_next, kn, RB, XR);
      const int n_rows_next = __builtin_amdgcn_readfirstlane(ns_l[kn]);
      asm volatile("" ::: "memory");   // the requests stay here, ahead of the gather and the MFMAs

      // ---- gather: col[c][pixel j] for this lane's 16 channels of the chunk
      float colv[16];
      SDK_GATHER_ROWS(rows, 0, true);
      if (n_rows > RB) {
        if constexpr (XR > 0) SDK_GATHER_ROWS_N(xrows, RB, false, XR);
        for (int r0 = RB + XR; r0 < n_rows; r0 += RB) {
          int2 more[RB];
          SDK_LOAD_ROWS(more, k, r0);
          SDK_GATHER_ROWS(more, r0, false);
        }
      }
      // ---- contraction
      const float* at = &As[buf][j * kWE + 16 * h];
      if constexpr (MM == kMmF32) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float4 aq[NB];
#pragma unroll
          for (int a = 0; a < NB; ++a)
            aq[a] = *reinterpret_cast<const float4*>(at + a * 32 * kWE + 4 * q);
#pragma unroll
          for (int a = 0; a < NB; ++a) {
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[a].x, colv[4 * q + 0], acc[a], 0, 0, 0);
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[a].y, colv[4 * q + 1], acc[a], 0, 0, 0);
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[a].z, colv[4 * q + 2], acc[a], 0, 0, 0);
            acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(aq[a].w, colv[4 * q + 3], acc[a], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const float fb[8] = {colv[8 * t + 0], colv[8 * t + 1], colv[8 * t + 2], colv[8 * t + 3],
                               colv[8 * t + 4], colv[8 * t + 5], colv[8 * t + 6], colv[8 * t + 7]};
          Bf16Frag b16;
          Bf16Split b3;
          if constexpr (MM == kMmSplit) b3 = split_bf16x8(fb);
          else b16 = pack_bf16x8(fb);
#pragma unroll
          for (int a = 0; a < NB; ++a) {
            const float4 lo = *reinterpret_cast<const float4*>(at + a * 32 * kWE + 8 * t);
            const float4 hi = *reinterpret_cast<const float4*>(at + a * 32 * kWE + 8 * t + 4);
            const float fa[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            if constexpr (MM == kMmSplit) acc[a] = mfma_split(split_bf16x8(fa), b3, acc[a]);
            else acc[a] = mfma_bf16(pack_bf16x8(fa), b16, acc[a]);
          }
        }
      }
      SDK_STORE_WEIGHTS(buf ^ 1);
      lds_barrier();
      buf ^= 1;
      n_rows = n_rows_next;
#pragma unroll
      for (int u = 0; u < RB; ++u) rows[u] = rows_next[u];
      if constexpr (XR > 0) {
#pragma unroll
        for (int u = 0; u < XR; ++u) xrows[u] = xrows_next[u];
      }
    }
  }
  // ---- epilogue: store.  Accumulator register v of lane l: row 8*(v/4) + 4*h + v%4
  // (pixel-side channel), column j (pixel).
  const int oy = ty0 + (p_local >> pt.tx_shift), ox = tx0 + (p_local & (pt.TX() - 1));
  if (oy < pt.OH && ox < pt.OW) {
    float* out = pix + (size_t)blockIdx.y * Cp * M + (size_t)oy * pt.OW + ox;
#pragma unroll
    for (int a = 0; a < NB; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = n0 + 32 * a + 8 * (v >> 2) + 4 * h + (v & 3);
        if (n < Cp) out[(size_t)n * M] = acc[a][v];
      }
  }
#undef SDK_LOAD_WEIGHTS
#undef SDK_STORE_WEIGHTS
#undef SDK_LOAD_ROWS
#undef SDK_LOAD_ROWS_N
#undef SDK_GATHER_ROWS
#undef SDK_GATHER_ROWS_N
}


// ---------------------------------------------------------------------------
// Product form.  In the inverse direction of an up-sampling or strided map the image is finer
// than the pixel grid: the 128 image pixels of a tile draw on few source pixels (a quarter as
// many at stride 2, plus a border), and gathering first means contracting all 128 of them
// against every sample.  Here, per sample k,
//
//   T_k[s][n] = sum_c W[n, (c, k)] * src[c][s]          for the tile's source pixels s  (MFMA)
//   out[n][u] += sum_r coefficient(u, k, r) * T_k[source(u, k, r)][n]                   (LDS)
//
// The window of source pixels (at most kProductCap = 64, every channel) stays in LDS for the
// whole tile and feeds the MFMAs as it lies: no operand is built.  T_k goes through LDS, and a
// thread gathers, for its image pixel and 64 of the 128 produced channels, the rows its plan
// rows name (window index, coefficient).
//
//   workgroup = one image tile x 128 produced channels x one batch element
//   MFMA role:   wave w = source pixels 32 (w % 2) .. + 31 x produced channels 64 (w / 2) .. + 63
//   gather role: thread t = image pixel t % 128 of the tile, produced channels 64 (t / 128) .. + 63
//
// CH: 32-channel chunks of the gathered tensor the window holds (2, 4 or 8).
// ---------------------------------------------------------------------------

template <int CH, int NBP>
__global__ __launch_bounds__(kWgThreads, CH <= 4 ? 2 : 1) void window_product_kernel(
    const float* __restrict__ img, const int* __restrict__ hdr, const int* __restrict__ ns,
    const int2* __restrict__ taps, const int* __restrict__ list, const int* __restrict__ count,
    const float* __restrict__ Wp, const float* __restrict__ bias, float* __restrict__ pix, int Cg,
    int H, int W, int Cp, int K, int S, int CpP, int chunks, PixelTiling pt, int n_tiles,
    const int* __restrict__ gate) {
  if (gate != nullptr && *gate != 0) return;
  constexpr int XS = 32 * CH + 4;   // floats per source pixel in the window
  constexpr int kPrT = 64 * NBP + 4;   // floats per row of T: the channels + 4 of skew
  // Two copies of T for the 64-channel form: the products of sample k + 1 are written while
  // other waves still gather sample k, and one barrier per sample is enough.
  constexpr int TB = NBP == 1 ? 2 : 1;
  constexpr int TSZ = (kProductCap + 1) * kPrT;   // (+ a row of zeros)
  __shared__ __align__(16) float X[kProductCap * XS];
  __shared__ __align__(16) float Tl[TB * TSZ];
  __shared__ int src[kProductCap];
  __shared__ int ns_l[kPlanKMax];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int j = lane & 31, h = lane >> 5;
  const int cnt = *count;
  const int per = (cnt + 7) >> 3;
  const int wg = blockIdx.x / n_tiles;
  const int slot = (wg & 7) * per + (wg >> 3);
  if ((wg >> 3) >= per || slot >= cnt) return;
  const int tile = list[slot];
  constexpr int TN = 64 * NBP, HN = TN / 2;   // channels per workgroup, per wave pair / thread
  const int n0 = (blockIdx.x % n_tiles) * TN;
  const int ty0 = (tile / pt.tiles_x) * pt.TY(), tx0 = (tile % pt.tiles_x) << pt.tx_shift;
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + (size_t)blockIdx.y * Cg * HW;

  const int RS = min(hdr[tile * kHdrStride + 2] * hdr[tile * kHdrStride + 3], kProductCap);
  load_region_lut(hdr + (size_t)tile * kHdrStride, RS, src);
  for (int k = tid; k < K; k += kWgThreads) ns_l[k] = ns[(size_t)tile * K + k];
  for (int i = tid; i < TB * kPrT; i += kWgThreads)
    Tl[(i / kPrT) * TSZ + kProductCap * kPrT + i % kPrT] = 0.0f;
  __syncthreads();
  {
    // window: lane = source pixel, wave w = channels 8w .. 8w+7 of every chunk; the channels of
    // a chunk lie in the order the MFMA steps take them (as in window_gemm_kernel)
    const int o = lane < RS ? src[lane] : -1;
    for (int chunk = 0; chunk < chunks; ++chunk) {
      const int cw = chunk * kCC + 8 * wave;
      const char* cbase = reinterpret_cast<const char*>(img_b + (size_t)min(cw, Cg - 1) * HW);
      const unsigned plane = (unsigned)HW * 4u;
      float v[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const bool ok = o >= 0 && cw + i < Cg;
        const float d = *reinterpret_cast<const float*>(
            cbase + (ok ? (unsigned)i * plane + (unsigned)o * 4u : 0u));
        v[i] = ok ? d : 0.0f;
      }
      float* dst = X + lane * XS + chunk * kCC;
      *reinterpret_cast<float4*>(dst + 4 * wave) = make_float4(v[0], v[2], v[4], v[6]);
      *reinterpret_cast<float4*>(dst + 16 + 4 * wave) = make_float4(v[1], v[3], v[5], v[7]);
    }
  }

  // gather role
  const int p_local = tid & 127, hh = tid >> 7;
  const int2* rows_p = taps + (size_t)tile * K * S * 128 + p_local;
  float oacc[HN];
#pragma unroll
  for (int i = 0; i < HN; ++i) {
    const int n = n0 + HN * hh + i;
    oacc[i] = (bias != nullptr && n < Cp) ? bias[n] : 0.0f;
  }
  // MFMA role
  const int pb = wave & 1, cb = wave >> 1;
  const float* xrow = X + (32 * pb + j) * XS + 16 * h;
  // weights of (k, chunk), rows n0 + HN cb + 32 a + j, this lane's 16 values: 4 x 16 bytes
  auto weight_ptr = [&](int k, int chunk, int a) {
    return reinterpret_cast<const float4*>(
        Wp + (((size_t)k * chunks + chunk) * CpP + n0 + HN * cb + 32 * a + j) * kCC + 16 * h);
  };
  // Weights come from global memory (the L2) straight into A operands.  Where the registers
  // allow it (WS) all of a sample's weights are requested a whole sample ahead; otherwise one
  // chunk ahead, which at 16 MFMAs per block and chunk does not always cover the read.
  constexpr bool WS = NBP == 1 && CH <= 4;
  constexpr int WC = WS ? CH : 1;
  float4 wa[WC][NBP][4], wn[WC][NBP][4];
#pragma unroll
  for (int c = 0; c < WC; ++c)
#pragma unroll
    for (int a = 0; a < NBP; ++a)
#pragma unroll
      for (int q = 0; q < 4; ++q) wa[c][a][q] = weight_ptr(0, min(c, chunks - 1), a)[q];
  __syncthreads();   // the window is complete

  for (int k = 0; k < K; ++k) {
    const int n_rows = ns_l[k];
    int2 rows[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) rows[u] = rows_p[((size_t)k * S + min(u, S - 1)) * 128];
    floatx16 acc[NBP];
#pragma unroll
    for (int a = 0; a < NBP; ++a)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[a][v] = 0.0f;
#define SDK_PRODUCT_CHUNK(chunkv, wv)                                                        \
  do {                                                                                        \
    const float4* xp = reinterpret_cast<const float4*>(xrow + (chunkv) * kCC);                \
    _Pragma("unroll") for (int q = 0; q < 4; ++q) {                                           \
      const float4 b = xp[q];                                                                 \
      _Pragma("unroll") for (int a = 0; a < NBP; ++a) {                                       \
        acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[a][q].x, b.x, acc[a], 0, 0, 0);      \
        acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[a][q].y, b.y, acc[a], 0, 0, 0);      \
        acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[a][q].z, b.z, acc[a], 0, 0, 0);      \
        acc[a] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[a][q].w, b.w, acc[a], 0, 0, 0);      \
      }                                                                                       \
    }                                                                                         \
  } while (0)
    if constexpr (WS) {
      const int kn = k + 1 < K ? k + 1 : 0;   // (after the last sample: the first again, unused)
#pragma unroll
      for (int c = 0; c < WC; ++c)
#pragma unroll
        for (int a = 0; a < NBP; ++a)
#pragma unroll
          for (int q = 0; q < 4; ++q) wn[c][a][q] = weight_ptr(kn, min(c, chunks - 1), a)[q];
#pragma unroll
      for (int c = 0; c < WC; ++c)
        if (c < chunks) SDK_PRODUCT_CHUNK(c, wa[c]);
#pragma unroll
      for (int c = 0; c < WC; ++c)
#pragma unroll
        for (int a = 0; a < NBP; ++a)
#pragma unroll
          for (int q = 0; q < 4; ++q) wa[c][a][q] = wn[c][a][q];
    } else {
      for (int chunk = 0; chunk < chunks; ++chunk) {
        // the next weights (of the next sample after the last chunk; the first ones again at the end)
        const bool last_c = chunk + 1 == chunks;
        const int kn = last_c ? (k + 1 < K ? k + 1 : 0) : k, cn = last_c ? 0 : chunk + 1;
#pragma unroll
        for (int a = 0; a < NBP; ++a)
#pragma unroll
          for (int q = 0; q < 4; ++q) wn[0][a][q] = weight_ptr(kn, cn, a)[q];
        SDK_PRODUCT_CHUNK(chunk, wa[0]);
#pragma unroll
        for (int a = 0; a < NBP; ++a)
#pragma unroll
          for (int q = 0; q < 4; ++q) wa[0][a][q] = wn[0][a][q];
      }
    }
#undef SDK_PRODUCT_CHUNK
    if (TB == 1 && k > 0) __syncthreads();   // the gather of the sample before is done with T
    float* Tk = Tl + (TB == 2 ? (k & 1) * TSZ : 0);
    // T[s][n]: accumulator register v of lane (j, h): row n = 8 (v / 4) + 4 h + v % 4, column s = j
    {
      float* trow = Tk + (32 * pb + j) * kPrT + HN * cb + 4 * h;
#pragma unroll
      for (int a = 0; a < NBP; ++a)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4)
          *reinterpret_cast<float4*>(trow + 32 * a + 8 * g4) =
              make_float4(acc[a][4 * g4], acc[a][4 * g4 + 1], acc[a][4 * g4 + 2], acc[a][4 * g4 + 3]);
    }
    __syncthreads();
    // gather: rows of this thread's image pixel (a row past the sample's count or of weight 0
    // reads the row of zeros)
    auto add_row = [&](int2 ec) {
      const float co = __int_as_float(ec.y);
      const int e = co != 0.0f ? min(ec.x, kProductCap - 1) : kProductCap;
      const float4* tp = reinterpret_cast<const float4*>(Tk + e * kPrT + HN * hh);
#pragma unroll
      for (int i = 0; i < HN / 4; ++i) {
        const float4 t = tp[i];
        oacc[4 * i + 0] = __builtin_fmaf(co, t.x, oacc[4 * i + 0]);
        oacc[4 * i + 1] = __builtin_fmaf(co, t.y, oacc[4 * i + 1]);
        oacc[4 * i + 2] = __builtin_fmaf(co, t.z, oacc[4 * i + 2]);
        oacc[4 * i + 3] = __builtin_fmaf(co, t.w, oacc[4 * i + 3]);
      }
    };
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (u < n_rows) add_row(rows[u]);
    for (int r = 4; r < n_rows; ++r) add_row(rows_p[((size_t)k * S + r) * 128]);
  }
  // ---- store
  const int oy = ty0 + (p_local >> pt.tx_shift), ox = tx0 + (p_local & (pt.TX() - 1));
  if (oy < pt.OH && ox < pt.OW) {
    float* out = pix + (size_t)blockIdx.y * Cp * M + (size_t)oy * pt.OW + ox;
#pragma unroll
    for (int i = 0; i < HN; ++i) {
      const int n = n0 + HN * hh + i;
      if (n < Cp) out[(size_t)n * M] = oacc[i];
    }
  }
}

}  // namespace


bool window_gemm_supported(const ConvGeom& g) {
  return plan_supported(g) && g.Cp >= 1 && g.B <= 65535 &&
         (int64_t)g.H * g.W <= ((int64_t)1 << 24);
}

size_t window_gemm_weight_bytes(const ConvGeom& g) {
  const size_t CpP = (size_t)(g.Cp + 127) / 128 * 128;
  const size_t chunks = (size_t)(g.Cg + kCC - 1) / kCC;
  return (size_t)g.K * chunks * CpP * kCC * sizeof(float);
}

size_t tile_lists_bytes(const ConvGeom& g) {
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  return ((size_t)7 * pt.tiles_x * pt.tiles_y + 8) * sizeof(int);
}

void load_tile_lists(const Plan& plan, void* workspace, TileLists* out) {
  int* lists = static_cast<int*>(workspace);
  out->inside = lists;
  out->rest = lists + plan.tiles;
  out->big = lists + (size_t)2 * plan.tiles;
  out->rest_small = lists + (size_t)3 * plan.tiles;
  out->product = lists + (size_t)4 * plan.tiles;
  out->inside_large = lists + (size_t)5 * plan.tiles;
  out->not_big = lists + (size_t)6 * plan.tiles;
  out->count = lists + (size_t)7 * plan.tiles;
}

int build_tile_lists(const Plan& plan, void* workspace, hipStream_t stream, TileLists* out,
                     int max_rows, int small_cap) {
  load_tile_lists(plan, workspace, out);
  launch(tile_lists_kernel, dim3(1), dim3(1024), stream, plan.hdr, plan.tiles,
         const_cast<int*>(out->inside), const_cast<int*>(out->count), max_rows, small_cap);
  SDK_LAUNCH_CHECK("tile_lists");
  return SDK_OK;
}

int window_gemm(const ConvGeom& g, int mm, const Plan& plan, const TileLists& tl,
                const float* img, const float* Wm, bool swapped, const float* bias, float* pix,
                float* weights, const int* gate, hipStream_t stream, int which) {
  const int CpP = (g.Cp + 127) / 128 * 128;
  const int chunks = (g.Cg + kCC - 1) / kCC;
  const bool big = which == kListBig;
  if (!big) {
    const size_t total = (size_t)g.K * chunks * CpP * kCC;
    const int blocks = (int)std::min<size_t>((total + kWgThreads - 1) / kWgThreads, 2048);
    launch(window_weight_kernel, dim3(blocks), dim3(kWgThreads), stream, Wm, weights, g.Cp, g.Cg,
           g.K, CpP, chunks, mm != kMmF32 ? 1 : 0, swapped ? 1 : 0);
    SDK_LAUNCH_CHECK("window_weight");
  } else if (big && plan.big_lut == nullptr) {
    return SDK_OK;
  }
  const bool wide = g.Cp > 64, thin = g.Cp <= 32;
  const int TN = wide ? 128 : (thin ? 32 : 64);
  const int n_tiles = (int)ceil_div(g.Cp, TN);
  // list entries are dealt to the XCDs in eighths: whole multiples of 8 workgroups
  const dim3 grid((unsigned)((plan.tiles + 7) / 8 * 8 * n_tiles), (unsigned)g.B);
  const int* list = big ? tl.big : (which == kListInsideLarge ? tl.inside_large : tl.inside);
  const int* count = big ? tl.count + 2 : (which == kListInsideLarge ? tl.count + 5 : tl.count);
  // (an inverse plan is what this function is given with swapped weights)
  // (wide layers only: with fewer MFMAs per sample the two extra requests cost more than the
  // exposed reads they save; configuration 5's up-sampling layer 0.35 -> 0.38 ms)
  const bool more_rows = swapped && plan.S > 4 && wide;
#define WG4(MMv, NBv, CAPv, XRv)                                                               \
  launch(window_gemm_kernel<MMv, NBv, CAPv, XRv>, grid, dim3(kWgThreads), stream, img,         \
         plan.hdr, plan.ns, plan.taps, list, count, (const float*)weights, bias, pix, g.Cg,    \
         g.H, g.W, g.Cp, g.K, plan.S, CpP, chunks, plan.pt, plan.tiles, n_tiles, gate,         \
         plan.big_lut)
#define WG3(MMv, NBv, CAPv)                                                    \
  do {                                                                         \
    if (more_rows) WG4(MMv, NBv, CAPv, 2); else WG4(MMv, NBv, CAPv, 0);        \
  } while (0)
#define WG1R(MMv, NBv)                                                                         \
  launch(window_gemm_kernel<MMv, NBv, kRegionCap, 0, 1>, grid, dim3(kWgThreads), stream, img,  \
         plan.hdr, plan.ns, plan.taps, list, count, (const float*)weights, bias, pix, g.Cg,    \
         g.H, g.W, g.Cp, g.K, plan.S, CpP, chunks, plan.pt, plan.tiles, n_tiles, gate,         \
         plan.big_lut)
#define WG2(MMv, NBv)                                                 \
  do {                                                                \
    if (big) WG3(MMv, NBv, kBigCap);                                  \
    else if (plan.S == 1) WG1R(MMv, NBv);                             \
    else WG3(MMv, NBv, kRegionCap);                                   \
  } while (0)
#define WG1(MMv)                                                            \
  do {                                                                      \
    if (wide) WG2(MMv, 4); else if (thin) WG2(MMv, 1); else WG2(MMv, 2);    \
  } while (0)
  if (mm == kMmBf16) WG1(kMmBf16);
  else if (mm == kMmSplit) WG1(kMmSplit);
  else WG1(kMmF32);
#undef WG1
#undef WG1R
#undef WG2
#undef WG3
#undef WG4
  SDK_LAUNCH_CHECK(big ? "window_gemm(big)" : "window_gemm");
  return SDK_OK;
}

bool window_product_supported(const ConvGeom& g, int mm) {
  return mm == kMmF32 && window_gemm_supported(g) && g.Cg <= 256;
}

int window_product(const ConvGeom& g, const Plan& plan, const TileLists& tl, const float* img,
                   const float* bias, float* pix, const float* weights, const int* gate,
                   hipStream_t stream) {
  const int CpP = (g.Cp + 127) / 128 * 128;
  const int chunks = (g.Cg + kCC - 1) / kCC;
  const bool wide = g.Cp > 64;
  const int n_tiles = (int)ceil_div(g.Cp, wide ? 128 : 64);
  const dim3 grid((unsigned)((plan.tiles + 7) / 8 * 8 * n_tiles), (unsigned)g.B);
#define WP2(CHv, NBPv)                                                                        \
  launch(window_product_kernel<CHv, NBPv>, grid, dim3(kWgThreads), stream, img, plan.hdr,     \
         plan.ns, plan.taps, tl.product, tl.count + 4, weights, bias, pix, g.Cg, g.H, g.W,    \
         g.Cp, g.K, plan.S, CpP, chunks, plan.pt, n_tiles, gate)
#define WP(CHv)                                     \
  do {                                              \
    if (wide) WP2(CHv, 2); else WP2(CHv, 1);        \
  } while (0)
  if (chunks <= 2) WP(2); else if (chunks <= 4) WP(4); else WP(8);
#undef WP
#undef WP2
  SDK_LAUNCH_CHECK("window_product");
  return SDK_OK;
}

namespace {
struct InverseOffsets {
  size_t gate, cnt, raw_co, raw_off, hdr, ns, taps, big_lut, total;
};
InverseOffsets inverse_offsets(const ConvGeom& g) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const PixelTiling it = plan_tiling(g.H, g.W);
  const size_t tiles = (size_t)it.tiles_x * it.tiles_y;
  const size_t rows = tiles * g.K * kInvRows * 128;
  InverseOffsets o;
  o.gate = 0;
  o.cnt = 256;
  o.raw_co = o.cnt + up((size_t)g.H * g.W * g.K * sizeof(int));   // gate, cnt, raw_co: cleared together
  o.raw_off = o.raw_co + up(rows * sizeof(float));
  o.hdr = o.raw_off + up(rows * sizeof(int));
  o.ns = o.hdr + up(tiles * kHdrStride * sizeof(int));
  o.taps = o.ns + up(tiles * g.K * sizeof(int));
  o.big_lut = o.taps + up(rows * sizeof(int2));
  o.total = o.big_lut + up(tiles * kBigStride * sizeof(int));
  return o;
}
}  // namespace

size_t inverse_plan_bytes(const ConvGeom& g) { return inverse_offsets(g).total; }

void load_inverse_plan(const ConvGeom& g, void* workspace, InversePlan* out) {
  const InverseOffsets o = inverse_offsets(g);
  const PixelTiling it = plan_tiling(g.H, g.W);
  char* ws = static_cast<char*>(workspace);
  out->plan.pt = it;
  out->plan.tiles = it.tiles_x * it.tiles_y;
  out->plan.S = kInvRows;
  out->plan.hdr = reinterpret_cast<int*>(ws + o.hdr);
  out->plan.ns = reinterpret_cast<int*>(ws + o.ns);
  out->plan.taps = reinterpret_cast<int2*>(ws + o.taps);
  out->plan.big_lut = reinterpret_cast<int*>(ws + o.big_lut);
  out->gate = reinterpret_cast<int*>(ws + o.gate);
  out->raw_off = reinterpret_cast<int*>(ws + o.raw_off);
  out->raw_co = reinterpret_cast<float*>(ws + o.raw_co);
}

int build_inverse_plan(const ConvGeom& g, const float* map, const float* wts, void* workspace,
                       hipStream_t stream, InversePlan* out) {
  load_inverse_plan(g, workspace, out);
  const InverseOffsets o = inverse_offsets(g);
  char* ws = static_cast<char*>(workspace);
  int* cnt = reinterpret_cast<int*>(ws + o.cnt);
  int* raw_off = const_cast<int*>(out->raw_off);
  float* raw_co = const_cast<float*>(out->raw_co);
  int rc = zero_fill(ws, o.raw_off, stream);
  if (rc) return rc;
  const int64_t total = (int64_t)g.M * g.K;
  if (ceil_div(total, kWgThreads) >= ((int64_t)1 << 31))
    return fail(SDK_ERR_UNSUPPORTED, "inverse plan: too many samples");
  SDK_DISPATCH_INTERP(g.interp, g.P,
                      (launch(inverse_fill_tiled_kernel<INTERP, WEIGHTED>,
                              dim3((unsigned)ceil_div(total, kWgThreads)), dim3(kWgThreads), stream,
                              map, wts, g.M, g.K, g.P, g.H, g.W, out->plan.pt, cnt, raw_off, raw_co,
                              out->gate)));
  SDK_LAUNCH_CHECK("inverse_fill");
  launch(inverse_plan_kernel, dim3((unsigned)out->plan.tiles), dim3(kWgThreads), stream,
         (const int*)cnt, raw_off, raw_co, out->plan.pt, g.K, g.M / g.OW, g.OW,
         const_cast<int*>(out->plan.hdr), const_cast<int*>(out->plan.ns),
         const_cast<int2*>(out->plan.taps), (const int*)out->gate,
         const_cast<int*>(out->plan.big_lut));
  SDK_LAUNCH_CHECK("inverse_plan");
  return SDK_OK;
}

}  // namespace sdk
