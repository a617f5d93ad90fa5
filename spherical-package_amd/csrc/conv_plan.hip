// Tap plan construction and the plan-driven weight-gradient kernel (gfx950,
// float32 tensors).  Layout of a plan: conv_plan.hpp.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "conv_plan.hpp"
#include "sdk_host.hpp"
#include "sdk_mfma.hpp"

namespace sdk {

constexpr int kPlThreads = 256;

// ---------------------------------------------------------------------------
// Plan construction: one workgroup per tile.  Thread = (pixel of the tile,
// parity of the kernel sample).  Pass 1 finds the bounding box of all active
// taps and the per-sample row counts, pass 2 writes the encoded rows.  When the
// tile's part of the map (128 pixels x K samples x points, 12 bytes each with
// the point weights) fits kPlanStage bytes it is first copied to LDS with
// coalesced reads; both passes then read LDS instead of striding through HBM.
// ---------------------------------------------------------------------------
constexpr int kPlanStage = 56 * 1024;

template <int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kPlThreads) void plan_kernel(
    const float* __restrict__ map, const float* __restrict__ wts, PixelTiling pt, int K, int P,
    int H, int W, int S, int* __restrict__ hdr, int* __restrict__ ns_out,
    int2* __restrict__ taps, const int* __restrict__ gate, int* __restrict__ big_lut) {
  if (gate != nullptr && *gate == 0) return;
  __shared__ int bb[4];
  __shared__ int ns_l[kPlanKMax];
  __shared__ __align__(8) float stage[kPlanStage / sizeof(float)];
  __shared__ WindowSet wset;
  const int tid = threadIdx.x, lane = tid & 63;
  const int tile = blockIdx.x;
  const int ty0 = (tile / pt.tiles_x) * pt.TY(), tx0 = (tile % pt.tiles_x) << pt.tx_shift;
  const int p = tid & 127, kpar = tid >> 7;
  const int oy = ty0 + (p >> pt.tx_shift), ox = tx0 + (p & (pt.TX() - 1));
  const bool pix_ok = oy < pt.OH && ox < pt.OW;
  const int q = WEIGHTED ? P : 1;
  constexpr int NT = Taps2D<INTERP>::N;

  // anchor: centre-ish sample of the tile's first pixel (same value in every thread)
  const size_t s0 = (((size_t)ty0 * pt.OW + tx0) * K + K / 2) * q;
  const int ax = wrap_index(to_int_clamped(round_t(map[s0 * 2])), W);
  const int ay = min(max(to_int_clamped(round_t(map[s0 * 2 + 1])), 0), H - 1);

  // ---- stage the tile's coordinates (and point weights): per tile pixel K*q (x, y) pairs
  const int per_pix = K * q;   // samples x points of one pixel
  const bool staged = (size_t)128 * per_pix * (WEIGHTED ? 12 : 8) <= (size_t)kPlanStage;
  float* st_xy = stage;                      // [128][per_pix][2]
  float* st_w = stage + 128 * per_pix * 2;   // [128][per_pix]
  if (staged) {
    const int run = per_pix * 2;   // floats per pixel
    for (int i = tid; i < 128 * run; i += kPlThreads) {
      const int pl = i / run, o = i - pl * run;
      const int py = ty0 + (pl >> pt.tx_shift), px = tx0 + (pl & (pt.TX() - 1));
      st_xy[i] = (py < pt.OH && px < pt.OW) ? map[((size_t)py * pt.OW + px) * run + o] : 0.0f;
    }
    if constexpr (WEIGHTED) {
      for (int i = tid; i < 128 * per_pix; i += kPlThreads) {
        const int pl = i / per_pix, o = i - pl * per_pix;
        const int py = ty0 + (pl >> pt.tx_shift), px = tx0 + (pl & (pt.TX() - 1));
        st_w[i] = (py < pt.OH && px < pt.OW) ? wts[((size_t)py * pt.OW + px) * per_pix + o] : 0.0f;
      }
    }
  }
  // sample point (x, y, weight) of this thread's pixel
  auto point = [&](int k, int pp, float& x, float& y, float& w) {
    if (staged) {
      const int o = p * per_pix + k * q + pp;
      x = st_xy[2 * o];
      y = st_xy[2 * o + 1];
      w = WEIGHTED ? st_w[o] : 1.0f;
    } else {
      const size_t sidx = (((size_t)oy * pt.OW + ox) * K + k) * q + pp;
      x = map[sidx * 2];
      y = map[sidx * 2 + 1];
      w = WEIGHTED ? wts[sidx] : 1.0f;
    }
  };

  for (int k = tid; k < K; k += kPlThreads) ns_l[k] = 0;
  if (tid == 0) {
    bb[0] = INT_MAX;
    bb[1] = INT_MIN;
    bb[2] = INT_MAX;
    bb[3] = INT_MIN;
  }
  __syncthreads();

  Taps2D<INTERP> t;
  int dy0 = INT_MAX, dy1 = INT_MIN, dx0 = INT_MAX, dx1 = INT_MIN;
  for (int k = kpar; k < K; k += 2) {
    int cnt = 0;
    if (pix_ok) {
      for (int pp = 0; pp < q; ++pp) {
        float sx, sy, sw;
        point(k, pp, sx, sy, sw);
        t.set(sx, sy, H, W, sw);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          if (t.w[i] != 0.0f) {
            const int dy = t.y[i] - ay;
            int dx = t.x[i] - ax;
            dx += (dx > W / 2) ? -W : ((dx < -(W / 2)) ? W : 0);
            dy0 = min(dy0, dy);
            dy1 = max(dy1, dy);
            dx0 = min(dx0, dx);
            dx1 = max(dx1, dx);
            ++cnt;
          }
        }
      }
    }
    cnt = wave_max(cnt);
    if (lane == 0) atomicMax(&ns_l[k], cnt);
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
  __syncthreads();
  Region rg = choose_region(bb[0], bb[1], bb[2], bb[3], ay, ax, pt.TY(), pt.TX(), W);
  // the window is the whole bounding box of the taps unless that exceeded the capacity
  bool whole = bb[0] > bb[1] || (bb[1] - bb[0] + 1) * min(bb[3] - bb[2] + 1, W) <= kRegionCap;
  int listed = -1;   // >= 0: elements of a listed window
  int big = -1;      // >= 0: elements of the tile's big window
  if (!whole) {
    // the distinct elements the tile touches may still fit: try a listed window
    set_clear(wset);
    __syncthreads();
    if (pix_ok) {
      for (int k = kpar; k < K; k += 2) {
        for (int pp = 0; pp < q; ++pp) {
          float sx, sy, sw;
          point(k, pp, sx, sy, sw);
          t.set(sx, sy, H, W, sw);
#pragma unroll
          for (int i = 0; i < NT; ++i)
            if (t.w[i] != 0.0f) set_insert(wset, t.y[i] * W + t.x[i]);
        }
      }
    }
    __syncthreads();
    const int distinct = set_finish(wset);
    if (distinct >= 0 && distinct <= kRegionCap) {
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
    tile_hdr[5] = most;   // the longest row list of the tile's samples
    tile_hdr[6] = listed >= 0 ? 1 : 0;
    tile_hdr[7] = big >= 0 ? 1 : 0;
  }
  if (listed >= 0) {
    for (int e = tid; e < listed; e += kPlThreads) tile_hdr[kHdrLut + e] = wset.list[e];
  } else {
    write_region_lut(rg, H, W, tile_hdr + kHdrLut);
  }
  if (big >= 0) {
    int* bl = big_lut + (size_t)tile * kBigStride;
    if (tid == 0) bl[0] = big;
    for (int e = tid; e < big; e += kPlThreads) {
      const int off = wset.list[e], y = off / W;
      bl[kBigLut + e] = off;
      bl[kBigLut + kBigCap + e] = rg.encode(y, off - y * W, W);
    }
  }
  for (int k = tid; k < K; k += kPlThreads) ns_out[(size_t)tile * K + k] = ns_l[k];

  for (int k = kpar; k < K; k += 2) {
    const int n = ns_l[k];
    int2* row = taps + ((size_t)tile * K + k) * S * 128 + p;
    int cnt = 0;
    if (pix_ok) {
      for (int pp = 0; pp < q; ++pp) {
        float sx, sy, sw;
        point(k, pp, sx, sy, sw);
        t.set(sx, sy, H, W, sw);
#pragma unroll
        for (int i = 0; i < NT; ++i) {
          if (t.w[i] != 0.0f) {
            const int off = t.y[i] * W + t.x[i];
            const int at = listed >= 0 ? set_rank(wset, listed, off)
                           : (big >= 0 ? set_rank(wset, big, off) : rg.encode(t.y[i], t.x[i], W));
            row[(size_t)cnt * 128] = make_int2(at, __float_as_int(t.w[i]));
            ++cnt;
          }
        }
      }
    }
    for (; cnt < n; ++cnt) row[(size_t)cnt * 128] = make_int2(0, 0);
  }
}

// ---------------------------------------------------------------------------
// planned_wgrad:  gW[n][c][k] += sum_{b, m} pix[b][n][m] * col[b][(c, k)][m]
//
// Workgroup (256 threads, 4 waves): one chunk of 32 image channels c, one tile
// of 128 pixel-side channels n (wave w owns rows 32w .. 32w+31), one block of
// KB kernel samples, one batch element and a run of consecutive pixel tiles.
// One 32 x 32 accumulator per kernel sample stays in registers over the whole
// run and is added to gW once at the end.
//
// Per pixel tile the 32 channels of the tile's image window are staged in LDS
// with coalesced loads.  The tile is processed in two halves of 64 pixels.  Per
// half all global reads are issued together: each lane's A fragments (pix values
// of its row n for the 64 pixels) and the half's plan rows, which go to LDS.
// Then, per kernel sample, every lane gathers the column values of one pixel and
// 8 channels from the LDS window (plan row -> ds_read + fma), the 32 x 64 column
// tile is exchanged through LDS and each wave multiplies it with its A
// fragments.  No global read sits between two samples.
//
// Contraction order inside a half (m = pixel 0..63 of the half), fp32
// v_mfma_f32_32x32x2_f32: step 4g+i of lane half h contracts m = 8g + 4h + i, so
// a lane reads its A values and its column values as 16-byte vectors.  bf16
// v_mfma_f32_32x32x16_bf16: instruction t contracts m = 16t + 8h + 0..7.
// ---------------------------------------------------------------------------
constexpr int kColLd = 68;            // column tile row stride (floats): 16-byte rows, 4-bank skew
constexpr int kRegE = 36;             // window element stride (floats): 32 channels + 4 of skew
constexpr int kRowCap = 36;           // plan rows of one half held in LDS at a time
constexpr int kSplitLd = 72;          // row stride (bf16 elements) of the split column tiles: 16-byte rows

// Window layout: region[e * kRegE + c], channels fastest.  A lane reads or writes the 8
// channels of its group for one element as two 16-byte accesses; 8 lanes on consecutive
// elements are 144 bytes apart and cover all 32 banks once.

// NW: 32-row blocks of pixel-side channels per workgroup (4, 2 or 1).  With NW < 4 the waves
// also split the 64 pixels of a half tile (4 / NW ways), so narrow layers waste no MFMAs on
// padding; waves that share rows add their partial sums to gW independently.
// Workgroup barrier that orders LDS traffic only: global loads issued before it may still be
// in flight afterwards (__syncthreads() would wait for them too).
__device__ __forceinline__ void lds_only_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// REST: the launch covers a list of tiles most of whose taps lie outside their window (polar
// rows of a spherical map).  All rows of a sample (up to four) are then requested from the
// image together, one sample ahead, whatever the lanes' taps say, so that one memory latency
// per run of samples is exposed instead of one per pair of rows.
template <int KB, int MM, int NW, bool REST>
__global__ __launch_bounds__(kPlThreads, 2) void planned_wgrad_kernel(
    const float* __restrict__ pix, const float* __restrict__ img, const int* __restrict__ hdr,
    const int* __restrict__ ns, const int2* __restrict__ taps, float* __restrict__ gW,
    float* __restrict__ partial, int Cg, int H, int W, int Cp, int K, int S, PixelTiling pt,
    int tiles, int groups, int batches, int c_chunks, int n_tiles, int kblocks, int vec4,
    const int* __restrict__ tile_list, const int* __restrict__ tile_count,
    const int* __restrict__ big_lut) {
  constexpr bool BF16 = MM != kMmF32;     // operands enter the matrix unit as bf16 fragments
  constexpr bool SPLIT = MM == kMmSplit;  // ... three per operand, whose sum is the float
  __shared__ __align__(16) float region[kRegionCap * kRegE];
  __shared__ __align__(16) float colT[2][kCC * kColLd];
  __shared__ __align__(16) int2 prow[kRowCap * 64];
  __shared__ int src[kRegionCap];
  __shared__ int ns_l[KB];

  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  // 1-D grid; workgroup ids go round-robin over the 8 XCDs.  All workgroups of one
  // tile run (every batch element, channel chunk and sample block) read the same
  // plan rows, and those of one batch element the same pix tiles; they are given
  // consecutive slots of one XCD, so they meet in its L2.
  const int kinds = c_chunks * n_tiles * kblocks * batches;
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int kind = slot % kinds, group = (slot / kinds) * 8 + xcd;
  if (group >= groups) return;
  const int kb = kind % kblocks, nt = (kind / kblocks) % n_tiles;
  const int cc = (kind / (kblocks * n_tiles)) % c_chunks;
  const int batch = kind / (kblocks * n_tiles * c_chunks);
  const int k0 = kb * KB, kcount = min(KB, K - k0);
  const int c0 = cc * kCC, n0 = nt * (32 * NW);
  const int M = pt.OH * pt.OW;
  const size_t HW = (size_t)H * W;
  const float* img_b = img + ((size_t)batch * Cg) * HW;
  const float* pix_b = pix + ((size_t)batch * Cp) * M;

  // roles: gather (pixel px16 of the wave's 16, channel group cg), MFMA (row/column nl, half h)
  const int px16 = lane & 15, cg = lane >> 4;
  const int m_local = wave * 16 + px16;
  const int nl = lane & 31, h = lane >> 5;
  constexpr int PSPLIT = 4 / NW;         // waves sharing a row block split the pixels
  constexpr int PXW = 64 / PSPLIT;       // pixels of a half tile per wave
  const int nbw = wave % NW;             // this wave's row block
  const int poff = (wave / NW) * PXW;    // ... and its first pixel inside a half tile
  const int n_row = n0 + 32 * nbw + nl;
  const bool n_ok = n_row < Cp;
  const float* pix_row = pix_b + (size_t)(n_ok ? n_row : 0) * M;

  floatx16 acc[KB];
#pragma unroll
  for (int i = 0; i < KB; ++i)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

  // REST: byte offset of this lane's channel 8 cg + j inside the chunk's planes.  Channels past
  // Cg repeat the last one: their columns of the product are dropped at the end.
  unsigned ch_off[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
    ch_off[j] = REST ? (unsigned)min(8 * cg + j, Cg - 1 - c0) * ((unsigned)HW * 4u) : 0u;

  // Tiles are dealt round-robin to the tile runs: costly tiles (taps outside the window,
  // e.g. polar rows of a spherical map) are spread over all workgroups.
  int buf = 0;
  // all tiles, or the listed ones (tile_list[i], i < *tile_count)
  const int n_listed = tile_list != nullptr ? *tile_count : tiles;
  if (n_listed == 0) return;   // (the summing kernel sees the same count and adds nothing)
  for (int ti = group; ti < n_listed; ti += groups) {
    const int tile = tile_list != nullptr ? tile_list[ti] : ti;
    const int ty0 = (tile / pt.tiles_x) * pt.TY(), tx0 = (tile % pt.tiles_x) << pt.tx_shift;
    // pixel index (inside the image of the pixel side) of tile-local pixel p, or -1
    auto pixel_index = [&](int p) -> int {
      const int oy = ty0 + (p >> pt.tx_shift), ox = tx0 + (p & (pt.TX() - 1));
      return (oy < pt.OH && ox < pt.OW) ? oy * pt.OW + ox : -1;
    };
    Region rg;
    rg.ry0 = hdr[tile * kHdrStride + 0];
    rg.rx0 = hdr[tile * kHdrStride + 1];
    rg.RH = hdr[tile * kHdrStride + 2];
    rg.RW = hdr[tile * kHdrStride + 3];
    rg.RS = rg.RH * rg.RW;
    rg.RSp = rg.RS;
    // plan rows of this tile and sample block: uniform base, 32-bit lane offsets
    const char* tile_taps = reinterpret_cast<const char*>(taps + ((size_t)tile * K + k0) * S * 128);
    // a big tile is taken like any other tile outside its window: its rows name ranks
    const bool big_tile = big_lut != nullptr && hdr[tile * kHdrStride + 7] != 0;
    const int* big_l = big_lut + (big_tile ? (size_t)tile * kBigStride : 0);

    __syncthreads();  // every wave is done with the previous tile's window, rows and column tiles
    if (tid < kcount) ns_l[tid] = ns[(size_t)tile * K + k0 + tid];
    load_region_lut(hdr + (size_t)tile * kHdrStride, rg.RS, src);
    __syncthreads();
    {
      // wave w stages channels 8w .. 8w+7; a lane owns window elements lane, lane+64, ...
      // (at most 5 of them) and has all its loads in flight before the first LDS write
      constexpr int PER_WAVE = kCC / 4, ITER = (kRegionCap + 63) / 64;
      const char* cbase = reinterpret_cast<const char*>(
          img_b + (size_t)min(c0 + wave * PER_WAVE, Cg - 1) * HW);
      const unsigned plane = (unsigned)HW * 4u;
      float v[ITER][PER_WAVE];
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int e = lane + 64 * it;
        const int o = e < rg.RS ? src[e] : -1;
#pragma unroll
        for (int j = 0; j < PER_WAVE; ++j) {
          const bool ok = o >= 0 && c0 + wave * PER_WAVE + j < Cg;
          const float d = *reinterpret_cast<const float*>(
              cbase + (ok ? (unsigned)j * plane + (unsigned)o * 4u : 0u));
          v[it][j] = ok ? d : 0.0f;
        }
      }
#pragma unroll
      for (int it = 0; it < ITER; ++it) {
        const int e = lane + 64 * it;
        if (e < rg.RS) {
          float4* dst = reinterpret_cast<float4*>(region + e * kRegE + wave * PER_WAVE);
          dst[0] = make_float4(v[it][0], v[it][1], v[it][2], v[it][3]);
          dst[1] = make_float4(v[it][4], v[it][5], v[it][6], v[it][7]);
        }
      }
    }
    // (the window becomes visible with the barrier that follows the first row staging)

#pragma unroll 1
    for (int half = 0; half < 2; ++half) {
      // ---- A fragments of this lane's row n for the 64 pixels of the half
      float afrag[BF16 ? 1 : PXW / 2];
      Bf16Frag afrag16[(BF16 && !SPLIT) ? PXW / 16 : 1];
      Bf16Split afrag3[SPLIT ? PXW / 16 : 1];
      {
        constexpr int GROUPS = BF16 ? PXW / 16 : PXW / 8;   // groups of pixels per lane half ...
        constexpr int RUN = BF16 ? 8 : 4;                   // ... of which this lane holds RUN
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
          const int p0 = half * 64 + poff + (BF16 ? 16 * g + 8 * h : 8 * g + 4 * h);
          float f[RUN];
          if (vec4) {
            const int m0 = pixel_index(p0);
#pragma unroll
            for (int u = 0; u < RUN / 4; ++u) {
              float4 x = make_float4(0.f, 0.f, 0.f, 0.f);
              if (n_ok && m0 >= 0) x = *reinterpret_cast<const float4*>(pix_row + m0 + 4 * u);
              f[4 * u + 0] = x.x;
              f[4 * u + 1] = x.y;
              f[4 * u + 2] = x.z;
              f[4 * u + 3] = x.w;
            }
          } else {
#pragma unroll
            for (int u = 0; u < RUN; ++u) {
              const int mi = pixel_index(p0 + u);
              f[u] = (n_ok && mi >= 0) ? pix_row[mi] : 0.0f;
            }
          }
          if constexpr (SPLIT) {
            afrag3[g] = split_bf16x8(reinterpret_cast<const float(&)[8]>(f));
          } else if constexpr (BF16) {
            afrag16[g] = pack_bf16x8(reinterpret_cast<const float(&)[8]>(f));
          } else {
#pragma unroll
            for (int u = 0; u < 4; ++u) afrag[4 * g + u] = f[u];
          }
        }
      }

      // Samples are taken in runs whose plan rows fit the LDS row buffer.
      int kk_beg = 0;
      while (kk_beg < kcount) {
        int kk_end = kk_beg, rows = 0;
        while (kk_end < kcount && rows + ns_l[kk_end] <= kRowCap) rows += ns_l[kk_end++];
        // (ns <= S <= kRowCap is a launch condition, so every run holds at least one sample)
        // ---- stage the rows of samples kk_beg .. kk_end-1 for the 64 pixels of the half
        {
          int kk = kk_beg, r0 = 0;   // row r of the run belongs to sample kk, its row r - r0
          for (int i = tid; i < rows * 64; i += kPlThreads) {
            const int r = i >> 6, p = i & 63;
            while (r - r0 >= ns_l[kk]) r0 += ns_l[kk++];
            const char* row = tile_taps + (size_t)(kk * S + (r - r0)) * (128 * sizeof(int2));
            int2 ec = *reinterpret_cast<const int2*>(row + (unsigned)(half * 64 + p) * (unsigned)sizeof(int2));
            if (__int_as_float(ec.y) != 0.0f) ec.x = plan_row_at(ec.x, big_tile, big_l);
            prow[i] = ec;
          }
        }
        __syncthreads();

        int row0 = 0;
        // Image values of the next sample's first row, for lanes whose tap lies outside the
        // window: requested one sample ahead so that they arrive during the MFMAs (maps without
        // locality, e.g. mesh neighbourhoods, have all their taps there).
        // (The variants with nine accumulators of 128 rows and fp32 or split A fragments have no
        // registers left for it.)
        constexpr bool PRE = !REST && !(KB == 9 && NW == 4 && MM != kMmBf16);
        float pre[8];
        bool pre_valid = false;
#pragma unroll
        for (int j = 0; j < 8; ++j) pre[j] = 0.0f;
        // REST: image values of rows 0..3 of the sample about to be gathered
        float pre0[8], pre1[8], pre2[8], pre3[8];
        const char* const rest_base =
            reinterpret_cast<const char*>(img_b + (size_t)c0 * HW);
        // requests the image values of row R of the sample whose rows start at BASE (NR rows);
        // lanes whose tap lies in the window (or weighs nothing) read the image's first pixel
#define SDK_REQ_ROW(R, BASE, NR)                                                              \
  if ((R) < (NR)) {                                                                           \
    const int2 ec = prow[((BASE) + (R)) * 64 + m_local];                                      \
    const bool out = ec.x < 0 && __int_as_float(ec.y) != 0.0f;                                \
    const unsigned o0 = out ? (unsigned)(-ec.x - 1) * 4u : 0u;                                \
    _Pragma("unroll") for (int j = 0; j < 8; ++j)                                             \
      pre##R[j] = *reinterpret_cast<const float*>(rest_base + (o0 + ch_off[j]));              \
  }
        // adds row R (window value or requested image value, times the coefficient) to col[];
        // a tap outside the window that weighs nothing takes the window's first element, as
        // the padding rows of a plan do
#define SDK_USE_ROW(R, BASE, NR)                                                              \
  if ((R) < (NR)) {                                                                           \
    const int2 ec = prow[((BASE) + (R)) * 64 + m_local];                                      \
    const int e = ec.x;                                                                       \
    const float co = __int_as_float(ec.y);                                                    \
    const bool out = e < 0 && co != 0.0f;                                                     \
    const float4* rp =                                                                        \
        reinterpret_cast<const float4*>(region + (e >= 0 ? e : 0) * kRegE + 8 * cg);          \
    const float4 l0 = rp[0], l1 = rp[1];                                                      \
    const float dl[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};                     \
    _Pragma("unroll") for (int j = 0; j < 8; ++j)                                             \
      col[j] = __builtin_fmaf(co, out ? pre##R[j] : dl[j], col[j]);                           \
  }
        if constexpr (REST) {
          const int nr = min(__builtin_amdgcn_readfirstlane(ns_l[kk_beg]), 4);
          SDK_REQ_ROW(0, 0, nr) SDK_REQ_ROW(1, 0, nr) SDK_REQ_ROW(2, 0, nr) SDK_REQ_ROW(3, 0, nr)
        }
#pragma unroll 1
        for (int kk = kk_beg; kk < kk_end; ++kk) {
          const int nrows = REST ? __builtin_amdgcn_readfirstlane(ns_l[kk]) : ns_l[kk];
          // ---- gather: column values of pixel m_local, channels 8*cg + j
          float col[8];
#pragma unroll
          for (int j = 0; j < 8; ++j) col[j] = 0.0f;
          if constexpr (REST) {
            const int nr = min(nrows, 4);
            SDK_USE_ROW(0, row0, nr) SDK_USE_ROW(1, row0, nr) SDK_USE_ROW(2, row0, nr) SDK_USE_ROW(3, row0, nr)
            for (int r = 4; r < nrows; ++r) {   // further rows: one at a time, not requested ahead
              const int2 ec = prow[(row0 + r) * 64 + m_local];
              const int e = ec.x;
              const float co = __int_as_float(ec.y);
              const bool out = e < 0 && co != 0.0f;
              const float4* rp =
                  reinterpret_cast<const float4*>(region + (e >= 0 ? e : 0) * kRegE + 8 * cg);
              const float4 l0 = rp[0], l1 = rp[1];
              const float dl[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
              const unsigned o0 = out ? (unsigned)(-e - 1) * 4u : 0u;
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                const float dg = *reinterpret_cast<const float*>(rest_base + (o0 + ch_off[j]));
                col[j] = __builtin_fmaf(co, out ? dg : dl[j], col[j]);
              }
            }
            row0 += nrows;
            if (kk + 1 < kk_end) {
              const int nn = min(__builtin_amdgcn_readfirstlane(ns_l[kk + 1]), 4);
              SDK_REQ_ROW(0, row0, nn) SDK_REQ_ROW(1, row0, nn) SDK_REQ_ROW(2, row0, nn) SDK_REQ_ROW(3, row0, nn)
            }
          } else {
          // adds one row (window index or image offset e, coefficient co) to col[]
          auto tap_any = [&](int e, float co) {
            // some lane's tap lies outside the window: that lane reads the image directly
            // (uniform base, 32-bit byte offsets; 32 planes of < 2^24 elements fit)
            const bool out = e < 0 && co != 0.0f;
            const float4* rp = reinterpret_cast<const float4*>(region + (e >= 0 ? e : 0) * kRegE + 8 * cg);
            const float4 l0 = rp[0], l1 = rp[1];
            const float dl[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
            const char* gbase = reinterpret_cast<const char*>(img_b + (size_t)c0 * HW);
            const unsigned plane = (unsigned)HW * 4u;
            const unsigned o0 = out ? (unsigned)(8 * cg) * plane + (unsigned)(-e - 1) * 4u : 0u;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const bool g_ok = out && c0 + 8 * cg + j < Cg;
              const float dg =
                  *reinterpret_cast<const float*>(gbase + (g_ok ? o0 + (unsigned)j * plane : 0u));
              col[j] = __builtin_fmaf(co, e >= 0 ? dl[j] : (g_ok ? dg : 0.0f), col[j]);
            }
          };
          int r_first = 0;
          if (PRE && pre_valid) {   // first row: outside lanes use the values requested a sample ago
            const int2 ec = prow[row0 * 64 + m_local];
            const int e = ec.x;
            const float co = __int_as_float(ec.y);
            const bool out = e < 0 && co != 0.0f;
            const float4* rp = reinterpret_cast<const float4*>(region + (e >= 0 ? e : 0) * kRegE + 8 * cg);
            const float4 l0 = rp[0], l1 = rp[1];
            const float dl[8] = {l0.x, l0.y, l0.z, l0.w, l1.x, l1.y, l1.z, l1.w};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const bool g_ok = out && c0 + 8 * cg + j < Cg;
              col[j] = __builtin_fmaf(co, e >= 0 ? dl[j] : (g_ok ? pre[j] : 0.0f), col[j]);
            }
            r_first = 1;
          }
          for (int r = r_first; r < nrows; r += 2) {
            // two rows per step so that their LDS reads overlap
            const int2 ec0 = prow[(row0 + r) * 64 + m_local];
            const int2 ec1 = (r + 1 < nrows) ? prow[(row0 + r + 1) * 64 + m_local] : make_int2(0, 0);
            const float co0 = __int_as_float(ec0.y), co1 = __int_as_float(ec1.y);
            if (__all((ec0.x >= 0 || co0 == 0.0f) && (ec1.x >= 0 || co1 == 0.0f))) {
              const float4* rp0 = reinterpret_cast<const float4*>(
                  region + (ec0.x >= 0 ? ec0.x : 0) * kRegE + 8 * cg);
              const float4* rp1 = reinterpret_cast<const float4*>(
                  region + (ec1.x >= 0 ? ec1.x : 0) * kRegE + 8 * cg);
              const float4 a0 = rp0[0], a1 = rp0[1], b0 = rp1[0], b1 = rp1[1];
              const float d0[8] = {a0.x, a0.y, a0.z, a0.w, a1.x, a1.y, a1.z, a1.w};
              const float d1[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                col[j] = __builtin_fmaf(co0, d0[j], col[j]);
                col[j] = __builtin_fmaf(co1, d1[j], col[j]);
              }
            } else {
              tap_any(ec0.x, co0);
              tap_any(ec1.x, co1);
            }
          }
          row0 += nrows;
          // ---- request the outside values of the next sample's first row
          pre_valid = false;
          if (PRE && kk + 1 < kk_end && ns_l[kk + 1] > 0) {
            const int2 ec = prow[row0 * 64 + m_local];
            const bool out = ec.x < 0 && __int_as_float(ec.y) != 0.0f;
            if (__any(out)) {
              const char* gbase = reinterpret_cast<const char*>(img_b + (size_t)c0 * HW);
              const unsigned plane = (unsigned)HW * 4u;
              const unsigned o0 = out ? (unsigned)(8 * cg) * plane + (unsigned)(-ec.x - 1) * 4u : 0u;
#pragma unroll
              for (int j = 0; j < 8; ++j) {
                const bool g_ok = out && c0 + 8 * cg + j < Cg;
                pre[j] = *reinterpret_cast<const float*>(gbase + (g_ok ? o0 + (unsigned)j * plane : 0u));
              }
              pre_valid = true;
            }
          }
          }  // !REST
          float* ct = colT[buf];
          if constexpr (SPLIT) {
            // The column tile is split where it is written, once, instead of by each of the four
            // waves that read it: three bf16 tiles piece[c][m] (rows of kSplitLd elements, pixel
            // bits 4-5 flipped by the channel group to spread the groups over the banks), in
            // the space of one fp32 tile, so the tile is single-buffered here.
            unsigned short* pt = reinterpret_cast<unsigned short*>(&colT[0][0]);
            const int ms = m_local ^ (cg << 4);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const unsigned hb = __float_as_uint(col[j]) & 0xffff0000u;
              const float r = col[j] - __uint_as_float(hb);
              const unsigned mb = __float_as_uint(r) & 0xffff0000u;
              const float r2 = r - __uint_as_float(mb);
              const unsigned lb = __float_as_uint(r2) & 0xffff0000u;
              const int at = (8 * cg + j) * kSplitLd + ms;
              pt[at] = (unsigned short)(hb >> 16);
              pt[kCC * kSplitLd + at] = (unsigned short)(mb >> 16);
              pt[2 * kCC * kSplitLd + at] = (unsigned short)(lb >> 16);
            }
          } else {
#pragma unroll
            for (int j = 0; j < 8; ++j) ct[(8 * cg + j) * kColLd + (m_local ^ ((cg & 1) << 4))] = col[j];
          }
          lds_only_barrier();   // the requests above stay in flight

          // ---- D[n][c] += A[n][m] * col[c][m]; one copy of this block per accumulator
          // rows of channel group cg = nl / 8 were written with pixel bit 4 flipped by cg
          const float* bt = ct + nl * kColLd;
          const int sw = ((nl >> 3) & 1) << 4;
          auto mma = [&](floatx16& d) {
            if constexpr (SPLIT) {
              const unsigned short* pt = reinterpret_cast<const unsigned short*>(&colT[0][0]);
              const int sws = ((nl >> 3) & 3) << 4;
#pragma unroll
              for (int t = 0; t < PXW / 16; ++t) {
                const int at = nl * kSplitLd + ((poff + 16 * t + 8 * h) ^ sws);
                Bf16Split b;
                b.hi.v = *reinterpret_cast<const bf16x8*>(pt + at);
                b.mid.v = *reinterpret_cast<const bf16x8*>(pt + kCC * kSplitLd + at);
                b.lo.v = *reinterpret_cast<const bf16x8*>(pt + 2 * kCC * kSplitLd + at);
                d = mfma_split(afrag3[t], b, d);
              }
            } else if constexpr (BF16) {
#pragma unroll
              for (int t = 0; t < PXW / 16; ++t) {
                const float4 lo = *reinterpret_cast<const float4*>(bt + ((poff + 16 * t + 8 * h) ^ sw));
                const float4 hi = *reinterpret_cast<const float4*>(bt + ((poff + 16 * t + 8 * h + 4) ^ sw));
                const float f[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
                d = mfma_bf16(afrag16[t], pack_bf16x8(f), d);
              }
            } else {
              float4 b = *reinterpret_cast<const float4*>(bt + ((poff + 4 * h) ^ sw));
#pragma unroll
              for (int g = 0; g < PXW / 8; ++g) {
                float4 bn = b;
                if (g < PXW / 8 - 1)
                  bn = *reinterpret_cast<const float4*>(bt + ((poff + 8 * (g + 1) + 4 * h) ^ sw));
                d = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * g + 0], b.x, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * g + 1], b.y, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * g + 2], b.z, d, 0, 0, 0);
                d = __builtin_amdgcn_mfma_f32_32x32x2f32(afrag[4 * g + 3], b.w, d, 0, 0, 0);
                b = bn;
              }
            }
          };
#pragma unroll
          for (int u = 0; u < KB; ++u)
            if (u == kk) mma(acc[u]);
          if constexpr (SPLIT) lds_only_barrier();   // single tile: all reads before the next writes
          else buf ^= 1;
        }
#undef SDK_REQ_ROW
#undef SDK_USE_ROW
        kk_beg = kk_end;
      }
    }
  }

  // ---- with a partial-sum buffer: every accumulator register is stored as it lies
  // (register-major, thread fastest: full 256-byte rows per wave) and wgrad_reduce_kernel sums the
  // workgroups' copies.  All workgroups finish together, so adding 147 KB each to the same
  // addresses of gW here would queue their device-scope atomics behind one another.
  if (partial != nullptr) {
    float* dst = partial + (size_t)blockIdx.x * (KB * 16 * kPlThreads) + tid;
#pragma unroll
    for (int kk = 0; kk < KB; ++kk)
#pragma unroll
      for (int v = 0; v < 16; ++v) dst[(kk * 16 + v) * kPlThreads] = acc[kk][v];
    return;
  }
  // ---- gW[n][c*K + k] += D[n][c]; accumulator register v: row 8*(v/4) + 4*h + v%4, column nl
  const int c = c0 + nl;
  if (c < Cg) {
#pragma unroll
    for (int kk = 0; kk < KB; ++kk) {
      if (kk < kcount) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int n = n0 + 32 * nbw + 8 * (v >> 2) + 4 * h + (v & 3);
          if (n < Cp)
            atomic_add_noret(gW + (size_t)n * Cg * K + (size_t)c * K + k0 + kk, acc[kk][v]);
        }
      }
    }
  }
}

// Sums the accumulator copies planned_wgrad_kernel left in `partial` and adds them to gW.
// Block (x, y, z): accumulator register x = kk * 16 + v of thread threadIdx.x, for the
// workgroup kind y (channel chunk, row-block tile, sample block), over every z-th of the
// batches * groups workgroups of that kind.  The index arithmetic mirrors the kernel's.
__global__ __launch_bounds__(kPlThreads) void wgrad_reduce_kernel(
    const float* __restrict__ partial, float* __restrict__ gW, int Cg, int Cp, int K, int KB,
    int NW, int groups, int batches, int c_chunks, int n_tiles, int kblocks,
    const int* __restrict__ tile_count) {
  if (tile_count != nullptr && *tile_count == 0) return;   // nothing was summed
  const int tid = threadIdx.x, kkv = blockIdx.x, kk = kkv >> 4, v = kkv & 15;
  const int kb = blockIdx.y % kblocks, nt = (blockIdx.y / kblocks) % n_tiles;
  const int cc = blockIdx.y / (kblocks * n_tiles);
  const int kinds = c_chunks * n_tiles * kblocks * batches;
  const int total = batches * groups;
  const size_t per_wg = (size_t)KB * 16 * kPlThreads;
  // four reads in flight per thread (a plain loop waits for each in turn)
  auto at = [&](int i) {
    const int ic = min(i, total - 1);
    const int b = ic / groups, grp = ic % groups;
    const int kind = ((b * c_chunks + cc) * n_tiles + nt) * kblocks + kb;
    const size_t wg = ((size_t)(grp >> 3) * kinds + kind) * 8 + (grp & 7);
    const float val = partial[wg * per_wg + (size_t)kkv * kPlThreads + tid];
    return i < total ? val : 0.0f;
  };
  float s0 = 0.0f, s1 = 0.0f, s2 = 0.0f, s3 = 0.0f;
  const int step = gridDim.z;
  for (int i = blockIdx.z; i < total; i += 4 * step) {
    const float v0 = at(i), v1 = at(i + step), v2 = at(i + 2 * step), v3 = at(i + 3 * step);
    s0 += v0;
    s1 += v1;
    s2 += v2;
    s3 += v3;
  }
  const float s = (s0 + s1) + (s2 + s3);
  const int wave = tid >> 6, lane = tid & 63, nl = lane & 31, h = lane >> 5;
  const int c = cc * kCC + nl;
  const int n = nt * (32 * NW) + 32 * (wave % NW) + 8 * (v >> 2) + 4 * h + (v & 3);
  const int k = kb * KB + kk;
  if (c < Cg && n < Cp && k < K) atomic_add_noret(gW + (size_t)n * Cg * K + (size_t)c * K + k, s);
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------
PixelTiling plan_tiling(int OH, int OW) {
  PixelTiling pt;
  pt.OH = OH;
  pt.OW = OW;
  pt.tx_shift = (OH >= 8) ? 4 : (OH >= 4 ? 5 : (OH >= 2 ? 6 : 7));
  // narrow grids: no wider than the grid needs
  while (pt.tx_shift > 0 && (1 << (pt.tx_shift - 1)) >= OW) --pt.tx_shift;
  pt.tiles_x = (int)ceil_div(OW, pt.TX());
  pt.tiles_y = (int)ceil_div(OH, pt.TY());
  return pt;
}

static int plan_slots(const ConvGeom& g) {
  return pts(g.P) * ((g.interp == 1 || g.interp == 2) ? 4 : 1);
}

bool plan_supported(const ConvGeom& g) {
  if (g.OW < 1 || g.M % g.OW != 0 || g.K > kPlanKMax) return false;
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  const int64_t tiles = (int64_t)pt.tiles_x * pt.tiles_y;
  return tiles * g.K * plan_slots(g) * 128 < ((int64_t)1 << 40) && tiles * kHdrStride < ((int64_t)1 << 31);
}

static size_t align16(size_t v) { return (v + 15) & ~(size_t)15; }

namespace {
// [header][rows per sample][plan rows][big windows]
struct PlanOffsets {
  size_t ns, taps, big_lut, total;
};
PlanOffsets plan_offsets(const ConvGeom& g) {
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  const size_t tiles = (size_t)pt.tiles_x * pt.tiles_y;
  PlanOffsets o;
  o.ns = align16(tiles * kHdrStride * sizeof(int));
  o.taps = o.ns + align16(tiles * g.K * sizeof(int));
  o.big_lut = o.taps + tiles * g.K * plan_slots(g) * 128 * sizeof(int2);
  o.total = o.big_lut + align16(tiles * kBigStride * sizeof(int));
  return o;
}
}  // namespace

size_t plan_bytes(const ConvGeom& g) { return plan_offsets(g).total; }

void load_plan(const ConvGeom& g, void* workspace, Plan* plan) {
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  const PlanOffsets o = plan_offsets(g);
  char* base = static_cast<char*>(workspace);
  plan->pt = pt;
  plan->tiles = pt.tiles_x * pt.tiles_y;
  plan->S = plan_slots(g);
  plan->hdr = reinterpret_cast<int*>(base);
  plan->ns = reinterpret_cast<int*>(base + o.ns);
  plan->taps = reinterpret_cast<int2*>(base + o.taps);
  plan->big_lut = reinterpret_cast<int*>(base + o.big_lut);
}

int build_plan(const ConvGeom& g, const float* map, const float* wts, void* workspace,
               hipStream_t stream, Plan* plan, const int* gate, bool with_big) {
  load_plan(g, workspace, plan);
  if (!with_big) plan->big_lut = nullptr;
  SDK_DISPATCH_INTERP(g.interp, g.P,
                      (launch(plan_kernel<INTERP, WEIGHTED>, dim3((unsigned)plan->tiles),
                              dim3(kPlThreads), stream, map, wts, plan->pt, g.K, g.P, g.H, g.W,
                              plan->S, const_cast<int*>(plan->hdr), const_cast<int*>(plan->ns),
                              const_cast<int2*>(plan->taps), gate,
                              const_cast<int*>(plan->big_lut))));
  SDK_LAUNCH_CHECK("plan");
  return SDK_OK;
}

bool planned_wgrad_supported(const ConvGeom& g) {
  return plan_supported(g) && plan_slots(g) <= kRowCap && g.B <= 65535;
}

namespace {
// Launch shape of planned_wgrad_kernel: KB samples per workgroup, NW row blocks, and how many
// tile runs (`groups`) each kind of workgroup is split into.
struct WgradGrid {
  int KB, kb_count, NW, c_chunks, n_tiles, groups;
  int64_t kinds, slots;
};

// rest: the launch shape of the REST variant of the kernel (at most 5 samples per workgroup,
// which leaves registers for the values requested ahead).
WgradGrid wgrad_grid(const ConvGeom& g, int tiles, bool rest) {
  WgradGrid w;
  const int kblocks = (int)ceil_div(g.K, rest ? 5 : 9);
  const int per = (int)ceil_div(g.K, kblocks);
  w.KB = per <= 1 ? 1 : (per <= 4 ? 4 : (rest ? 5 : (per <= 7 ? 7 : 9)));
  w.kb_count = (int)ceil_div(g.K, w.KB);
  w.NW = g.Cp > 64 ? 4 : (g.Cp > 32 ? 2 : 1);
  w.c_chunks = (int)ceil_div(g.Cg, kCC);
  w.n_tiles = (int)ceil_div(g.Cp, 32 * w.NW);
  w.kinds = (int64_t)w.c_chunks * w.n_tiles * w.kb_count * g.B;
  // tile runs: a multiple of 8 (one set per XCD), about two workgroups per CU overall
  const int64_t want = std::max<int64_t>(8, ceil_div(ceil_div(512, w.kinds), 8) * 8);
  w.groups = (int)std::min<int64_t>(tiles, want);
  const int tpg = (int)ceil_div(tiles, w.groups);
  w.groups = (int)ceil_div(tiles, tpg);
  w.slots = ceil_div(w.groups, 8) * 8 * w.kinds;
  return w;
}

// Largest partial-sum buffer worth reserving; calls that would need more add to gW directly.
constexpr size_t kWgradPartialCap = (size_t)160 << 20;
}  // namespace

size_t planned_wgrad_partial_bytes(const ConvGeom& g) {
  if (g.B == 0 || !planned_wgrad_supported(g)) return 0;
  const PixelTiling pt = plan_tiling(g.M / g.OW, g.OW);
  // room for either launch shape
  size_t bytes = 0;
  for (int rest = 0; rest < 2; ++rest) {
    const WgradGrid w = wgrad_grid(g, pt.tiles_x * pt.tiles_y, rest != 0);
    if (w.slots >= ((int64_t)1 << 31)) return 0;
    bytes = std::max(bytes, (size_t)w.slots * w.KB * 16 * kPlThreads * sizeof(float));
  }
  return bytes <= kWgradPartialCap ? bytes : 0;
}

int planned_wgrad(const ConvGeom& g, int mm, const Plan& plan, const float* pix,
                  const float* img, float* gW, float* partial, hipStream_t stream,
                  const int* tile_list, const int* tile_count) {
  // A listed launch in float32 covers the tiles the window kernel left.  Where the plain
  // variant has no registers to request values ahead (nine samples, 128 rows), the REST
  // variant takes its place.
  const WgradGrid plain = wgrad_grid(g, plan.tiles, false);
  const bool rest = tile_list != nullptr && mm == kMmF32 && plain.KB == 9 && plain.NW == 4;
  const WgradGrid wg = rest ? wgrad_grid(g, plan.tiles, true) : plain;
  const int KB = wg.KB, kb_count = wg.kb_count, NW = wg.NW;
  const int c_chunks = wg.c_chunks, n_tiles = wg.n_tiles, groups = wg.groups;
  const int64_t slots = wg.slots;
  if (slots >= ((int64_t)1 << 31)) return fail(SDK_ERR_UNSUPPORTED, "planned_wgrad: grid too large");
  const int TX = plan.pt.TX();
  // a lane loads one run of 4 (fp32) or 8 (bf16, split) consecutive pixels of a tile row with
  // 16-byte loads and checks the run's first pixel only: runs must not straddle the row end
  const int run = mm != kMmF32 ? 8 : 4;
  const int vec4 = (g.OW % run == 0 && TX >= run &&
                    reinterpret_cast<uintptr_t>(pix) % 16 == 0) ? 1 : 0;
  const dim3 grid((unsigned)slots);
#define PW3(KBv, BFv, NWv)                                                                      \
  launch(planned_wgrad_kernel<KBv, BFv, NWv, false>, grid, dim3(kPlThreads), stream, pix, img,         \
         plan.hdr, plan.ns, plan.taps, gW, partial, g.Cg, g.H, g.W, g.Cp, g.K, plan.S, plan.pt, \
         plan.tiles, groups, (int)g.B, c_chunks, n_tiles, kb_count, vec4, tile_list, tile_count, \
         plan.big_lut)
#define PW(KBv, BFv)                                                                            \
  do {                                                                                          \
    if (NW == 4) PW3(KBv, BFv, 4); else if (NW == 2) PW3(KBv, BFv, 2); else PW3(KBv, BFv, 1);   \
  } while (0)
  if (mm == kMmBf16) {
    if (KB == 1) PW(1, kMmBf16); else if (KB == 4) PW(4, kMmBf16); else if (KB == 7) PW(7, kMmBf16); else PW(9, kMmBf16);
  } else if (mm == kMmSplit) {
    if (KB == 1) PW(1, kMmSplit); else if (KB == 4) PW(4, kMmSplit); else if (KB == 7) PW(7, kMmSplit); else PW(9, kMmSplit);
  } else if (rest) {
#define PR3(KBv, NWv)                                                                           \
  launch(planned_wgrad_kernel<KBv, kMmF32, NWv, true>, grid, dim3(kPlThreads), stream, pix, img, \
         plan.hdr, plan.ns, plan.taps, gW, partial, g.Cg, g.H, g.W, g.Cp, g.K, plan.S, plan.pt, \
         plan.tiles, groups, (int)g.B, c_chunks, n_tiles, kb_count, vec4, tile_list, tile_count, \
         plan.big_lut)
    if (KB == 4) PR3(4, 4); else PR3(5, 4);   // K = 10 .. 16 -> two or more blocks of 4 or 5
#undef PR3
  } else {
    if (KB == 1) PW(1, kMmF32); else if (KB == 4) PW(4, kMmF32); else if (KB == 7) PW(7, kMmF32); else PW(9, kMmF32);
  }
#undef PW
#undef PW3
  SDK_LAUNCH_CHECK("planned_wgrad");
  if (partial != nullptr) {
    const int kinds0 = c_chunks * n_tiles * kb_count, total = (int)g.B * groups;
    // enough blocks to fill the GPU: the workgroups of a kind are summed in up to 16 parts
    const int parts = (int)std::min<int64_t>(std::min(total, 16), ceil_div(2048, (int64_t)KB * 16 * kinds0));
    launch(wgrad_reduce_kernel, dim3((unsigned)(KB * 16), (unsigned)kinds0, (unsigned)std::max(parts, 1)),
           dim3(kPlThreads), stream, (const float*)partial, gW, g.Cg, g.Cp, g.K, KB, NW, groups,
           (int)g.B, c_chunks, n_tiles, kb_count, tile_list != nullptr ? tile_count : nullptr);
    SDK_LAUNCH_CHECK("wgrad_reduce");
  }
  return SDK_OK;
}

}  // namespace sdk
