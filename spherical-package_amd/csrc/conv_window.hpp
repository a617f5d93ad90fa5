// Building blocks of the LDS-staged convolution kernels (conv_plan_scatter.hip, conv_plan.hip):
// 2-D taps, the per-workgroup image region and its addressing.
//
// A workgroup owns a small 2-D tile of map pixels.  The union of everything its
// K x P samples touch in the image is, for a locally coherent map, a slightly
// larger 2-D window of the image.  That window ("region") is staged in LDS per
// chunk of channels: gathers read it instead of global memory, scatters
// accumulate into it with LDS atomics and flush once.  Columns of the window
// wrap modulo the image width, so a tile at the longitude seam stays compact.
// Taps that fall outside the window (incoherent maps, polar rows) still work:
// they go to global memory directly.
#pragma once
#include <hip/hip_runtime.h>

#include <climits>

#include "sdk_taps.hpp"

namespace sdk {

constexpr int kCC = 32;          // channels staged per region chunk
constexpr int kRegionCap = 288;  // region elements per channel (kCC * 289 * 4 B = 36 KB)
// A plan's header: kHdrStride ints per tile.  [0..3] window origin and size (row, column,
// rows, columns; a listed window reads 0, 0, 1, count), [4] 1 when every tap of the tile lies
// inside the window, [5] most rows of a sample, [6] 1 for a listed window, [8 + e] the flat
// image offset of window element e (-1: outside the image).
constexpr int kHdrLut = 8;
constexpr int kHdrStride = kHdrLut + kRegionCap;
// A tile whose taps fit no window of kRegionCap elements but touch at most kBigCap distinct
// ones gets, besides its ordinary plan rows, a second set over a listed window of that size
// ("big" tile; conv_plan.hpp), for kernels that give the window most of a CU's LDS.
constexpr int kBigCap = 768;
constexpr int kBigLut = 8;                         // [0] elements, [kBigLut + e] flat offset,
constexpr int kBigStride = kBigLut + 2 * kBigCap;  // [kBigLut + kBigCap + e] ordinary encoding

// Up to four taps of one sample point as (row, column, coefficient).  A tap that
// is out of range or has zero weight gets coefficient 0 (and row = column = 0).
template <int INTERP>
struct Taps2D {
  static constexpr int N = (INTERP == 0) ? 1 : 4;
  int y[N], x[N];
  float w[N];

  __device__ __forceinline__ void set(float px, float py, int H, int W, float scale) {
    if constexpr (INTERP == 0) {
      const int xi = to_int_clamped(round_t(px));
      const int yi = to_int_clamped(round_t(py));
      const bool ok = (unsigned)xi < (unsigned)W && (unsigned)yi < (unsigned)H;
      x[0] = ok ? xi : 0;
      y[0] = ok ? yi : 0;
      w[0] = ok ? scale : 0.0f;
    } else {
      const float fx = floor_t(px), fy = floor_t(py);
      const int x1 = to_int_clamped(fx), y1 = to_int_clamped(fy);
      const float A = (fy + 1.0f) - py, B = (fx + 1.0f) - px, C = px - fx, D = py - fy;
      const bool y1ok = (unsigned)y1 < (unsigned)H;
      const bool y2ok = y1 >= -1 && y1 < H - 1;
      int c1, c2;
      bool x1ok, x2ok;
      if constexpr (INTERP == 2) {
        c1 = wrap_index(x1, W);
        c2 = (c1 + 1 == W) ? 0 : c1 + 1;
        x1ok = x2ok = true;
      } else {
        c1 = x1;
        c2 = x1 + 1;
        x1ok = (unsigned)x1 < (unsigned)W;
        x2ok = x1 >= -1 && x1 < W - 1;
      }
      const float ww[4] = {scale * (A * B), scale * (A * C), scale * (D * B), scale * (D * C)};
      const bool ok[4] = {x1ok && y1ok, x2ok && y1ok, x1ok && y2ok, x2ok && y2ok};
      const int yy[4] = {y1, y1, y1 + 1, y1 + 1};
      const int xx[4] = {c1, c2, c1, c2};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool on = ok[i] && ww[i] != 0.0f;
        w[i] = on ? ww[i] : 0.0f;
        y[i] = on ? yy[i] : 0;
        x[i] = on ? xx[i] : 0;
      }
    }
  }
};

// Window of the image staged in LDS: rows [ry0, ry0+RH), columns
// (rx0 + [0, RW)) mod W.  RSp, the per-channel stride, is odd so that lanes
// addressing the same element of consecutive channels hit distinct banks.
struct Region {
  int ry0, rx0, RH, RW, RS, RSp;

  // >= 0: element index inside one channel's window; < 0: -(flat image offset) - 1.
  __device__ __forceinline__ int encode(int y, int x, int W) const {
    const int ry = y - ry0;
    int rx = x - rx0;
    rx += rx < 0 ? W : 0;
    const bool inside = (unsigned)ry < (unsigned)RH && (unsigned)rx < (unsigned)RW;
    return inside ? ry * RW + rx : -(y * W + x) - 1;
  }
};

__device__ __forceinline__ int wave_min(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = min(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ int wave_max(int v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = max(v, __shfl_xor(v, o, 64));
  return v;
}

// 2-D tiling of the OH x OW pixel grid: 128 pixels per workgroup as TY x TX with
// TX = 1 << tx_shift.
struct PixelTiling {
  int OH, OW, tx_shift, tiles_x, tiles_y;
  __host__ __device__ int TX() const { return 1 << tx_shift; }
  __host__ __device__ int TY() const { return 128 >> tx_shift; }
};

// Turns the bounding box [dy0, dy1] x [dx0, dx1] of a tile's taps (relative to the
// anchor (ay, ax), columns unwrapped) into the staged window: the whole box when it
// fits the capacity, otherwise a window around the tile; what falls outside is
// served from global memory.
__device__ __forceinline__ Region choose_region(int dy0, int dy1, int dx0, int dx1, int ay, int ax,
                                                int TY, int TX, int W) {
  Region r;
  if (dy0 > dy1) {  // no active tap at all
    r.ry0 = ay;
    r.rx0 = ax;
    r.RH = 1;
    r.RW = 1;
  } else {
    int RH = dy1 - dy0 + 1, RW = min(dx1 - dx0 + 1, W);
    int ry0 = ay + dy0, rx0 = ax + dx0;
    if (RH * RW > kRegionCap) {
      const int RHc = min(RH, 16);
      const int RWc = min(RW, kRegionCap / RHc);
      const int cy = (RH <= 2 * RHc) ? ay + (dy0 + dy1) / 2 : ay + TY / 2;
      const int cx = (RW <= 2 * RWc) ? ax + (dx0 + dx1) / 2 : ax + TX / 2;
      ry0 = cy - RHc / 2;
      rx0 = cx - RWc / 2;
      RH = RHc;
      RW = RWc;
    }
    r.ry0 = ry0;
    r.rx0 = wrap_index(rx0, W);
    r.RH = RH;
    r.RW = RW;
  }
  r.RS = r.RH * r.RW;
  r.RSp = r.RS | 1;
  return r;
}

// lut[e], e < RS: flat offset inside one image plane of element e of a box window, or -1
// for a row outside the image.  Written into the plan's header by the kernels that build plans.
__device__ __forceinline__ void write_region_lut(const Region& r, int H, int W,
                                                 int* __restrict__ lut) {
  for (int e = threadIdx.x; e < r.RS; e += blockDim.x) {
    const int ry = e / r.RW, rx = e - ry * r.RW;
    const int y = r.ry0 + ry;
    int x = r.rx0 + rx;
    x -= x >= W ? W : 0;
    lut[e] = ((unsigned)y < (unsigned)H) ? y * W + x : -1;
  }
}

// src[e] = the tile's window LUT (tile_hdr = hdr + tile * kHdrStride), e < RS.
__device__ __forceinline__ void load_region_lut(const int* __restrict__ tile_hdr, int RS,
                                                int* __restrict__ src) {
  for (int e = threadIdx.x; e < RS; e += blockDim.x) src[e] = tile_hdr[kHdrLut + e];
}

// ---------------------------------------------------------------------------
// Listed windows.  A tile whose taps have a bounding box beyond kRegionCap (neighbour lists
// of a mesh, whose indices say little about distance) may still touch few distinct image
// elements.  The kernels that build plans collect the tile's distinct offsets in an LDS hash
// set; when there are at most kRegionCap, the sorted list becomes the window and a tap's
// window index is its rank in it; up to kBigCap they make the window of a big tile.
// ---------------------------------------------------------------------------
constexpr int kSetSlots = 2048;  // hash slots (> kBigCap + the threads that may insert at once)
constexpr int kSetSort = 1024;   // length of the padded sorted list (power of two >= kBigCap)

struct WindowSet {
  int table[kSetSlots];
  int list[kSetSort];
  int count;   // distinct offsets claimed; inserting stops once it exceeds kBigCap
  int filled;
};

// All threads; a barrier must follow.
__device__ __forceinline__ void set_clear(WindowSet& ws) {
  for (int i = threadIdx.x; i < kSetSlots; i += blockDim.x) ws.table[i] = -1;
  for (int i = threadIdx.x; i < kSetSort; i += blockDim.x) ws.list[i] = INT_MAX;
  if (threadIdx.x == 0) {
    ws.count = 0;
    ws.filled = 0;
  }
}

__device__ __forceinline__ void set_insert(WindowSet& ws, int off) {
  if (*reinterpret_cast<volatile int*>(&ws.count) > kBigCap) return;
  unsigned h = ((unsigned)off * 2654435761u) >> 21;
  for (int probe = 0; probe < kSetSlots; ++probe) {
    const int prev = atomicCAS(&ws.table[h], -1, off);
    if (prev == -1) {
      atomicAdd(&ws.count, 1);
      return;
    }
    if (prev == off) return;
    h = (h + 1) & (kSetSlots - 1);
  }
}

// All threads, after a barrier behind the last set_insert.  Returns the number of distinct
// offsets when there are at most kBigCap (ws.list[0 .. n) is then sorted), otherwise -1.
__device__ __forceinline__ int set_finish(WindowSet& ws) {
  const int n = ws.count;
  if (n > kBigCap) return -1;
  const int len = n <= kSetSort / 2 ? kSetSort / 2 : kSetSort;   // (the padding sorts to the end)
  for (int i = threadIdx.x; i < kSetSlots; i += blockDim.x) {
    const int key = ws.table[i];
    if (key != -1) ws.list[atomicAdd(&ws.filled, 1)] = key;
  }
  __syncthreads();
  for (int k = 2; k <= len; k <<= 1) {
    for (int j = k >> 1; j > 0; j >>= 1) {
      for (int i = threadIdx.x; i < len; i += blockDim.x) {
        const int o = i ^ j;
        if (o > i) {
          const int a = ws.list[i], b = ws.list[o];
          const bool up = (i & k) == 0;
          if ((a > b) == up) {
            ws.list[i] = b;
            ws.list[o] = a;
          }
        }
      }
      __syncthreads();
    }
  }
  return n;
}

// Rank of `off` in the sorted list of n offsets (it is one of them).
__device__ __forceinline__ int set_rank(const WindowSet& ws, int n, int off) {
  int lo = 0, hi = n - 1;
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (ws.list[mid] < off) lo = mid + 1;
    else hi = mid;
  }
  return lo;
}

}  // namespace sdk
