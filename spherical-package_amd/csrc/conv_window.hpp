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

// src[e], e < RS: flat offset inside one image plane of region element e, or -1
// for a row outside the image.
__device__ __forceinline__ void build_region_lut(const Region& r, int H, int W,
                                                 int* __restrict__ src) {
  for (int e = threadIdx.x; e < r.RS; e += blockDim.x) {
    const int ry = e / r.RW, rx = e - ry * r.RW;
    const int y = r.ry0 + ry;
    int x = r.rx0 + rx;
    x -= x >= W ? W : 0;
    src[e] = ((unsigned)y < (unsigned)H) ? y * W + x : -1;
  }
}

}  // namespace sdk
