// Mapped max / average pooling from an LDS window (gfx950, float32 planes, unweighted maps).
//
// The per-pixel pooling kernels gather every sample of every plane from global memory: K
// gather instructions per pixel and plane, the rate at which they issue bounds them.  Here
// a workgroup owns one tile of the tap plan (128 pixels whose taps all lie inside the tile's
// window of at most kRegionCap image elements, conv_plan.hpp) and 32 planes: the window of
// those planes is staged in LDS once with coalesced reads (region[element][plane], planes
// fastest: a lane reads 16 planes of one element as four 16-byte accesses), and every sample
// of every pixel is formed from it with the plan's rows (window index, coefficient).
//
//   thread t: pixel t % 128 of the tile, planes 16 (t / 128) .. + 15 of the chunk
//
// Values are formed as the per-pixel kernels form them (common/mapped_max_pool.h:13-57,
// common/mapped_avg_pool.h:13-40 of the reference): products coefficient * value summed in tap
// order, a sample without an active tap is 0, the first maximum wins and NaN never does; the
// index is ((pixel * K + sample) * 2), -1 when no sample won.
#include <hip/hip_runtime.h>

#include <cfloat>

#include "pool_window.hpp"
#include "sdk_host.hpp"

namespace sdk {
namespace {

constexpr int kPwThreads = 256;
constexpr int kPwPlanes = 32;   // planes per workgroup
constexpr int kPwE = 36;        // floats per window element: 32 planes + 4 of skew

template <bool AVG>
__global__ __launch_bounds__(kPwThreads) void pool_window_kernel(
    const float* __restrict__ in, const int* __restrict__ hdr, const int* __restrict__ ns,
    const int2* __restrict__ taps, const int* __restrict__ list, const int* __restrict__ count,
    float* __restrict__ out, int64_t* __restrict__ idx, int planes, int H, int W, int K, int S,
    PixelTiling pt) {
  __shared__ __align__(16) float region[kRegionCap * kPwE];
  __shared__ int src[kRegionCap];
  __shared__ int ns_l[kPlanKMax];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  // workgroup ids go round-robin over the 8 XCDs: XCD x takes an eighth of the list
  const int cnt = *count, per = (cnt + 7) >> 3;
  const int wg = blockIdx.x, slot = (wg & 7) * per + (wg >> 3);
  if ((wg >> 3) >= per || slot >= cnt) return;
  const int tile = list[slot];
  const int plane0 = blockIdx.y * kPwPlanes;
  const size_t HW = (size_t)H * W;
  const int M = pt.OH * pt.OW;
  const int* tile_hdr = hdr + (size_t)tile * kHdrStride;
  const int RS = tile_hdr[2] * tile_hdr[3];
  load_region_lut(tile_hdr, RS, src);
  for (int k = tid; k < K; k += kPwThreads) ns_l[k] = ns[(size_t)tile * K + k];
  __syncthreads();
  {
    // wave w stages planes 8w .. 8w+7; a lane owns window elements lane, lane + 64, ... and
    // has all its reads in flight before the first LDS write
    constexpr int PER_WAVE = kPwPlanes / 4, ITER = (kRegionCap + 63) / 64;
    float v[ITER][PER_WAVE];
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = lane + 64 * it;
      const int o = e < RS ? src[e] : -1;
#pragma unroll
      for (int j = 0; j < PER_WAVE; ++j) {
        const int plane = plane0 + wave * PER_WAVE + j;
        const bool ok = o >= 0 && plane < planes;
        const float d = in[ok ? (size_t)plane * HW + o : 0];
        v[it][j] = ok ? d : 0.0f;
      }
    }
#pragma unroll
    for (int it = 0; it < ITER; ++it) {
      const int e = lane + 64 * it;
      if (e < RS) {
        float4* dst = reinterpret_cast<float4*>(region + e * kPwE + wave * PER_WAVE);
        dst[0] = make_float4(v[it][0], v[it][1], v[it][2], v[it][3]);
        dst[1] = make_float4(v[it][4], v[it][5], v[it][6], v[it][7]);
      }
    }
  }
  __syncthreads();

  const int p = tid & 127, hh = tid >> 7;
  const int oy = (tile / pt.tiles_x) * pt.TY() + (p >> pt.tx_shift);
  const int ox = ((tile % pt.tiles_x) << pt.tx_shift) + (p & (pt.TX() - 1));
  const bool live = oy < pt.OH && ox < pt.OW;
  const int2* rows_p = taps + (size_t)tile * K * S * 128 + p;
  float best[16];
  int best_k[16];
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    best[j] = AVG ? 0.0f : -FLT_MAX;
    best_k[j] = -1;
  }
  for (int k = 0; k < K; ++k) {
    const int nrows = ns_l[k];
    float v[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) v[j] = 0.0f;
    for (int r = 0; r < nrows; ++r) {
      const int2 ec = rows_p[(size_t)(k * S + r) * 128];
      const float co = __int_as_float(ec.y);
      const float4* rp = reinterpret_cast<const float4*>(region + ec.x * kPwE + 16 * hh);
      const float4 a = rp[0], b = rp[1], c = rp[2], d = rp[3];
      const float x[16] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w,
                           c.x, c.y, c.z, c.w, d.x, d.y, d.z, d.w};
      // (a padding row has coefficient 0 and must add nothing, whatever the window holds)
      if (r == 0) {
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = co != 0.0f ? co * x[j] : 0.0f;
      } else {
#pragma unroll
        for (int j = 0; j < 16; ++j) v[j] = co != 0.0f ? v[j] + co * x[j] : v[j];
      }
    }
    if constexpr (AVG) {
#pragma unroll
      for (int j = 0; j < 16; ++j) best[j] += v[j];
    } else {
#pragma unroll
      for (int j = 0; j < 16; ++j)
        if (v[j] > best[j]) {   // strict: first maximum wins, NaN never wins
          best[j] = v[j];
          best_k[j] = k;
        }
    }
  }
  if (live) {
    const int m = oy * pt.OW + ox;
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int plane = plane0 + 16 * hh + j;
      if (plane < planes) {
        const size_t o = (size_t)plane * M + m;
        if constexpr (AVG) {
          out[o] = best[j] / (float)K;
        } else {
          out[o] = best[j];
          idx[o] = best_k[j] < 0 ? (int64_t)-1 : (int64_t)(((size_t)m * K + best_k[j]) * 2);
        }
      }
    }
  }
}

}  // namespace

int window_pool(const float* in, const Plan& plan, const TileLists& tl, float* out, int64_t* idx,
                int64_t planes, int H, int W, int K, hipStream_t stream) {
  const int64_t chunks = ceil_div(planes, kPwPlanes);
  if (chunks > 65535) return fail(SDK_ERR_UNSUPPORTED, "window_pool: too many planes");
  const dim3 grid((unsigned)((plan.tiles + 7) / 8 * 8), (unsigned)chunks);
  if (idx != nullptr)
    launch(pool_window_kernel<false>, grid, dim3(kPwThreads), stream, in, plan.hdr, plan.ns,
           plan.taps, tl.inside, tl.count, out, idx, (int)planes, H, W, K, plan.S, plan.pt);
  else
    launch(pool_window_kernel<true>, grid, dim3(kPwThreads), stream, in, plan.hdr, plan.ns,
           plan.taps, tl.inside, tl.count, out, idx, (int)planes, H, W, K, plan.S, plan.pt);
  SDK_LAUNCH_CHECK("window_pool");
  return SDK_OK;
}

}  // namespace sdk
