// Mapped max / average pooling through full-width row bands staged in LDS, for float32 maps
// of single nearest taps (ext_modules/include/common/mapped_max_pool.h:13-57, :81-133;
// common/mapped_avg_pool.h:13-40, :70-105).
//
// A workgroup owns a band of R whole rows of the pooled grid and a range of planes.  The taps
// of the band are resolved once (one thread = up to IPT pooled pixels, K offsets each, in
// registers) and reused for every plane of the range.  The input rows the band's taps fall
// into are min..max of the tap rows: a handful of whole image rows whatever the longitude
// of a tap is (a kernel next to a pole, or at the wrap seam, spreads over the whole row but
// not over more rows), contiguous in memory, so one plane's share is one contiguous run
// that is copied to LDS with 16-byte loads.  Per pass PG planes are staged, the next pass's
// run is requested into registers before the taps of the current one are read from LDS.
// A band whose rows do not fit in LDS takes one plane per pass, and past that reads its
// taps from global memory; the choice is made per workgroup on the device.
#include <hip/hip_runtime.h>

#include <cfloat>
#include <climits>

#include "pool_band.hpp"
#include "sdk_host.hpp"
#include "sdk_taps.hpp"

namespace sdk {
namespace {

constexpr int kBandBlock = 256;
constexpr int kBandLdsBytes = 52 * 1024;   // three workgroups per CU
constexpr int kBandLdsFloats = kBandLdsBytes / 4;
// 16-byte piece as a plain vector (an array of these is promoted to registers; one of the
// runtime's float4 structs stays in private memory)
typedef float vec4 __attribute__((ext_vector_type(4)));

// One pooled element from the K values of its samples, in ascending sample order.
template <bool AVG, int K>
struct PoolOp {
  float acc = AVG ? 0.0f : -FLT_MAX;
  int best = -1;
  __device__ __forceinline__ void take(float v, int k) {
    if constexpr (AVG) {
      acc += v;
    } else if (v > acc) {   // strict: the first maximum wins, NaN never wins
      acc = v;
      best = k;
    }
  }
  __device__ __forceinline__ float value() const { return AVG ? acc / float(K) : acc; }
};

// Requests the band rows of the planes p .. p + PGX - 1 (clamped to the last plane) into
// registers: thread t takes the 16-byte pieces t, t + 256, ... of each plane's run.
template <int PGX, int NV>
__device__ __forceinline__ void request_band(vec4 (&pre)[PGX][NV], const float* __restrict__ in,
                                             size_t HW, int row_start, int n_vec, int p,
                                             int p_end) {
  const int t = threadIdx.x;
#pragma unroll
  for (int g = 0; g < PGX; ++g) {
    const int plane = min(p + g, p_end - 1);
    const vec4* src = reinterpret_cast<const vec4*>(in + (size_t)plane * HW + row_start);
#pragma unroll
    for (int i = 0; i < NV; ++i) pre[g][i] = src[min(t + kBandBlock * i, n_vec - 1)];
  }
}

template <bool AVG, int K, int IPT, int PGX>
__device__ __forceinline__ void run_band(const float* __restrict__ in, float* __restrict__ out,
                                         int64_t* __restrict__ idx, float* lds,
                                         int (&off)[IPT][K], int pix0, int npix, int p_begin,
                                         int p_end, size_t HW, int M, int row_start, int n_vec) {
  constexpr int NV = (kBandLdsFloats / PGX / 4 + kBandBlock - 1) / kBandBlock;
  const int t = threadIdx.x;
  const int band_elems = n_vec * 4;
  const int plane_stride = band_elems + 4;   // floats; the element behind the band holds zero
  // taps as byte offsets into one plane's share of the LDS band
#pragma unroll
  for (int j = 0; j < IPT; ++j)
#pragma unroll
    for (int k = 0; k < K; ++k)
      off[j][k] = off[j][k] < 0 ? band_elems * 4 : (off[j][k] - row_start) * 4;
  if (t < PGX) lds[t * plane_stride + band_elems] = 0.0f;

  // (a band none of whose taps lies in the image has no rows: n_vec = 0, the loads below
  // then read the first piece of the plane and nothing is stored to LDS)
  // PGX > 1: the next pass's rows wait in registers while this pass's taps are read.  The
  // one-plane form (bands too tall for two planes) stages in place, four pieces at a time.
  constexpr bool AHEAD = PGX > 1;
  vec4 pre[AHEAD ? PGX : 1][AHEAD ? NV : 4];
  if constexpr (AHEAD) request_band<PGX, NV>(pre, in, HW, row_start, max(n_vec, 1), p_begin, p_end);
  for (int p = p_begin; p < p_end; p += PGX) {
    if constexpr (AHEAD) {
#pragma unroll
      for (int g = 0; g < PGX; ++g) {
        vec4* dst = reinterpret_cast<vec4*>(lds + g * plane_stride);
#pragma unroll
        for (int i = 0; i < NV; ++i)
          if (t + kBandBlock * i < n_vec) dst[t + kBandBlock * i] = pre[g][i];
      }
    } else {
      const vec4* src = reinterpret_cast<const vec4*>(in + (size_t)p * HW + row_start);
      vec4* dst = reinterpret_cast<vec4*>(lds);
      for (int i0 = 0; i0 * kBandBlock < n_vec; i0 += 4) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          pre[0][i] = src[min(t + kBandBlock * (i0 + i), n_vec - 1)];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (t + kBandBlock * (i0 + i) < n_vec) dst[t + kBandBlock * (i0 + i)] = pre[0][i];
      }
    }
    __syncthreads();
    if constexpr (AHEAD) {
      if (p + PGX < p_end)
        request_band<PGX, NV>(pre, in, HW, row_start, max(n_vec, 1), p + PGX, p_end);
    }
#pragma unroll
    for (int j = 0; j < IPT; ++j) {
      const int i = t + kBandBlock * j;
      if (i >= npix) continue;
      // (one pooled pixel's reads at a time: hoisting all of them costs the registers that
      // hold the next pass)
      __builtin_amdgcn_sched_barrier(0);
      const int pix = pix0 + i;
      float v[PGX][K];
#pragma unroll
      for (int g = 0; g < PGX; ++g)
#pragma unroll
        for (int k = 0; k < K; ++k)
          v[g][k] = *reinterpret_cast<const float*>(reinterpret_cast<const char*>(lds) +
                                                    g * plane_stride * 4 + off[j][k]);
#pragma unroll
      for (int g = 0; g < PGX; ++g) {
        if (p + g >= p_end) continue;
        PoolOp<AVG, K> op;
#pragma unroll
        for (int k = 0; k < K; ++k) op.take(v[g][k], k);
        const size_t o = (size_t)(p + g) * M + pix;
        // results are not read again by this kernel: stored past the caches, which the
        // band rows shared by neighbouring workgroups then keep (max pooling of a
        // 8 x 64 x 256 x 512 input: 102 -> 82 us)
        __builtin_nontemporal_store(op.value(), out + o);
        if constexpr (!AVG)
          __builtin_nontemporal_store(
              op.best < 0 ? (int64_t)-1 : (int64_t)(((size_t)pix * K + op.best) * 2), idx + o);
      }
    }
    __syncthreads();
  }
}

// The same band without LDS: every tap is read from global memory.
template <bool AVG, int K, int IPT>
__device__ __forceinline__ void run_direct(const float* __restrict__ in, float* __restrict__ out,
                                           int64_t* __restrict__ idx, const int (&off)[IPT][K],
                                           int pix0, int npix, int p_begin, int p_end, size_t HW,
                                           int M) {
  const int t = threadIdx.x;
  for (int p = p_begin; p < p_end; ++p) {
    const float* plane = in + (size_t)p * HW;
#pragma unroll
    for (int j = 0; j < IPT; ++j) {
      const int i = t + kBandBlock * j;
      if (i >= npix) continue;
      const int pix = pix0 + i;
      float v[K];
#pragma unroll
      for (int k = 0; k < K; ++k) v[k] = plane[off[j][k] < 0 ? 0 : off[j][k]];
      PoolOp<AVG, K> op;
#pragma unroll
      for (int k = 0; k < K; ++k) op.take(off[j][k] < 0 ? 0.0f : v[k], k);
      const size_t o = (size_t)p * M + pix;
      out[o] = op.value();
      if constexpr (!AVG)
        idx[o] = op.best < 0 ? (int64_t)-1 : (int64_t)(((size_t)pix * K + op.best) * 2);
    }
  }
}

// grid.x = 8 * nbands * ceil(chunks / 8): workgroup ids go round-robin over the 8 XCDs; XCD x
// takes the plane chunks x, x + 8, ... and, for each, all bands, so that the rows neighbouring
// bands share are read through one L2.
template <bool AVG, int K, int IPT, int PG>
__global__ __launch_bounds__(kBandBlock, 3) void pool_band_kernel(
    const float* __restrict__ in, const float* __restrict__ map, float* __restrict__ out,
    int64_t* __restrict__ idx, int planes, int H, int W, int OW, int M, int R, int nbands,
    int chunks) {
  __shared__ __attribute__((aligned(16))) float lds[kBandLdsFloats];
  __shared__ int s_rows[2];
  const int t = threadIdx.x;
  const int xcd = blockIdx.x & 7, within = blockIdx.x >> 3;
  const int band = within % nbands;
  const int chunk = (within / nbands) * 8 + xcd;
  if (chunk >= chunks) return;
  const int p_begin = (int)((int64_t)chunk * planes / chunks);
  const int p_end = (int)((int64_t)(chunk + 1) * planes / chunks);
  const int pix0 = band * R * OW;
  const int npix = min(R * OW, M - pix0);
  const size_t HW = (size_t)H * W;

  if (t == 0) {
    s_rows[0] = INT_MAX;
    s_rows[1] = -1;
  }
  __syncthreads();
  int off[IPT][K];
  int rmin = INT_MAX, rmax = -1;
#pragma unroll
  for (int j = 0; j < IPT; ++j) {
    const int i = t + kBandBlock * j;
    const float2* coords = reinterpret_cast<const float2*>(map) + (size_t)(pix0 + min(i, npix - 1)) * K;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const float2 c = coords[k];
      PointTaps<float, 0> tp;
      tp.set(c.x, c.y, H, W);
      off[j][k] = i < npix ? tp.off[0] : -1;
      if (off[j][k] >= 0) {
        rmin = min(rmin, tp.ty[0]);
        rmax = max(rmax, tp.ty[0]);
      }
    }
  }
  if (rmax >= 0) {
    atomicMin(&s_rows[0], rmin);
    atomicMax(&s_rows[1], rmax);
  }
  __syncthreads();
  const int row0 = s_rows[0], row1 = s_rows[1];
  const int nrows = row1 < 0 ? 0 : row1 - row0 + 1;
  const int row_start = row1 < 0 ? 0 : row0 * W;      // W % 4 == 0: 16-byte aligned in every plane
  const int64_t band_elems = (int64_t)nrows * W;
  if (PG > 1 && (band_elems + 4) * PG <= kBandLdsFloats)
    run_band<AVG, K, IPT, PG>(in, out, idx, lds, off, pix0, npix, p_begin, p_end, HW, M, row_start,
                              (int)(band_elems / 4));
  else if (band_elems + 4 <= kBandLdsFloats)
    run_band<AVG, K, IPT, 1>(in, out, idx, lds, off, pix0, npix, p_begin, p_end, HW, M, row_start,
                             (int)(band_elems / 4));
  else
    run_direct<AVG, K, IPT>(in, out, idx, off, pix0, npix, p_begin, p_end, HW, M);
}

template <bool AVG, int K, int IPT>
void launch_band(const float* in, const float* map, float* out, int64_t* idx, int planes, int H,
                 int W, int OW, int M, int R, hipStream_t stream) {
  const int nbands = (int)ceil_div(M / OW, R);
  // about three workgroups per CU, every workgroup at least eight planes, chunks in eighths
  int chunks = (int)std::max<int64_t>(1, std::min<int64_t>(planes / 8, 768 / nbands));
  chunks = std::max(8, chunks / 8 * 8);
  chunks = (int)std::min<int64_t>(chunks, std::max<int64_t>(planes, 1));
  const unsigned grid = 8u * (unsigned)nbands * (unsigned)ceil_div(chunks, 8);
  launch(pool_band_kernel<AVG, K, IPT, 2>, dim3(grid), dim3(kBandBlock), stream, in, map, out, idx,
         planes, H, W, OW, M, R, nbands, chunks);
}

template <bool AVG, int K>
bool dispatch_ipt(int ipt, const float* in, const float* map, float* out, int64_t* idx, int planes,
                  int H, int W, int OW, int M, int R, hipStream_t stream) {
  switch (ipt) {
    case 1: launch_band<AVG, K, 1>(in, map, out, idx, planes, H, W, OW, M, R, stream); return true;
    case 2: launch_band<AVG, K, 2>(in, map, out, idx, planes, H, W, OW, M, R, stream); return true;
    case 3:
    case 4: launch_band<AVG, K, 4>(in, map, out, idx, planes, H, W, OW, M, R, stream); return true;
  }
  return false;
}

}  // namespace

bool pool_band_launch(bool avg, const float* in, const float* map, float* out, int64_t* idx,
                      int64_t planes, int H, int W, int OH, int OW, int K, hipStream_t stream) {
  // 16-byte row runs, few pooled pixels per thread, enough planes to amortise the tap decode
  if (W % 4 != 0 || ((uintptr_t)in & 15) != 0 || planes < 16 || OW > 1024) return false;
  if (K != 4 && K != 9) return false;
  // rows a band of R pooled rows is expected to touch: R strides plus a kernel's own height
  const int sy = (int)ceil_div(H, OH);
  int R = 0;
  for (int r : {8, 4, 2, 1}) {
    const int64_t rows = (int64_t)r * sy + 2 * sy + 1;
    if (ceil_div((int64_t)r * OW, kBandBlock) <= 4 && (rows * W + 4) <= kBandLdsFloats) {
      R = r;
      break;
    }
  }
  if (R == 0) return false;
  R = std::min(R, OH);
  const int ipt = (int)ceil_div((int64_t)R * OW, kBandBlock);
  const int M = OH * OW;
  if (K == 9)
    return avg ? dispatch_ipt<true, 9>(ipt, in, map, out, idx, (int)planes, H, W, OW, M, R, stream)
               : dispatch_ipt<false, 9>(ipt, in, map, out, idx, (int)planes, H, W, OW, M, R, stream);
  return avg ? dispatch_ipt<true, 4>(ipt, in, map, out, idx, (int)planes, H, W, OW, M, R, stream)
             : dispatch_ipt<false, 4>(ipt, in, map, out, idx, (int)planes, H, W, OW, M, R, stream);
}

}  // namespace sdk
