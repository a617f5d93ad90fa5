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


// ---------------------------------------------------------------------------
// Unpooling by image row bands (max: common/mapped_max_pool.h:60-78, :136-171; average:
// common/mapped_avg_pool.h:42-68, :107-140).  A workgroup owns RB whole image rows and a
// range of planes, sums what reaches those rows in LDS and stores every element once, 16 bytes
// at a time: no zero fill, no atomics in memory.  What can reach a band is fixed by the map:
// a table (built once per map by unpool_band_rows_kernel, kept in the caller's workspace or
// plan) holds per band the range of pooled rows with a tap in it.  A thread owns up to eight
// pooled pixels of that range (four in average unpooling); the positions of their K taps
// inside the band are worked out once, packed two to a register (in every workgroup, or once
// per map into the plan: unpool_band_taps_kernel), and serve every plane, so per plane a
// pooled pixel costs one index read, one gradient read, a select by the winning sample and
// one LDS add.
//
// table: [0] 1 when every band's range fits (kUbWindowPixels pooled pixels), else 0 (the
// caller then takes its other route); [3] 1 when the build looked for pooled pixels that have
// the same sample k at the same image pixel; [4] 1 when the packed taps behind the table are
// there; [8 + 2b] last pooled row of band b + 1 (0: nothing reaches it); [9 + 2b] kUbBig -
// first pooled row; [8 + 2 nbands + b] raised when two such pooled pixels meet in band b
// (where [3] is set and this is 0, average unpooling adds band b sample by sample without
// atomics).  All grow by atomicMax from a zero fill.
// ---------------------------------------------------------------------------
constexpr int kUbWindowPixels = 2048;   // pooled pixels a band's range may hold
constexpr int kUbLdsBytes = 32 * 1024;
constexpr int kUbLdsFloats = kUbLdsBytes / 4;
constexpr int kUbBig = 1 << 30;
constexpr unsigned kUbNone = 0xFFFFu;

// seen: nullptr, or one zeroed word per image pixel; bit k is set by the first pooled pixel
// whose sample k lands there, and a second one marks the band.
__global__ __launch_bounds__(kBandBlock) void unpool_band_rows_kernel(
    const float* __restrict__ map, int M, int OW, int K, int H, int W, int RB, int nbands,
    int* __restrict__ table, unsigned* __restrict__ seen) {
  const int pix = blockIdx.x * kBandBlock + threadIdx.x;
  if (pix == 0) table[3] = seen != nullptr ? 1 : 0;
  if (pix >= M) return;
  const int r = pix / OW;
  const float2* coords = reinterpret_cast<const float2*>(map) + (size_t)pix * K;
  int bmin = INT_MAX, bmax = -1;
  for (int k = 0; k < K; ++k) {
    const float2 c = coords[k];
    PointTaps<float, 0> tp;
    tp.set(c.x, c.y, H, W);
    if (tp.off[0] >= 0) {
      bmin = min(bmin, tp.ty[0] / RB);
      bmax = max(bmax, tp.ty[0] / RB);
      if (seen != nullptr) {
        const unsigned bit = 1u << k;
        if (atomicOr(seen + tp.off[0], bit) & bit)
          atomicMax(&table[8 + 2 * nbands + tp.ty[0] / RB], 1);
      }
    }
  }
  // every band between the first and the last one touched (a superset does no harm: a pooled
  // pixel of the range without a tap in the band adds nothing)
  for (int b = bmin; b <= bmax; ++b) {
    int* e = table + 8 + 2 * b;
    if (e[0] < r + 1) atomicMax(&e[0], r + 1);
    if (e[1] < kUbBig - r) atomicMax(&e[1], kUbBig - r);
  }
}

__global__ __launch_bounds__(kBandBlock) void unpool_band_verdict_kernel(int* __restrict__ table,
                                                                        int nbands, int OW) {
  __shared__ int bad;
  if (threadIdx.x == 0) bad = 0;
  __syncthreads();
  for (int b = threadIdx.x; b < nbands; b += kBandBlock) {
    const int hi1 = table[8 + 2 * b];
    if (hi1 > 0) {
      const int lo = kUbBig - table[9 + 2 * b];
      if ((int64_t)(hi1 - lo) * OW > kUbWindowPixels) bad = 1;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) table[0] = bad ? 0 : 1;
}

constexpr int kUbTapWords = 5;   // packed taps of a pooled pixel, K <= 9 (two to a word)

// Word h of a pooled pixel's packed taps: the positions inside the band (rows y0 .. y0 +
// band_rows - 1) of its samples 2h and 2h + 1, kUbNone for a sample outside the band or the
// image and where !on.  perm: the even columns of a band row in the row's first half, the odd
// ones in the second (average unpooling: the samples of a strided or dilated map land two
// columns apart, and a wave's adds would otherwise use half of the LDS banks).
__device__ __forceinline__ unsigned packed_tap_word(const float2* coords, int h, int K, int H,
                                                    int W, int y0, int band_rows, bool on,
                                                    bool perm) {
  unsigned half[2];
#pragma unroll
  for (int e = 0; e < 2; ++e) {
    const int k = 2 * h + e;
    half[e] = kUbNone;
    if (k < K) {
      const float2 c = coords[k];
      PointTaps<float, 0> tp;
      tp.set(c.x, c.y, H, W);
      const int ry = tp.ty[0] - y0;
      const int col = perm ? (tp.tx[0] >> 1) + (tp.tx[0] & 1) * (W >> 1) : tp.tx[0];
      if (on && tp.off[0] >= 0 && (unsigned)ry < (unsigned)band_rows)
        half[e] = (unsigned)(ry * W + col);
    }
  }
  return half[0] | (half[1] << 16);
}

// The packed taps of every band's pooled pixels, worked out once per map: taps[(band *
// kUbTapWords + h) * kUbWindowPixels + i] for pooled pixel i of the band's range.  grid =
// (kUbWindowPixels / 256, nbands).  Sets table[4] (read by the band kernel) when it has run.
__global__ __launch_bounds__(kBandBlock) void unpool_band_taps_kernel(
    const float* __restrict__ map, int* __restrict__ table, unsigned* __restrict__ taps, int K,
    int H, int W, int OW, int RB, int perm) {
  if (table[0] == 0) return;
  const int band = blockIdx.y;
  const int i = blockIdx.x * kBandBlock + threadIdx.x;
  if (band == 0 && i == 0) table[4] = 1;
  const int y0 = band * RB;
  const int band_rows = min(RB, H - y0);
  const int hi1 = table[8 + 2 * band];
  const int lo = hi1 > 0 ? kUbBig - table[9 + 2 * band] : 0;
  const int npw = hi1 > 0 ? (hi1 - lo) * OW : 0;
  const int pix = lo * OW + min(i, max(npw - 1, 0));
  const float2* coords = reinterpret_cast<const float2*>(map) + (size_t)pix * K;
  for (int h = 0; h < (K + 1) / 2; ++h)
    taps[((size_t)band * kUbTapWords + h) * kUbWindowPixels + i] =
        packed_tap_word(coords, h, K, H, W, y0, band_rows, i < npw, perm != 0);
}

// One 64-bit compare-and-swap loop that adds (a, b) to an aligned pair of floats in LDS.
__device__ __forceinline__ void lds_add_f32x2(float2* addr, float a, float b) {
  unsigned long long* ip = reinterpret_cast<unsigned long long*>(addr);
  unsigned long long old = __hip_atomic_load(ip, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  while (true) {
    const unsigned long long assumed = old;
    old = atomicCAS(ip, assumed, add_pair(assumed, a, b));
    if (old == assumed) break;
  }
}

// Piece v (four floats) of a band row run, past the caches; one 16-byte store where the
// tensor is 16-byte aligned (aligned: the same for every thread of the launch).
__device__ __forceinline__ void store_piece(float* dst, int v, vec4 val, int aligned) {
  if (aligned) {
    __builtin_nontemporal_store(val, reinterpret_cast<vec4*>(dst) + v);
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) __builtin_nontemporal_store(val[e], dst + 4 * v + e);
  }
}

// Tap k of a pooled pixel from its packed taps, by a chain of selects.  Each word passes
// through an empty asm first: seen as plain array elements, the compiler turns the chain into
// one load at a computed address and the whole array moves from registers to private memory.
template <int K>
__device__ __forceinline__ unsigned packed_tap(const unsigned (&offp)[(K + 1) / 2], int k) {
  unsigned w = offp[0];
  asm volatile("" : "+v"(w));
#pragma unroll
  for (int h = 1; h < (K + 1) / 2; ++h) {
    unsigned x = offp[h];
    asm volatile("" : "+v"(x));
    w = (k >> 1) == h ? x : w;
  }
  return (k & 1) ? (w >> 16) : (w & 0xFFFFu);
}

// gate: raised (and the caller's atomic route then redoes the call) when an index names a
// sample of another pooled pixel than its own, which mapped_max_pool never writes but the
// scatter accepts: such a sample may reach a band whose range does not hold the pixel.
//
// Two planes per pass.  The LDS adds are compare-and-swap loops (the native float add to LDS
// runs at a fraction of their rate on this GPU: 788 against 198 us for the average unpooling
// of an 8 x 64 x 128 x 256 gradient), one after the other (issued as a batch, with the taps
// outside the band masked or sent to a spare word, they were slower).  Max unpooling keeps
// the two planes apart (their winners differ); average unpooling interleaves them, (plane 0,
// plane 1) per band element, and adds both with one 64-bit swap per tap.  In a band where the table says that sample k of
// different pooled pixels never shares an image pixel, average unpooling needs no atomics at
// all: the samples are added one k at a time, a barrier between them, every lane reading,
// adding to and writing back elements no other lane touches in that round, with all of a
// thread's reads of a round in flight together; the sums then come in a fixed order.
template <bool AVG, int K>
__global__ __launch_bounds__(AVG ? 512 : 256, AVG ? 2 : 3) void unpool_band_kernel(
    const float* __restrict__ gout, const int64_t* __restrict__ idx, const float* __restrict__ map,
    float* __restrict__ gin, const int* __restrict__ table, const unsigned* __restrict__ taps,
    int* __restrict__ gate, int planes, int H, int W, int OW, int M, int RB, int nbands,
    int chunks, int map_elems, int aligned) {
  if (table[0] == 0) return;
  constexpr int PG = 2;
  // average unpooling: twice the threads with half the pooled pixels each (its sample-by-sample
  // rounds hold a pixel's sums in registers beside its taps)
  constexpr int BLK = AVG ? 512 : 256, IPT = kUbWindowPixels / BLK;
  constexpr bool PERM = AVG;   // packed_tap_word
  __shared__ __attribute__((aligned(16))) float acc[kUbLdsFloats];
  constexpr int KH = (K + 1) / 2;
  const int t = threadIdx.x;
  const int xcd = blockIdx.x & 7, within = blockIdx.x >> 3;
  const int band = within % nbands;
  const int chunk = (within / nbands) * 8 + xcd;
  if (chunk >= chunks) return;
  const int p_begin = (int)((int64_t)chunk * planes / chunks);
  const int p_end = (int)((int64_t)(chunk + 1) * planes / chunks);
  const size_t HW = (size_t)H * W;
  const int y0 = band * RB;
  const int band_rows = min(RB, H - y0);
  const int band_elems = band_rows * W;       // <= kUbLdsFloats / PG, W % 4 == 0
  const int n_vec = band_elems / 4;
  const int hi1 = table[8 + 2 * band];
  const int lo = hi1 > 0 ? kUbBig - table[9 + 2 * band] : 0;
  const int npw = hi1 > 0 ? (hi1 - lo) * OW : 0;   // pooled pixels that may reach the band
  const int pw0 = lo * OW;
  const bool ordered = AVG && table[3] != 0 && table[8 + 2 * nbands + band] == 0;

  // the packed taps of the thread's pooled pixels: from the plan where it holds them (one
  // read of neighbouring words per word), else worked out here from the map
  unsigned offp[IPT][KH];
  if (taps != nullptr && table[4] != 0) {
    const unsigned* mine = taps + (size_t)band * kUbTapWords * kUbWindowPixels;
#pragma unroll
    for (int j = 0; j < IPT; ++j)
#pragma unroll
      for (int h = 0; h < KH; ++h) offp[j][h] = mine[h * kUbWindowPixels + t + BLK * j];
  } else {
    const float2* map2 = reinterpret_cast<const float2*>(map);
#pragma unroll
    for (int j = 0; j < IPT; ++j) {
      const int i = t + BLK * j;
      const int pix = pw0 + min(i, max(npw - 1, 0));
#pragma unroll
      for (int h = 0; h < KH; ++h)
        offp[j][h] = packed_tap_word(map2 + (size_t)pix * K, h, K, H, W, y0, band_rows, i < npw,
                                     PERM);
    }
  }
  vec4* acc4 = reinterpret_cast<vec4*>(acc);
  for (int v = t; v < PG * n_vec; v += BLK) acc4[v] = vec4{0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  // Stores the band sums of the planes q, q + 1 (the second only below p_end) and clears them.
  auto store_pass = [&](int q) {
    for (int v = t; v < n_vec; v += BLK) {
      vec4 a, b;
      if constexpr (AVG) {
        // (p0, p1) of two columns each: c, c + 1 and c + 2, c + 3, or with PERM c, c + 2 and
        // c + 1, c + 3
        const int ia = PERM ? (v / (W >> 2)) * (W >> 1) + v % (W >> 2) : 2 * v;
        const int ib = PERM ? ia + (W >> 2) : 2 * v + 1;
        const vec4 lo4 = acc4[ia], hi4 = acc4[ib];
        acc4[ia] = vec4{0.f, 0.f, 0.f, 0.f};
        acc4[ib] = vec4{0.f, 0.f, 0.f, 0.f};
        if constexpr (PERM) {
          a = vec4{lo4[0], hi4[0], lo4[2], hi4[2]} / float(K);
          b = vec4{lo4[1], hi4[1], lo4[3], hi4[3]} / float(K);
        } else {
          a = vec4{lo4[0], lo4[2], hi4[0], hi4[2]} / float(K);
          b = vec4{lo4[1], lo4[3], hi4[1], hi4[3]} / float(K);
        }
      } else {
        a = acc4[v];
        b = acc4[n_vec + v];
        acc4[v] = vec4{0.f, 0.f, 0.f, 0.f};
        acc4[n_vec + v] = vec4{0.f, 0.f, 0.f, 0.f};
      }
      store_piece(gin + (size_t)q * HW + (size_t)y0 * W, v, a, aligned);
      if (q + 1 < p_end) store_piece(gin + (size_t)(q + 1) * HW + (size_t)y0 * W, v, b, aligned);
    }
  };

  bool stray = false;
  for (int p = p_begin; p < p_end; p += PG) {
    // this pass's indices and gradients are requested first; the previous pass is stored
    // while they are on their way
    int64_t sv[IPT][PG];
    float gv[IPT][PG];
#pragma unroll
    for (int j = 0; j < IPT; ++j) {
      const int i = t + BLK * j;
      const size_t at = (size_t)pw0 + min(i, max(npw - 1, 0));
#pragma unroll
      for (int g = 0; g < PG; ++g) {
        const size_t e = (size_t)min(p + g, p_end - 1) * M + at;
        if constexpr (!AVG) sv[j][g] = idx[e];
        gv[j][g] = gout[e];
      }
    }
    if (p > p_begin) {
      store_pass(p - PG);
      __syncthreads();
    }
    const bool two = p + 1 < p_end;
    if (AVG && ordered) {
      float2* acc2 = reinterpret_cast<float2*>(acc);
#pragma unroll
      for (int k = 0; k < K; ++k) {
        unsigned o[IPT];
        float2 cur[IPT];
#pragma unroll
        for (int j = 0; j < IPT; ++j) {
          o[j] = (offp[j][k >> 1] >> ((k & 1) * 16)) & 0xFFFFu;   // kUbNone for i >= npw too
          cur[j] = float2{0.0f, 0.0f};
          if (o[j] != kUbNone) cur[j] = acc2[o[j]];
        }
#pragma unroll
        for (int j = 0; j < IPT; ++j)
          if (o[j] != kUbNone)
            acc2[o[j]] = float2{cur[j].x + gv[j][0], cur[j].y + (two ? gv[j][1] : 0.0f)};
        __syncthreads();
      }
    } else {
#pragma unroll
      for (int j = 0; j < IPT; ++j) {
        const int i = t + BLK * j;
        if (i >= npw) continue;
        if constexpr (AVG) {
          float2* acc2 = reinterpret_cast<float2*>(acc);
          const float gb = two ? gv[j][1] : 0.0f;
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const unsigned o16 = (offp[j][k >> 1] >> ((k & 1) * 16)) & 0xFFFFu;
            if (o16 != kUbNone) lds_add_f32x2(acc2 + o16, gv[j][0], gb);
          }
        } else {
          const int first = (pw0 + i) * K * 2;   // map element of the pixel's first sample
#pragma unroll
          for (int g = 0; g < PG; ++g) {
            if (g == 1 && !two) continue;
            const int64_t s64 = sv[j][g];
            const bool live = s64 >= 0 && s64 + 2 <= (int64_t)map_elems;   // others add nothing
            const int d = (int)s64 - first;
            const bool mine = d >= 0 && d < 2 * K && (d & 1) == 0;
            stray |= live && !mine;
            if (live && mine) {
              const unsigned o16 = packed_tap<K>(offp[j], d >> 1);
              if (o16 != kUbNone) lds_add_f32(acc + g * band_elems + o16, gv[j][g]);
            }
          }
        }
      }
      __syncthreads();
    }
  }
  store_pass(p_begin + (p_end - p_begin - 1) / PG * PG);   // the last pass
  if (stray) atomicAdd(gate, 1);
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

// Image rows per unpooling band: two planes of RB rows in the 32 KB of a workgroup's sums.
static int unpool_band_rows_per_band(int W) {
  if (W % 4 != 0) return 0;
  for (int rb : {16, 8, 4, 2, 1})
    if ((int64_t)rb * W * 2 <= kUbLdsFloats) return rb;
  return 0;
}

bool unpool_band_shape(int H, int W, int OH, int OW, int K) {
  return unpool_band_rows_per_band(W) > 0 && (K == 4 || K == 9) &&
         (int64_t)OH * OW * K * 2 < ((int64_t)1 << 31);
}

size_t unpool_band_taps_bytes(int H, int W) {
  const int rb = unpool_band_rows_per_band(W);
  const int64_t nbands = rb > 0 ? ceil_div(H, rb) : 0;
  const int64_t bytes = nbands * kUbTapWords * kUbWindowPixels * (int64_t)sizeof(unsigned);
  return bytes <= ((int64_t)32 << 20) ? (size_t)bytes : 0;
}

size_t unpool_band_table_bytes(int H, int W) {
  const int rb = unpool_band_rows_per_band(W);
  const int64_t nbands = rb > 0 ? ceil_div(H, rb) : 0;
  return (size_t)(8 + 3 * nbands) * sizeof(int);   // the verdict word is there for every plane
}

void unpool_band_build(const float* map, int* table, int H, int W, int OH, int OW, int K,
                       hipStream_t stream, unsigned* seen, unsigned* taps, bool perm) {
  const int rb = unpool_band_rows_per_band(W);
  const int M = OH * OW;
  launch(unpool_band_rows_kernel, dim3((unsigned)ceil_div(M, kBandBlock)), dim3(kBandBlock), stream,
         map, M, OW, K, H, W, rb, (int)ceil_div(H, rb), table, seen);
  launch(unpool_band_verdict_kernel, dim3(1), dim3(kBandBlock), stream, table,
         (int)ceil_div(H, rb), OW);
  if (taps != nullptr)
    launch(unpool_band_taps_kernel, dim3(kUbWindowPixels / kBandBlock, (unsigned)ceil_div(H, rb)),
           dim3(kBandBlock), stream, map, table, taps, K, H, W, OW, rb, perm ? 1 : 0);
}

void unpool_band_launch(bool avg, const float* gout, const int64_t* idx, const float* map,
                        float* gin, const int* table, const unsigned* taps, int* gate,
                        int64_t planes, int H, int W, int OH, int OW, int K, hipStream_t stream) {
  const int rb = unpool_band_rows_per_band(W);
  const int nbands = (int)ceil_div(H, rb);
  // one round of resident workgroups (three of 256 threads per CU for max unpooling, two of
  // 512 for average unpooling: as many as their registers allow), chunks in eighths (one per
  // XCD), at least two planes each
  int chunks = (int)std::max<int64_t>(1, std::min<int64_t>(planes / 2, (avg ? 512 : 768) / nbands));
  chunks = std::max(8, chunks / 8 * 8);
  chunks = (int)std::min<int64_t>(chunks, planes);
  const unsigned grid = 8u * (unsigned)nbands * (unsigned)ceil_div(chunks, 8);
  const int M = OH * OW;
#define UB(AVGv, Kv)                                                                        \
  launch(unpool_band_kernel<AVGv, Kv>, dim3(grid), dim3(AVGv ? 512 : 256), stream, gout, idx, \
         map, gin, table, taps, gate, (int)planes, H, W, OW, M, rb, nbands, chunks, M * K * 2, \
         ((uintptr_t)gin & 15) == 0 ? 1 : 0)
  if (K == 9) {
    if (avg) UB(true, 9); else UB(false, 9);
  } else {
    if (avg) UB(true, 4); else UB(false, 4);
  }
#undef UB
}

}  // namespace sdk
