// Memory-bound mapped gather / scatter kernels for gfx950 and their C entry
// points: resample_from_map / resample_to_map, mapped im2col / col2im, mapped
// max pool / unpool.
//
// Common shape of every kernel: one thread owns one map pixel (lanes of a
// wavefront own consecutive pixels, so sample-map reads, value reads and value
// writes are contiguous across the wave) and applies the pixel's taps to a
// chunk of PC image planes held in registers, so the tap arithmetic and the
// map traffic are amortised over PC planes and PC independent loads are in
// flight per lane.  grid.x walks pixels, grid.y walks plane chunks.
#include <hip/hip_runtime.h>

#include <mutex>

#include <cfloat>
#include <climits>

#include "conv_product.hpp"
#include "pool_band.hpp"
#include "sdk_host.hpp"
#include "sdk_lane_runs.hpp"
#include "sdk_taps.hpp"

namespace sdk {

constexpr int kBlock = 256;  // 4 wavefronts
constexpr int kPC = 8;       // planes per thread

// Pixel block of this workgroup.  Workgroup ids go round-robin over the 8 XCDs, each with
// its own L2; grid.x is 8 * per_xcd and XCD x walks the contiguous band of pixel blocks
// [x * per_xcd, (x + 1) * per_xcd) in order, so neighbouring map rows, which read the same
// image rows, meet in one L2 shortly after each other.  Blocks past the last pixel do nothing.
__device__ __forceinline__ int banded_pixel_block() {
  const int per_xcd = gridDim.x >> 3;
  return (blockIdx.x & 7) * per_xcd + (blockIdx.x >> 3);
}
inline unsigned banded_grid_x(int64_t pixels) {
  return 8u * (unsigned)ceil_div(ceil_div(pixels, kBlock), 8);
}

// ---------------------------------------------------------------------------
// Fill kernels (scatter targets start from zero; hipMemsetAsync is avoided so
// that callers may capture these entry points into a HIP graph).
// ---------------------------------------------------------------------------
// gate: optional device flag; a gated kernel runs only if *gate != 0.
template <typename T>
__global__ __launch_bounds__(kBlock) void fill_kernel(T* __restrict__ p, size_t n, T v,
                                                      const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += stride) p[i] = v;
}

// 16-byte stores for the bulk of a zero fill.
__global__ __launch_bounds__(kBlock) void zero16_kernel(uint4* __restrict__ p, size_t n16,
                                                        const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const size_t stride = (size_t)gridDim.x * kBlock;
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n16; i += stride) p[i] = z;
}

// Three buffers in one launch (the targets of a small layer's combined backward, where a launch
// costs as much as the kernel it starts): 16-byte stores for the bulk of each, words for the rest.
struct ZeroSeg {
  unsigned* p;
  size_t words;
};
__global__ __launch_bounds__(kBlock) void zero3_kernel(ZeroSeg s0, ZeroSeg s1, ZeroSeg s2) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x;
  const ZeroSeg segs[3] = {s0, s1, s2};
#pragma unroll
  for (int k = 0; k < 3; ++k) {
    const size_t n16 = (reinterpret_cast<uintptr_t>(segs[k].p) % 16 == 0) ? segs[k].words / 4 : 0;
    uint4* p16 = reinterpret_cast<uint4*>(segs[k].p);
    for (size_t i = first; i < n16; i += stride) p16[i] = make_uint4(0, 0, 0, 0);
    for (size_t i = n16 * 4 + first; i < segs[k].words; i += stride) segs[k].p[i] = 0u;
  }
}

int zero_fill3(void* a, size_t a_bytes, void* b, size_t b_bytes, void* c, size_t c_bytes,
               hipStream_t stream) {
  const size_t most = std::max(a_bytes, std::max(b_bytes, c_bytes));
  if (most == 0) return SDK_OK;
  const int blocks = (int)std::min<size_t>(ceil_div((int64_t)(most / 16 + 1), kBlock), 256 * 16);
  launch(zero3_kernel, dim3(blocks), dim3(kBlock), stream, ZeroSeg{(unsigned*)a, a_bytes / 4},
         ZeroSeg{(unsigned*)b, b_bytes / 4}, ZeroSeg{(unsigned*)c, c_bytes / 4});
  SDK_LAUNCH_CHECK("zero_fill3");
  return SDK_OK;
}

int zero_fill_gated(void* ptr, size_t bytes, hipStream_t stream, const int* gate);
int zero_fill(void* ptr, size_t bytes, hipStream_t stream) {
  return zero_fill_gated(ptr, bytes, stream, nullptr);
}
int zero_fill_gated(void* ptr, size_t bytes, hipStream_t stream, const int* gate) {
  if (bytes == 0) return SDK_OK;
  // ptr comes from a framework allocator (>= 256-byte aligned) and all element
  // sizes divide 16, so only a tail of < 16 bytes needs the scalar kernel.
  const size_t n16 = ((uintptr_t)ptr % 16 == 0) ? bytes / 16 : 0;
  if (n16) {
    const int blocks = (int)std::min<size_t>(ceil_div((int64_t)n16, kBlock), 256 * 16);
    launch(zero16_kernel, dim3(blocks), dim3(kBlock), stream, (uint4*)ptr, n16, gate);
  }
  const size_t done = n16 * 16;
  if (done < bytes) {
    const size_t rest = bytes - done;
    const int blocks = (int)std::min<size_t>(ceil_div((int64_t)rest, kBlock), 256 * 16);
    launch(fill_kernel<unsigned char>, dim3(blocks), dim3(kBlock), stream,
                       (unsigned char*)ptr + done, rest, (unsigned char)0, gate);
  }
  SDK_LAUNCH_CHECK("zero_fill");
  return SDK_OK;
}

// ---------------------------------------------------------------------------
// resample_from_map (gather).  Body: ext_modules/include/common/resample.h:34-52,
// :85-107.  planes = B*C; image plane stride HW; out plane stride MP.
// ---------------------------------------------------------------------------
// PC planes per thread: 8 when there are many planes, fewer for small batches so that the grid
// still fills the GPU and no lane idles on planes that do not exist.
inline int planes_per_thread(int64_t planes) { return planes >= 32 ? 8 : (planes > 8 ? 4 : 2); }
// ... of the gather: 2 below 16 planes (12 planes at configuration 2: 17.7 us with 2, 19.7 with
// 4, 21.8 with 8; a wave's reads of a polar patch touch 30 to 40 lines per plane and row, and
// with fewer planes in flight the rows of neighbouring waves still find each other's lines in
// the vector cache)
inline int gather_planes_per_thread(int64_t planes) {
  return planes >= 32 ? 8 : (planes >= 16 ? 4 : 2);
}

template <typename T, int INTERP, bool WEIGHTED, int PC>
__global__ __launch_bounds__(kBlock) void resample_from_map_kernel(
    const T* __restrict__ image, const T* __restrict__ map, const T* __restrict__ wts,
    T* __restrict__ out, int planes, int H, int W, int MP, int P) {
  // (pixel blocks in launch order, dealt round-robin to the XCDs: with contiguous bands of
  // blocks per XCD the tangent-patch gather takes 24.5 instead of 21 us, the polar patches,
  // whose reads are the slowest, all landing on two XCDs)
  const int pix = blockIdx.x * kBlock + threadIdx.x;
  if (pix >= MP) return;
  const int plane0 = blockIdx.y * PC;
  const int np = min(PC, planes - plane0);
  const size_t HW = (size_t)H * W;
  const int q = WEIGHTED ? P : 1;
  T acc[PC];
  if constexpr (INTERP != 0 && !WEIGHTED) {
    // The two taps of an image row are neighbours in memory: one read of two elements (from
    // any element boundary) fetches both, which halves the read instructions and, where
    // neighbouring lanes lie about two pixels apart and the reads are bound by the requests
    // the vector cache takes per cycle, the time with them.  The pair starts at column
    // clamp(x1, 0, W - 2); a tap takes the element of its own column from it.  Only the
    // wrapped neighbour of the last column (bispherical) is not in its pair and is read on its
    // own.  The blend is PointTaps::blend, on the same values.
    if (W >= 2) {
      PointTaps<T, INTERP> t;
      t.set(map[(size_t)pix * 2], map[(size_t)pix * 2 + 1], H, W);
      typedef T pair_t __attribute__((ext_vector_type(2)));
      const int cb = min(max(t.tx[0], 0), W - 2);
      const int r1 = min(max(t.ty[0], 0), H - 1), r2 = min(max(t.ty[2], 0), H - 1);
      const size_t o1 = (size_t)r1 * W + cb, o2 = (size_t)r2 * W + cb;
      const bool wrapped = INTERP == 2 && t.tx[1] != t.tx[0] + 1;   // x1 = W - 1, x2 = 0
      const T* base = image + (size_t)plane0 * HW;
      pair_t top[PC], bot[PC];
      T wrap_top[PC], wrap_bot[PC];
#pragma unroll
      for (int j = 0; j < PC; ++j) {
        const T* plane = base + (size_t)(j < np ? j : 0) * HW;
        __builtin_memcpy(&top[j], plane + o1, sizeof(pair_t));   // (element alignment only)
        __builtin_memcpy(&bot[j], plane + o2, sizeof(pair_t));
      }
      if (__any(wrapped)) {
#pragma unroll
        for (int j = 0; j < PC; ++j) {
          const T* plane = base + (size_t)(j < np ? j : 0) * HW;
          wrap_top[j] = plane[(size_t)r1 * W];
          wrap_bot[j] = plane[(size_t)r2 * W];
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      const bool first0 = t.tx[0] == cb, first1 = t.tx[1] == cb;
#pragma unroll
      for (int j = 0; j < PC; ++j) {
        T raw[4];
        raw[0] = first0 ? top[j].x : top[j].y;
        raw[2] = first0 ? bot[j].x : bot[j].y;
        raw[1] = wrapped ? wrap_top[j] : (first1 ? top[j].x : top[j].y);
        raw[3] = wrapped ? wrap_bot[j] : (first1 ? bot[j].x : bot[j].y);
        acc[j] = j < np ? t.blend(raw) : T(0);
      }
    } else {
      gather_sample<T, INTERP, WEIGHTED, PC>(image + (size_t)plane0 * HW, HW, np,
                                             map + (size_t)pix * 2, nullptr, P, H, W, acc);
    }
  } else {
    gather_sample<T, INTERP, WEIGHTED, PC>(image + (size_t)plane0 * HW, HW, np,
                                           map + (size_t)pix * q * 2,
                                           WEIGHTED ? wts + (size_t)pix * q : nullptr, P, H, W,
                                           acc);
  }
#pragma unroll
  for (int j = 0; j < PC; ++j)
    if (j < np) out[(size_t)(plane0 + j) * MP + pix] = acc[j];
}

// ---------------------------------------------------------------------------
// resample_to_map (scatter).  Body: common/resample.h:11-31, :55-82.
// ONES: the input is an implicit all-ones plane (weight-sum pass).
// ---------------------------------------------------------------------------
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void resample_to_map_kernel(
    const T* __restrict__ in, const T* __restrict__ map, const T* __restrict__ wts,
    T* __restrict__ out, T* __restrict__ wsum, int planes, int H, int W, int MP, int P,
    const int* __restrict__ gate, int group) {
  if (gate != nullptr && *gate == 0) return;
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= MP) return;
  const size_t HW = (size_t)H * W;
  const int q = WEIGHTED ? P : 1;
  const T* coords = map + (size_t)pix * q * 2;
  const T* pw = WEIGHTED ? wts + (size_t)pix * q : nullptr;
  const int chunks = (planes + kPC - 1) / kPC;
  if ((int)blockIdx.y >= chunks) {   // the extra row of the grid: the weight-sum plane
    const T one[1] = {T(1)};
    scatter_sample<T, INTERP, WEIGHTED, 1>(wsum, 0, 1, coords, pw, P, H, W, one);
    return;
  }
  const int plane0 = blockIdx.y * kPC;
  const int np = min(kPC, planes - plane0);
  // group > 1 (average unpooling): `group` consecutive map entries are the samples of one
  // source pixel, each of which receives the pixel's value divided by `group`
  const int src = group > 1 ? pix / group : pix;
  const size_t in_plane = group > 1 ? (size_t)(MP / group) : (size_t)MP;
  T val[kPC];
#pragma unroll
  for (int j = 0; j < kPC; ++j) {
    val[j] = j < np ? in[(size_t)(plane0 + j) * in_plane + src] : T(0);
    if (group > 1) val[j] = val[j] / T(group);
  }
  scatter_sample<T, INTERP, WEIGHTED, kPC>(out + (size_t)plane0 * HW, HW, np, coords, pw, P, H, W,
                                           val);
}

// Zero fill of two buffers in one launch (16-byte aligned, sizes in 16-byte units).
__global__ __launch_bounds__(kBlock) void zero16_pair_kernel(uint4* __restrict__ a, size_t na,
                                                             uint4* __restrict__ b, size_t nb,
                                                             const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const size_t stride = (size_t)gridDim.x * kBlock;
  const uint4 z = make_uint4(0, 0, 0, 0);
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < na + nb; i += stride) {
    if (i < na) a[i] = z;
    else b[i - na] = z;
  }
}

// ---------------------------------------------------------------------------
// resample_to_map as a gather over the inverted map.  inverse_fill: one thread per map
// pixel appends (pixel, tap weight) to the list of every image pixel its taps hit
// (slot = atomic counter per target; lists are [slot][target], kInvSlots long); taps that
// find their list full raise *gate, which switches the call to the atomic scatter above.
// inverse_gather: one thread per image pixel and 8 planes sums its list.
// ---------------------------------------------------------------------------
constexpr int kInvSlots = 16;

template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void resample_inverse_fill_kernel(
    const T* __restrict__ map, const T* __restrict__ wts, int H, int W, int MP, int P,
    int* __restrict__ cnt, int* __restrict__ src, T* __restrict__ co, int* __restrict__ gate,
    int group, const int* __restrict__ only_if) {
  if (only_if != nullptr && *only_if == 0) return;   // the lists are not needed
  const int pix = blockIdx.x * kBlock + threadIdx.x;
  if (pix >= MP) return;
  const int q = WEIGHTED ? P : 1;
  const size_t HW = (size_t)H * W;
  // group > 1 (average unpooling): `group` consecutive map entries are the samples of one
  // source pixel; the lists name that pixel
  const int source = group > 1 ? pix / group : pix;
  PointTaps<T, INTERP> t;
  for (int p = 0; p < q; ++p) {
    const size_t s = (size_t)pix * q + p;
    t.set(map[s * 2], map[s * 2 + 1], H, W);
    const T wt = WEIGHTED ? wts[s] : T(1);
#pragma unroll
    for (int i = 0; i < PointTaps<T, INTERP>::N; ++i) {
      if (t.off[i] >= 0) {
        const int u = t.off[i];
        const int slot = atomicAdd(&cnt[u], 1);
        if (slot < kInvSlots) {
          src[(size_t)slot * HW + u] = source;
          co[(size_t)slot * HW + u] = INTERP == 0 ? wt : t.w[i] * wt;
        } else {
          atomicAdd(gate, 1);
        }
      }
    }
  }
}

// Sorts every target's list by source (then by coefficient bits), in place.  The fill appends
// in the order its atomics are served, so entry s of neighbouring targets names unrelated
// sources; sorted, neighbouring targets read neighbouring sources with the same instruction
// (fewer cache lines per read), and the sum of a target no longer depends on scheduling.
// One thread per target; lists are short (kInvSlots at most): selection sort on global memory.
template <typename T>
__global__ __launch_bounds__(kBlock) void resample_inverse_sort_kernel(
    const int* __restrict__ cnt, int* __restrict__ src, T* __restrict__ co, int HW,
    const int* __restrict__ gate, const int* __restrict__ only_if) {
  if (only_if != nullptr && *only_if == 0) return;
  if (*gate != 0) return;   // some list overflowed: the call scatters instead
  const int u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= HW) return;
  const int n = min(cnt[u], kInvSlots);
  for (int i = 0; i + 1 < n; ++i) {
    int best = i, bs = src[(size_t)i * HW + u];
    T bc = co[(size_t)i * HW + u];
    const int first_s = bs;
    const T first_c = bc;
    for (int j = i + 1; j < n; ++j) {
      const int sj = src[(size_t)j * HW + u];
      const T cj = co[(size_t)j * HW + u];
      if (sj < bs || (sj == bs && cj < bc)) {
        best = j;
        bs = sj;
        bc = cj;
      }
    }
    if (best != i) {
      src[(size_t)best * HW + u] = first_s;
      co[(size_t)best * HW + u] = first_c;
      src[(size_t)i * HW + u] = bs;
      co[(size_t)i * HW + u] = bc;
    }
  }
}

template <typename T, int PC>
__global__ __launch_bounds__(kBlock) void resample_inverse_gather_kernel(
    const T* __restrict__ in, const int* __restrict__ cnt, const int* __restrict__ src,
    const T* __restrict__ co, T* __restrict__ out, T* __restrict__ wsum, int planes, int HW,
    int MP, const int* __restrict__ gate, int normalize, T eps, int group,
    const int* __restrict__ skip) {
  if (skip != nullptr && *skip != 0) return;   // the tiled kernel has written the output
  if (*gate != 0) return;
  const int u = banded_pixel_block() * kBlock + threadIdx.x;
  if (u >= HW) return;
  const int plane0 = blockIdx.y * PC;
  const size_t in_plane = group > 1 ? (size_t)(MP / group) : (size_t)MP;
  const int np = min(PC, planes - plane0);
  const int n = min(cnt[u], kInvSlots);
  T acc[PC];
#pragma unroll
  for (int j = 0; j < PC; ++j) acc[j] = T(0);
  T wtot = T(0);
  // List entries in batches of four: the four (source, coefficient) reads of a lane are in
  // flight together, then its 4 * PC value reads, so a wave pays two round trips per batch
  // instead of two per entry (a wave runs as long as its longest list).  Entries past a
  // lane's own count are read from their slot all the same (the slot exists, its content is
  // not used) and select a zero contribution; the sum keeps the ascending entry order.
  for (int s0 = 0; __any(s0 < n); s0 += 4) {
    int m[4];
    T c[4];
    bool on[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      on[i] = s0 + i < n;
      const size_t at = (size_t)min(s0 + i, kInvSlots - 1) * HW + u;
      m[i] = src[at];
      c[i] = co[at];
    }
    T v[4][PC];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const size_t mi = on[i] ? (size_t)m[i] : 0;
#pragma unroll
      for (int j = 0; j < PC; ++j) v[i][j] = in[(size_t)(plane0 + (j < np ? j : 0)) * in_plane + mi];
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      wtot += on[i] ? c[i] : T(0);
#pragma unroll
      for (int j = 0; j < PC; ++j) acc[j] += on[i] ? c[i] * v[i][j] : T(0);
    }
  }
  // average unpooling hands every sample value / group: divided once here, after the sum
  if (group > 1) {
#pragma unroll
    for (int j = 0; j < PC; ++j) acc[j] = acc[j] / T(group);
  }
  // normalised: the weight sum of the pixel is the sum of its list, no second pass needed
  const T den = wtot + eps;
#pragma unroll
  for (int j = 0; j < PC; ++j)
    if (j < np) out[(size_t)(plane0 + j) * HW + u] = normalize ? acc[j] / den : acc[j];
  if (wsum != nullptr && blockIdx.y == 0) wsum[u] = wtot;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void normalize_kernel(T* __restrict__ data,
                                                           const T* __restrict__ wsum, T eps,
                                                           size_t plane_size, size_t total,
                                                           const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride)
    data[i] = data[i] / (wsum[i % plane_size] + eps);
}

// ---------------------------------------------------------------------------
// UV resampling: every pixel of the image names one of NT textures (quad) and a point (u, v) in
// that texture's TH x TW plane; taps never leave the named texture.  Bodies:
// common/resample.h:132-158 (gather), :160-187 (its adjoint).  A texture index outside
// [0, NT) contributes nothing (the reference reads out of bounds there).
// ---------------------------------------------------------------------------
template <typename T, int INTERP, int PC>
__global__ __launch_bounds__(kBlock) void uv_gather_kernel(
    const T* __restrict__ textures, const int64_t* __restrict__ quad, const T* __restrict__ uv,
    T* __restrict__ out, int planes, int NT, int TH, int TW, int MP) {
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= MP) return;
  const int plane0 = blockIdx.y * PC;
  const int np = min(PC, planes - plane0);
  const size_t THW = (size_t)TH * TW, stride = THW * NT;
  const long long q = quad[pix];
  T acc[PC];
  if (q >= 0 && q < NT) {
    gather_sample<T, INTERP, false, PC>(textures + (size_t)plane0 * stride + (size_t)q * THW,
                                        stride, np, uv + (size_t)pix * 2, nullptr, 0, TH, TW, acc);
  } else {
#pragma unroll
    for (int j = 0; j < PC; ++j) acc[j] = T(0);
  }
#pragma unroll
  for (int j = 0; j < PC; ++j)
    if (j < np) out[(size_t)(plane0 + j) * MP + pix] = acc[j];
}

template <typename T, int INTERP>
__global__ __launch_bounds__(kBlock) void uv_scatter_kernel(
    const T* __restrict__ in, const int64_t* __restrict__ quad, const T* __restrict__ uv,
    T* __restrict__ textures, int planes, int NT, int TH, int TW, int MP,
    const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= MP) return;
  const long long q = quad[pix];
  if (q < 0 || q >= NT) return;
  const int plane0 = blockIdx.y * kPC;
  const int np = min(kPC, planes - plane0);
  const size_t THW = (size_t)TH * TW, stride = THW * NT;
  T val[kPC];
#pragma unroll
  for (int j = 0; j < kPC; ++j) val[j] = j < np ? in[(size_t)(plane0 + j) * MP + pix] : T(0);
  scatter_sample<T, INTERP, false, kPC>(textures + (size_t)plane0 * stride + (size_t)q * THW,
                                        stride, np, uv + (size_t)pix * 2, nullptr, 0, TH, TW, val);
}

// ---------------------------------------------------------------------------
// The adjoint by texture.  A texture is small (TH x TW texels fit in LDS) and receives many
// image pixels per texel, often hundreds near the poles of an equirectangular image, so neither
// atomics in memory nor a bounded inverse list suit it.  Instead the image pixels are bucketed
// by texture (count, scan, fill: a counting sort of pixel indices, keyed by quad), and one
// workgroup per (texture, plane chunk) sums its bucket into an LDS copy of the texture and
// writes that out with plain stores, zeros included, so no fill of the output is needed.
//
// Lanes own consecutive bucket entries, which are consecutive image pixels of one row wherever
// the map is coherent; these hit the same texel in runs.  Each run is summed across lanes first
// (segmented scan over shuffles) and only its last lane adds to LDS, which keeps the
// compare-and-swap adds nearly free of collisions.
// ---------------------------------------------------------------------------
constexpr int kUvMaxTextures = 1 << 20;
constexpr int kUvLdsBytes = 64 * 1024;

// count / cursor are kept in R copies ([R][NT]; a workgroup uses copy blockIdx % R), so that
// neighbouring workgroups, which mostly see the same texture, do not queue on one address.
// A texture's bucket is the concatenation of its R parts.
__global__ __launch_bounds__(kBlock) void uv_count_kernel(const int64_t* __restrict__ quad,
                                                          int NT, int MP, int R,
                                                          int* __restrict__ count) {
  const int pix = blockIdx.x * kBlock + threadIdx.x;
  const long long q = pix < MP ? quad[pix] : -1;
  const bool ok = q >= 0 && q < NT;
  const int t = ok ? (int)q : -1;
  const int below = __shfl_up(t, 1);
  const LaneRuns runs(below == t);
  if (ok && runs.tail) atomicAdd(&count[(size_t)(blockIdx.x % R) * NT + t], runs.dist + 1);
}

// Exclusive scan in bucket order (texture-major, copy-minor): cursor[r][t] = first slot of part
// r of texture t; offset[t] = first slot of texture t, offset[NT] = number of pixels listed.
// One workgroup; every thread owns a contiguous strip of the NT * R counters, so the counters
// are read in one sweep of independent loads.
__global__ __launch_bounds__(kBlock) void uv_scan_kernel(const int* __restrict__ count, int NT,
                                                         int R, int* __restrict__ offset,
                                                         int* __restrict__ cursor) {
  __shared__ int wave_total[kBlock / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n = NT * R;
  const int strip = (n + kBlock - 1) / kBlock;
  const int first = threadIdx.x * strip, last = min(n, first + strip);
  int mine = 0;
  for (int i = first; i < last; ++i) mine += count[(size_t)(i % R) * NT + i / R];
  int incl = mine;
  for (int d = 1; d < 64; d <<= 1) {
    const int below = __shfl_up(incl, d);
    if (lane >= d) incl += below;
  }
  if (lane == 63) wave_total[wave] = incl;
  __syncthreads();
  int run = incl - mine;
  for (int w = 0; w < wave; ++w) run += wave_total[w];
  for (int i = first; i < last; ++i) {
    const int t = i / R, r = i - t * R;
    cursor[(size_t)r * NT + t] = run;
    if (r == 0) offset[t] = run;
    run += count[(size_t)r * NT + t];
  }
  if (threadIdx.x == kBlock - 1) offset[NT] = run;
}

__global__ __launch_bounds__(kBlock) void uv_fill_kernel(const int64_t* __restrict__ quad, int NT,
                                                         int MP, int R, int* __restrict__ cursor,
                                                         int* __restrict__ list) {
  const int pix = blockIdx.x * kBlock + threadIdx.x;
  const long long q = pix < MP ? quad[pix] : -1;
  const bool ok = q >= 0 && q < NT;
  const int t = ok ? (int)q : -1;
  const int below = __shfl_up(t, 1);
  const LaneRuns runs(below == t);
  // the last lane of a run reserves the run's slots; the others read the start from it
  int start = 0;
  if (ok && runs.tail)
    start = atomicAdd(&cursor[(size_t)(blockIdx.x % R) * NT + t], runs.dist + 1);
  const int lane = threadIdx.x & 63;
  const unsigned long long tails = __ballot(runs.tail);
  const int tail_lane = __ffsll((long long)(tails & (~0ull << lane))) - 1;
  start = __shfl(start, tail_lane);
  if (ok) list[start + runs.dist] = pix;
}

constexpr int kUvBlock = 1024;   // 16 waves: a long bucket (a polar face) takes few rounds

template <typename T, int INTERP, int PL>
__global__ __launch_bounds__(kUvBlock) void uv_texture_scatter_kernel(
    const T* __restrict__ in, const T* __restrict__ uv, const int* __restrict__ offset,
    const int* __restrict__ list, T* __restrict__ textures, int planes, int NT, int TH, int TW,
    int MP) {
  extern __shared__ __align__(16) unsigned char uv_lds[];
  T* acc = reinterpret_cast<T*>(uv_lds);             // [PL][TH * TW]
  const int THW = TH * TW;
  const int t = blockIdx.x;
  const int plane0 = blockIdx.y * PL;
  const int np = min(PL, planes - plane0);
  // segment of the texture's bucket this workgroup sums (gridDim.z > 1: several workgroups
  // share a texture and add their sums to the zero-filled output)
  const int lo0 = offset[t], hi0 = offset[t + 1];
  const int per = (hi0 - lo0 + (int)gridDim.z - 1) / (int)gridDim.z;
  const int lo = lo0 + (int)blockIdx.z * per, hi = min(hi0, lo + per);
  for (int i = threadIdx.x; i < PL * THW; i += kUvBlock) acc[i] = T(0);
  __syncthreads();
  constexpr int N = PointTaps<T, INTERP>::N;
  // this round's pixel, point and values are loaded during the round before
  int e = lo + (int)threadIdx.x;
  int pix = e < hi ? list[e] : 0;
  T pu = uv[(size_t)pix * 2], pv = uv[(size_t)pix * 2 + 1];
  T val[PL];
#pragma unroll
  for (int j = 0; j < PL; ++j) val[j] = in[(size_t)(plane0 + (j < np ? j : 0)) * MP + pix];
  int pix_next = e + kUvBlock < hi ? list[e + kUvBlock] : 0;
  for (int base = lo; base < hi; base += kUvBlock) {   // uniform trip count over the workgroup
    const bool live = e < hi;
    PointTaps<T, INTERP> taps;
    taps.set(pu, pv, TH, TW);
    T cur[PL];
#pragma unroll
    for (int j = 0; j < PL; ++j) cur[j] = (live && j < np) ? val[j] : T(0);
    // next round's loads
    e += kUvBlock;
    pix = pix_next;
    pu = uv[(size_t)pix * 2];
    pv = uv[(size_t)pix * 2 + 1];
#pragma unroll
    for (int j = 0; j < PL; ++j) val[j] = in[(size_t)(plane0 + (j < np ? j : 0)) * MP + pix];
    pix_next = e + kUvBlock < hi ? list[e + kUvBlock] : 0;
    // lanes whose first tap is the same texel form a run: all their taps coincide
    const int ky = live ? taps.ty[0] : INT_MIN, kx = live ? taps.tx[0] : (int)threadIdx.x;
    const int by = __shfl_up(ky, 1), bx = __shfl_up(kx, 1);
    const LaneRuns runs(by == ky && bx == kx);
#pragma unroll
    for (int i = 0; i < N; ++i) {
      const T w = taps.off[i] >= 0 ? (INTERP == 0 ? T(1) : taps.w[i]) : T(0);
      const bool inside = (unsigned)taps.ty[i] < (unsigned)TH && (unsigned)taps.tx[i] < (unsigned)TW;
      const int o = inside ? taps.ty[i] * TW + taps.tx[i] : 0;
#pragma unroll
      for (int j = 0; j < PL; ++j) {
        const T total = runs.sum(w * cur[j]);
        if (live && runs.tail && inside && total != T(0)) lds_add(acc + j * THW + o, total);
      }
    }
  }
  __syncthreads();
  const size_t stride = (size_t)NT * THW;
  for (int i = threadIdx.x; i < THW; i += kUvBlock) {
#pragma unroll
    for (int j = 0; j < PL; ++j) {
      if (j < np) {
        T* dst = textures + (size_t)(plane0 + j) * stride + (size_t)t * THW + i;
        const T v = acc[j * THW + i];
        if (gridDim.z == 1) *dst = v;
        else if (v != T(0)) atomicAdd(dst, v);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// mapped im2col / col2im, batched.  Bodies: common/mapped_im2col.h:11-41, :44-77,
// :80-116, :119-158.  grid.y walks chunks of the B*C image planes; a plane's K
// column rows are (plane*K + k).
// ---------------------------------------------------------------------------
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_im2col_kernel(
    const T* __restrict__ im, const T* __restrict__ map, const T* __restrict__ wts,
    T* __restrict__ col, int planes, int H, int W, int M, int K, int P) {
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= M) return;
  const int plane0 = blockIdx.y * kPC;
  const int np = min(kPC, planes - plane0);
  const size_t HW = (size_t)H * W;
  const int q = WEIGHTED ? P : 1;
  for (int k = 0; k < K; ++k) {
    const size_t s = ((size_t)pix * K + k) * q;
    T acc[kPC];
    gather_sample<T, INTERP, WEIGHTED, kPC>(im + (size_t)plane0 * HW, HW, np, map + s * 2,
                                            WEIGHTED ? wts + s : nullptr, P, H, W, acc);
#pragma unroll
    for (int j = 0; j < kPC; ++j)
      if (j < np) col[((size_t)(plane0 + j) * K + k) * M + pix] = acc[j];
  }
}

template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_col2im_kernel(
    const T* __restrict__ col, const T* __restrict__ map, const T* __restrict__ wts,
    T* __restrict__ im, int planes, int H, int W, int M, int K, int P) {
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= M) return;
  const int plane0 = blockIdx.y * kPC;
  const int np = min(kPC, planes - plane0);
  const size_t HW = (size_t)H * W;
  const int q = WEIGHTED ? P : 1;
  for (int k = 0; k < K; ++k) {
    const size_t s = ((size_t)pix * K + k) * q;
    T val[kPC];
#pragma unroll
    for (int j = 0; j < kPC; ++j)
      val[j] = j < np ? col[((size_t)(plane0 + j) * K + k) * M + pix] : T(0);
    scatter_sample<T, INTERP, WEIGHTED, kPC>(im + (size_t)plane0 * HW, HW, np, map + s * 2,
                                             WEIGHTED ? wts + s : nullptr, P, H, W, val);
  }
}

// Values of KB consecutive samples (first: k0; samples past K repeat the last) of one pixel of
// an unweighted map for PC planes, v[g][j]: the coordinates of all KB samples are read
// together, then all taps of all planes, then the blends (as PointTaps::gather forms them).
// One round trip for the coordinates and one for the data per KB samples instead of per sample.
template <typename T, int INTERP, int PC, int KB>
__device__ __forceinline__ void gather_sample_batch(const T* __restrict__ base, size_t stride,
                                                    int np, const T* __restrict__ pixel_coords,
                                                    int k0, int K, int H, int W,
                                                    T (&v)[KB][PC]) {
  constexpr int N = PointTaps<T, INTERP>::N;
  T cx[KB], cy[KB];
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    const int k = min(k0 + g, K - 1);
    cx[g] = pixel_coords[2 * k];
    cy[g] = pixel_coords[2 * k + 1];
  }
  PointTaps<T, INTERP> t[KB];
  T raw[KB][PC][N];
#pragma unroll
  for (int g = 0; g < KB; ++g) {
    t[g].set(cx[g], cy[g], H, W);
#pragma unroll
    for (int j = 0; j < PC; ++j) t[g].load(base + (size_t)(j < np ? j : 0) * stride, raw[g][j]);
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int g = 0; g < KB; ++g)
#pragma unroll
    for (int j = 0; j < PC; ++j) v[g][j] = j < np ? t[g].blend(raw[g][j]) : T(0);
}

// ---------------------------------------------------------------------------
// mapped max pool.  Body: common/mapped_max_pool.h:13-57, :81-133 (device
// branch: running maximum starts at -FLT_MAX for every T, index at -1).
// ---------------------------------------------------------------------------
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_max_pool_kernel(
    const T* __restrict__ in, const T* __restrict__ map, const T* __restrict__ wts,
    T* __restrict__ out, int64_t* __restrict__ idx, int planes, int H, int W, int M, int K,
    int P) {
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= M) return;
  const int plane0 = blockIdx.y * kPC;
  const int np = min(kPC, planes - plane0);
  const size_t HW = (size_t)H * W;
  const int q = WEIGHTED ? P : 1;
  T best[kPC];
  int best_k[kPC];
#pragma unroll
  for (int j = 0; j < kPC; ++j) {
    best[j] = T(-FLT_MAX);
    best_k[j] = -1;
  }
  if constexpr (!WEIGHTED) {
    // samples in batches whose reads are in flight together
    constexpr int KB = INTERP == 0 ? 3 : 2;
    const T* coords = map + (size_t)pix * K * 2;
    for (int k0 = 0; k0 < K; k0 += KB) {
      T v[KB][kPC];
      gather_sample_batch<T, INTERP, kPC, KB>(in + (size_t)plane0 * HW, HW, np, coords, k0, K, H,
                                              W, v);
#pragma unroll
      for (int g = 0; g < KB; ++g)
        if (k0 + g < K) {
#pragma unroll
          for (int j = 0; j < kPC; ++j)
            if (v[g][j] > best[j]) {  // strict: first maximum wins, NaN never wins
              best[j] = v[g][j];
              best_k[j] = k0 + g;
            }
        }
    }
  } else {
    for (int k = 0; k < K; ++k) {
      const size_t s = ((size_t)pix * K + k) * q;
      T v[kPC];
      gather_sample<T, INTERP, WEIGHTED, kPC>(in + (size_t)plane0 * HW, HW, np, map + s * 2,
                                              WEIGHTED ? wts + s : nullptr, P, H, W, v);
#pragma unroll
      for (int j = 0; j < kPC; ++j)
        if (v[j] > best[j]) {  // strict: first maximum wins, NaN never wins
          best[j] = v[j];
          best_k[j] = k;
        }
    }
  }
#pragma unroll
  for (int j = 0; j < kPC; ++j)
    if (j < np) {
      const size_t o = (size_t)(plane0 + j) * M + pix;
      out[o] = best[j];
      idx[o] = best_k[j] < 0 ? (int64_t)-1
                             : (int64_t)(((size_t)pix * K + best_k[j]) * q * 2);
    }
}

// Average pool: body common/mapped_avg_pool.h:13-40, :70-105 (sum of the K samples in
// ascending order, divided by K).  Its adjoint (:42-68, :107-140: every sample of a pixel
// receives grad / K) is the resample scatter over the map read as [pixels * K] entries.
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_avg_pool_kernel(
    const T* __restrict__ in, const T* __restrict__ map, const T* __restrict__ wts,
    T* __restrict__ out, int planes, int H, int W, int M, int K, int P) {
  const int pix = banded_pixel_block() * kBlock + threadIdx.x;
  if (pix >= M) return;
  const int plane0 = blockIdx.y * kPC;
  const int np = min(kPC, planes - plane0);
  const size_t HW = (size_t)H * W;
  const int q = WEIGHTED ? P : 1;
  T sum[kPC];
#pragma unroll
  for (int j = 0; j < kPC; ++j) sum[j] = T(0);
  if constexpr (!WEIGHTED) {
    constexpr int KB = INTERP == 0 ? 3 : 2;
    const T* coords = map + (size_t)pix * K * 2;
    for (int k0 = 0; k0 < K; k0 += KB) {
      T v[KB][kPC];
      gather_sample_batch<T, INTERP, kPC, KB>(in + (size_t)plane0 * HW, HW, np, coords, k0, K, H,
                                              W, v);
#pragma unroll
      for (int g = 0; g < KB; ++g)
        if (k0 + g < K) {
#pragma unroll
          for (int j = 0; j < kPC; ++j) sum[j] += v[g][j];
        }
    }
  } else {
    for (int k = 0; k < K; ++k) {
      const size_t s = ((size_t)pix * K + k) * q;
      T v[kPC];
      gather_sample<T, INTERP, WEIGHTED, kPC>(in + (size_t)plane0 * HW, HW, np, map + s * 2,
                                              WEIGHTED ? wts + s : nullptr, P, H, W, v);
#pragma unroll
      for (int j = 0; j < kPC; ++j) sum[j] += v[j];
    }
  }
#pragma unroll
  for (int j = 0; j < kPC; ++j)
    if (j < np) out[(size_t)(plane0 + j) * M + pix] = sum[j] / T(K);
}

// Unpool: body common/mapped_max_pool.h:60-78, :136-171.  One thread per pooled
// element; the stored index names the winning sample inside the map (and,
// halved, inside the weights).  Indices outside [0, map_elems) contribute nothing.
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_max_unpool_kernel(
    const T* __restrict__ gout, const int64_t* __restrict__ idx, const T* __restrict__ map,
    const T* __restrict__ wts, T* __restrict__ gin, size_t total, int H, int W, int M, int P,
    int64_t map_elems, const int* __restrict__ gate) {
  if (gate != nullptr && *gate == 0) return;
  const int q = WEIGHTED ? P : 1;
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / (size_t)M;
    const int64_t s = idx[i];
    if (s < 0 || s + 2 * q > map_elems) continue;
    const T val[1] = {gout[i]};
    scatter_sample<T, INTERP, WEIGHTED, 1>(gin + plane * (size_t)H * W, 0, 1, map + s,
                                           WEIGHTED ? wts + s / 2 : nullptr, P, H, W, val);
  }
}

// After the row-band unpool of a call whose plan is known to run it: the band kernel has written
// every image pixel and added every sample whose index lies among its own pooled pixel's
// samples; it raised gate[0] if it met an index that names another pixel's sample ("stray":
// never produced by the pooling, allowed by the operator).  This kernel adds those samples
// where they point, as mapped_max_unpool_kernel would have, and the workgroup that finishes
// last clears gate[0] for the next call on the plan (gate[1] counts finished workgroups).
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_max_unpool_stray_kernel(
    const T* __restrict__ gout, const int64_t* __restrict__ idx, const T* __restrict__ map,
    const T* __restrict__ wts, T* __restrict__ gin, size_t total, int H, int W, int M, int K,
    int P, int64_t map_elems, int* gate) {
  if (*(volatile int*)gate == 0) return;
  const int q = WEIGHTED ? P : 1;
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / (size_t)M;
    const int64_t pix = (int64_t)(i - plane * (size_t)M);
    const int64_t s = idx[i];
    if (s < 0 || s + 2 * q > map_elems) continue;
    const int64_t d = s - pix * K * q * 2;
    if (d >= 0 && d < (int64_t)2 * K * q && (d & 1) == 0) continue;   // the band kernel's own
    const T val[1] = {gout[i]};
    scatter_sample<T, INTERP, WEIGHTED, 1>(gin + plane * (size_t)H * W, 0, 1, map + s,
                                           WEIGHTED ? wts + s / 2 : nullptr, P, H, W, val);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    __threadfence();
    if (atomicAdd(gate + 1, 1) == (int)gridDim.x - 1) {
      gate[1] = 0;
      gate[0] = 0;
    }
  }
}

// The adjoint of the unpool: every pooled element reads the image at the sample its index
// names (same index convention, same range rule: an index outside the map reads nothing).
// This is the gradient of unpooling with respect to the pooled values; the reference's own
// attempt at it (layers/functional/mapped_pooling.py:156-199) refers to undefined names and
// pools the gradient again instead, so there is no reference kernel to follow, only the
// transpose of common/mapped_max_pool.h:60-78, :136-171.
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void mapped_gather_at_index_kernel(
    const T* __restrict__ image, const int64_t* __restrict__ idx, const T* __restrict__ map,
    const T* __restrict__ wts, T* __restrict__ out, size_t total, int H, int W, int M, int P,
    int64_t map_elems) {
  const int q = WEIGHTED ? P : 1;
  const size_t stride = (size_t)gridDim.x * kBlock;
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += stride) {
    const size_t plane = i / (size_t)M;
    const int64_t s = idx[i];
    T v[1] = {T(0)};
    if (s >= 0 && s + 2 * q <= map_elems)
      gather_sample<T, INTERP, WEIGHTED, 1>(image + plane * (size_t)H * W, 0, 1, map + s,
                                            WEIGHTED ? wts + s / 2 : nullptr, P, H, W, v);
    out[i] = v[0];
  }
}

// ---------------------------------------------------------------------------
// Unpool by image tile.  A workgroup owns a tile of kUpTile image pixels and a group of
// planes, accumulates the tile in LDS and writes every pixel of it exactly once with a
// plain store: no zero fill of the image, no global atomics.  It has to look at every
// pooled pixel that can reach the tile, whichever sample wins: the map alone fixes that
// set, and two small kernels find, per tile, the window of the pooled grid that holds it
// (rows x columns, columns wrap modulo the pooled width):
//   unpool_anchor:  one thread per (pooled pixel, sample); every tile a tap of the sample
//       falls into records that pooled pixel (any one of them serves as the anchor).
//   unpool_window:  the same walk; the tile's window grows to hold the pooled pixel,
//       measured from the anchor so that a window may straddle the seam.
//   unpool_tiles:   per pass of up to kUpPlanes planes: clear the LDS tile; every thread
//       takes pooled pixels of the window (coalesced index and gradient reads), reads the
//       winning sample's coordinates from the map and adds the taps that fall inside the
//       tile to LDS; then the tile is stored.  Windows of neighbouring tiles overlap, so a
//       pooled pixel is read by every tile it can reach, and adds only what lands there.
// *gate is raised, and the call falls back to zero fill + atomic scatter, when a window is
// larger than kUpWindow pooled pixels (an incoherent map) or an index names a sample of
// another pooled pixel than its own (mapped_max_pool never writes one, but the scatter
// accepts it): such a sample may reach tiles whose windows do not hold the pixel.
// ---------------------------------------------------------------------------
constexpr int kUpTileLog2 = 11;
constexpr int kUpTile = 1 << kUpTileLog2;   // image pixels per workgroup
constexpr int kUpPer = kUpTile / kBlock;    // ... and per thread
constexpr int kUpWindow = 8192;   // pooled pixels a tile may have to look at
constexpr int kUpBytes = 32768;   // LDS of the tile accumulators: kUpTile x planes per pass
constexpr int kUpAhead = 3;       // pooled pixels of a lane whose reads are in flight together

struct UnpoolTiling {
  int H, W, tw_shift, tiles_x, tiles_y;
  __host__ __device__ int TW() const { return 1 << tw_shift; }
  __host__ __device__ int TH() const { return kUpTile >> tw_shift; }
  __device__ int tile_of(int y, int x) const {
    return (y >> (kUpTileLog2 - tw_shift)) * tiles_x + (x >> tw_shift);   // TH = kUpTile >> tw_shift
  }
};

// Per tile, 8 ints (cleared before the analysis): [0] anchor pooled pixel + 1 (0: nothing
// reaches the tile), [1..4] window extent around the anchor: rows up, rows down, columns
// left, columns right.
// A workgroup's samples reach a handful of tiles: their extents are first merged in a small
// LDS table (kWinSlots tiles, open addressing) and reach global memory once per tile and
// workgroup; a sample that finds the table full goes to global memory directly.
constexpr int kWinSlots = 8;

__device__ __forceinline__ void grow_window(int* w, int up, int down, int left, int right) {
  if (up > w[1]) atomicMax(&w[1], up);
  if (down > w[2]) atomicMax(&w[2], down);
  if (left > w[3]) atomicMax(&w[3], left);
  if (right > w[4]) atomicMax(&w[4], right);
}

template <typename T, int INTERP, bool WEIGHTED, bool GROW>
__global__ __launch_bounds__(kBlock) void unpool_window_kernel(
    const T* __restrict__ map, int64_t samples, int P, int K, int OW, UnpoolTiling ut,
    int* __restrict__ win, const int* __restrict__ skip) {
  if (skip != nullptr && skip[0] != 0) return;   // the row-band kernels do this call
  __shared__ int s_tile[kWinSlots];
  __shared__ int s_ext[kWinSlots][4];
  if (GROW) {
    if (threadIdx.x < kWinSlots) {
      s_tile[threadIdx.x] = -1;
      s_ext[threadIdx.x][0] = s_ext[threadIdx.x][1] = 0;
      s_ext[threadIdx.x][2] = s_ext[threadIdx.x][3] = 0;
    }
    __syncthreads();
  }
  const int64_t smp = (int64_t)blockIdx.x * kBlock + threadIdx.x;   // pooled pixel * K + k
  if (smp < samples) {
    const int q = WEIGHTED ? P : 1;
    const int o = (int)(smp / K);
    PointTaps<T, INTERP> t;
    for (int p = 0; p < q; ++p) {
      const size_t s = (size_t)smp * q + p;
      t.set(map[s * 2], map[s * 2 + 1], ut.H, ut.W);
#pragma unroll
      for (int i = 0; i < PointTaps<T, INTERP>::N; ++i) {
        if (t.off[i] < 0) continue;
        const int tile = ut.tile_of(t.ty[i], t.tx[i]);
        int* w = win + (size_t)tile * 8;
        if constexpr (!GROW) {
          w[0] = o + 1;
        } else {
          const int a = w[0] - 1;
          const int dy = o / OW - a / OW;
          int dx = o % OW - a % OW;
          dx += (dx > OW / 2) ? -OW : ((dx < -(OW / 2)) ? OW : 0);
          int slot = -1;
          for (int probe = 0; probe < kWinSlots && slot < 0; ++probe) {
            const int h = (tile + probe) & (kWinSlots - 1);
            const int seen = atomicCAS(&s_tile[h], -1, tile);
            if (seen == -1 || seen == tile) slot = h;
          }
          if (slot >= 0) {
            if (-dy > s_ext[slot][0]) atomicMax(&s_ext[slot][0], -dy);
            if (dy > s_ext[slot][1]) atomicMax(&s_ext[slot][1], dy);
            if (-dx > s_ext[slot][2]) atomicMax(&s_ext[slot][2], -dx);
            if (dx > s_ext[slot][3]) atomicMax(&s_ext[slot][3], dx);
          } else {
            grow_window(w, -dy, dy, -dx, dx);
          }
        }
      }
    }
  }
  if (GROW) {
    __syncthreads();
    if (threadIdx.x < kWinSlots && s_tile[threadIdx.x] >= 0)
      grow_window(win + (size_t)s_tile[threadIdx.x] * 8, s_ext[threadIdx.x][0],
                  s_ext[threadIdx.x][1], s_ext[threadIdx.x][2], s_ext[threadIdx.x][3]);
  }
}

template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void unpool_tiles_kernel(
    const T* __restrict__ gout, const int64_t* __restrict__ idx, const T* __restrict__ map,
    const T* __restrict__ wts, const int* __restrict__ win, T* __restrict__ gin,
    int* __restrict__ gate, UnpoolTiling ut, int planes, int planes_per_group, int M, int OW,
    int K, int P, int64_t map_elems, const int* __restrict__ skip) {
  if (*gate != 0 || (skip != nullptr && skip[0] != 0)) return;
  constexpr int PLMAX = kUpBytes / (kUpTile * (int)sizeof(T));   // planes per pass
  __shared__ T acc[PLMAX * kUpTile];
  const int tid = threadIdx.x, tile = blockIdx.x;
  const size_t HW = (size_t)ut.H * ut.W;
  const int p_begin = blockIdx.y * planes_per_group;
  const int p_end = min(planes, p_begin + planes_per_group);
  const int ty0 = (tile / ut.tiles_x) * ut.TH(), tx0 = (tile % ut.tiles_x) << ut.tw_shift;
  const int q = WEIGHTED ? P : 1;
  const int twoq = 2 * q;
  // window of pooled pixels
  const int* w = win + (size_t)tile * 8;
  const int anchor = w[0] - 1;
  int WH = 0, WW = 0, wy0 = 0, wx0 = 0;
  if (anchor >= 0) {
    const int ay = anchor / OW, ax = anchor % OW;
    WH = w[1] + w[2] + 1;
    const bool full = w[3] + w[4] + 1 >= OW;   // all around: columns as they are
    WW = full ? OW : w[3] + w[4] + 1;
    wy0 = ay - w[1];
    wx0 = full ? 0 : ax - w[3];
    wx0 += wx0 < 0 ? OW : 0;
  }
  if ((int64_t)WH * WW > kUpWindow) {
    if (tid == 0) atomicAdd(gate, 1);
    return;
  }
  const int WN = WH * WW;
  const float rcp_ww = WW > 0 ? 1.0f / (float)WW : 0.0f;
  const int per_pixel = K * twoq;   // map elements of one pooled pixel
  // the thread's 4 image pixels: waves own 4 consecutive 64-pixel runs of the tile
  int u[kUpPer];
#pragma unroll
  for (int j = 0; j < kUpPer; ++j) {
    const int L = (((tid >> 6) * kUpPer + j) << 6) + (tid & 63);
    const int y = ty0 + (L >> ut.tw_shift), x = tx0 + (L & (ut.TW() - 1));
    u[j] = (y < ut.H && x < ut.W) ? y * ut.W + x : -1;
  }
#pragma unroll
  for (int j = 0; j < kUpPer; ++j)
#pragma unroll
    for (int pl = 0; pl < PLMAX; ++pl)
      acc[pl * kUpTile + (((tid >> 6) * kUpPer + j) << 6) + (tid & 63)] = T(0);
  __syncthreads();
  for (int p0 = p_begin; p0 < p_end; p0 += PLMAX) {
    const int np = min(PLMAX, p_end - p0);
    // ---- pooled pixels of the window: a thread takes one at a time and walks the planes
    // of the pass, so the position arithmetic is shared and PLMAX independent (index,
    // gradient) pairs, then their map reads, are in flight together
    for (int o = tid; o < WN; o += kBlock) {
      const int r = (int)(((float)o + 0.5f) * rcp_ww);    // o / WW (o < 2^13: exact)
      int ox = wx0 + (o - r * WW);
      ox -= ox >= OW ? OW : 0;
      const int m = (wy0 + r) * OW + ox;
      const int first = m * per_pixel;   // map element of the pixel's first sample
      const size_t at = (size_t)p0 * M + m;
      int sv[PLMAX];
      T gv[PLMAX];
      bool live[PLMAX];
#pragma unroll
      for (int pl = 0; pl < PLMAX; ++pl) {
        const bool on = pl < np;
        const int64_t s64 = on ? idx[at + (size_t)pl * M] : (int64_t)-1;
        gv[pl] = on ? gout[at + (size_t)pl * M] : T(0);
        live[pl] = s64 >= 0 && s64 + twoq <= map_elems;   // others contribute nothing
        sv[pl] = (int)s64;                                  // map_elems < 2^31
      }
      __builtin_amdgcn_sched_barrier(0);   // indices and gradients are requested together
      T cx[PLMAX], cy[PLMAX];
      bool stray = false;
#pragma unroll
      for (int pl = 0; pl < PLMAX; ++pl) {
        const int d = sv[pl] - first;
        const bool mine = d >= 0 && d < per_pixel && d % twoq == 0;   // a sample of this pixel
        stray |= live[pl] && !mine;
        live[pl] = live[pl] && mine;
        sv[pl] = live[pl] ? sv[pl] : 0;
      }
      // unconditional reads (element 0 for planes that contribute nothing), so that the
      // coordinates of all planes are fetched in one round trip
#pragma unroll
      for (int pl = 0; pl < PLMAX; ++pl) {
        cx[pl] = map[sv[pl]];
        cy[pl] = map[sv[pl] + 1];
      }
      if (stray) atomicAdd(gate, 1);
#pragma unroll
      for (int pl = 0; pl < PLMAX; ++pl) {
        if (!live[pl]) continue;
        T* a = acc + pl * kUpTile;
        PointTaps<T, INTERP> taps;
        for (int p = 0; p < q; ++p) {
          T v = gv[pl];
          if (p == 0) {
            taps.set(cx[pl], cy[pl], ut.H, ut.W);
          } else {
            taps.set(map[sv[pl] + 2 * p], map[sv[pl] + 2 * p + 1], ut.H, ut.W);
          }
          if constexpr (WEIGHTED) v = wts[sv[pl] / 2 + p] * v;
#pragma unroll
          for (int n = 0; n < PointTaps<T, INTERP>::N; ++n) {
            const int ry = taps.ty[n] - ty0, rx = taps.tx[n] - tx0;
            if (taps.off[n] >= 0 && (unsigned)ry < (unsigned)ut.TH() &&
                (unsigned)rx < (unsigned)ut.TW())
              lds_add(a + (ry << ut.tw_shift) + rx, INTERP == 0 ? v : taps.w[n] * v);
          }
        }
      }
    }
    __syncthreads();
    // store the tile and clear it for the next pass
#pragma unroll
    for (int j = 0; j < kUpPer; ++j) {
#pragma unroll
      for (int pl = 0; pl < PLMAX; ++pl) {
        T* cell = acc + pl * kUpTile + (((tid >> 6) * kUpPer + j) << 6) + (tid & 63);
        const T v = *cell;
        *cell = T(0);
        if (u[j] >= 0 && pl < np) gin[(size_t)(p0 + pl) * HW + u[j]] = v;
      }
    }
    __syncthreads();
  }
}

// Average unpooling by image tile (body: common/mapped_avg_pool.h:42-69, :109-143, every
// sample of a pooled pixel receiving grad_output / K through the resampling scatter of
// core/resample.h): the tiling and the windows of unpool_tiles_kernel, but every
// pooled pixel of the window hands value / K to all K of its samples, so the taps of a sample
// are worked out once for the planes of a pass and no index is read.  A lane walks the samples
// of its own pooled pixel (neighbouring lanes then add to different image pixels).  Runs only
// where flags[0] says that every window fits (avg_unpool_verdict_kernel); the sums of a pixel
// are divided by K once, at the store, like the list gather does.
template <typename T, int INTERP, bool WEIGHTED>
__global__ __launch_bounds__(kBlock) void avg_unpool_tiles_kernel(
    const T* __restrict__ gout, const T* __restrict__ map, const T* __restrict__ wts,
    const int* __restrict__ win, const int* __restrict__ flags, T* __restrict__ gin,
    UnpoolTiling ut, int planes, int planes_per_group, int M, int OW, int K, int P,
    const int* __restrict__ skip) {
  if (flags[0] == 0 || (skip != nullptr && skip[0] != 0)) return;
  constexpr int PLMAX = kUpBytes / (kUpTile * (int)sizeof(T));   // planes per pass
  __shared__ T acc[PLMAX * kUpTile];
  const int tid = threadIdx.x, tile = blockIdx.x;
  const size_t HW = (size_t)ut.H * ut.W;
  const int p_begin = blockIdx.y * planes_per_group;
  const int p_end = min(planes, p_begin + planes_per_group);
  const int ty0 = (tile / ut.tiles_x) * ut.TH(), tx0 = (tile % ut.tiles_x) << ut.tw_shift;
  const int q = WEIGHTED ? P : 1;
  const int* w = win + (size_t)tile * 8;
  const int anchor = w[0] - 1;
  int WH = 0, WW = 0, wy0 = 0, wx0 = 0;
  if (anchor >= 0) {
    const int ay = anchor / OW, ax = anchor % OW;
    WH = w[1] + w[2] + 1;
    const bool full = w[3] + w[4] + 1 >= OW;   // all around: columns as they are
    WW = full ? OW : w[3] + w[4] + 1;
    wy0 = ay - w[1];
    wx0 = full ? 0 : ax - w[3];
    wx0 += wx0 < 0 ? OW : 0;
  }
  const int WN = WH * WW;   // <= kUpWindow (flags[0])
  const float rcp_ww = WW > 0 ? 1.0f / (float)WW : 0.0f;
  int u[kUpPer];
#pragma unroll
  for (int j = 0; j < kUpPer; ++j) {
    const int L = (((tid >> 6) * kUpPer + j) << 6) + (tid & 63);
    const int y = ty0 + (L >> ut.tw_shift), x = tx0 + (L & (ut.TW() - 1));
    u[j] = (y < ut.H && x < ut.W) ? y * ut.W + x : -1;
  }
#pragma unroll
  for (int j = 0; j < kUpPer; ++j)
#pragma unroll
    for (int pl = 0; pl < PLMAX; ++pl)
      acc[pl * kUpTile + (((tid >> 6) * kUpPer + j) << 6) + (tid & 63)] = T(0);
  __syncthreads();
  for (int p0 = p_begin; p0 < p_end; p0 += PLMAX) {
    const int np = min(PLMAX, p_end - p0);
    // kUpAhead pooled pixels per lane and round: their values and first coordinates are all
    // requested before the first of them is worked on
    for (int o0 = tid; o0 < WN; o0 += kUpAhead * kBlock) {
      size_t s0[kUpAhead];
      T gv[kUpAhead][PLMAX], cx0[kUpAhead], cy0[kUpAhead];
#pragma unroll
      for (int j = 0; j < kUpAhead; ++j) {
        const int o = o0 + j * kBlock < WN ? o0 + j * kBlock : o0;   // past the end: read again
        const int r = (int)(((float)o + 0.5f) * rcp_ww);    // o / WW (o < 2^13: exact)
        int ox = wx0 + (o - r * WW);
        ox -= ox >= OW ? OW : 0;
        const int m = (wy0 + r) * OW + ox;
        const size_t at = (size_t)p0 * M + m;
#pragma unroll
        for (int pl = 0; pl < PLMAX; ++pl)
          gv[j][pl] = gout[at + (size_t)(pl < np ? pl : 0) * M];
        s0[j] = (size_t)m * K * q;   // the pixel's first map point
        cx0[j] = map[s0[j] * 2];
        cy0[j] = map[s0[j] * 2 + 1];
      }
      const int pts_n = K * q;
#pragma unroll
      for (int j = 0; j < kUpAhead; ++j) {
        if (o0 + j * kBlock >= WN) break;
        T cx = cx0[j], cy = cy0[j];
        for (int s = 0; s < pts_n; ++s) {
          const T x_now = cx, y_now = cy;
          const size_t sn = s0[j] + min(s + 1, pts_n - 1);   // the next point, a turn ahead
          cx = map[sn * 2];
          cy = map[sn * 2 + 1];
          PointTaps<T, INTERP> taps;
          taps.set(x_now, y_now, ut.H, ut.W);
          const T wv = WEIGHTED ? wts[s0[j] + s] : T(1);
#pragma unroll
          for (int n = 0; n < PointTaps<T, INTERP>::N; ++n) {
            const int ry = taps.ty[n] - ty0, rx = taps.tx[n] - tx0;
            if (taps.off[n] >= 0 && (unsigned)ry < (unsigned)ut.TH() &&
                (unsigned)rx < (unsigned)ut.TW()) {
              const int cell = (ry << ut.tw_shift) + rx;
              const T c = INTERP == 0 ? wv : taps.w[n] * wv;
              if constexpr (sizeof(T) == 4) {
                int offs[PLMAX];
                float vals[PLMAX];
#pragma unroll
                for (int pl = 0; pl < PLMAX; ++pl) {
                  offs[pl] = pl * kUpTile + cell;
                  vals[pl] = c * gv[j][pl];
                }
                lds_add_f32_batch<PLMAX>(reinterpret_cast<float*>(acc), offs, vals);
              } else {
#pragma unroll
                for (int pl = 0; pl < PLMAX; ++pl)
                  lds_add(acc + pl * kUpTile + cell, c * gv[j][pl]);
              }
            }
          }
        }
      }
    }
    __syncthreads();
    // store the tile and clear it for the next pass
#pragma unroll
    for (int j = 0; j < kUpPer; ++j) {
#pragma unroll
      for (int pl = 0; pl < PLMAX; ++pl) {
        T* cell = acc + pl * kUpTile + (((tid >> 6) * kUpPer + j) << 6) + (tid & 63);
        const T v = *cell;
        *cell = T(0);
        if (u[j] >= 0 && pl < np) gin[(size_t)(p0 + pl) * HW + u[j]] = v / T(K);
      }
    }
    __syncthreads();
  }
}

// Flags of the tiled average unpooling, in front of its tile windows: [0] every window fits
// the tiled kernel, [1] the opposite (the inverse lists are needed), [2] the gate of the atomic
// fallback.  Stage 0 (after the windows): [0] and [1].  Stage 1 (after the lists, whose own
// gate counts the sources that found a list full): [2] = that gate where the lists are used;
// the word after the lists' gate receives a copy of [0].
// bands: the row-band table of these windows, or nullptr; where its verdict word says that the
// band kernels do the call, the windows (which may not have been built then) are not looked at.
__global__ __launch_bounds__(kBlock) void avg_unpool_verdict_kernel(
    const int* __restrict__ win, int tiles, int OW, int* __restrict__ flags,
    int* __restrict__ lists_gate, int stage, const int* __restrict__ bands) {
  if (stage == 1) {
    if (threadIdx.x == 0) {
      flags[2] = flags[0] != 0 ? 0 : lists_gate[0];
      lists_gate[1] = flags[0];   // for the host: sdk_resample_plan_complete
    }
    return;
  }
  __shared__ int too_big;
  if (threadIdx.x == 0) too_big = 0;
  __syncthreads();
  if (bands != nullptr && bands[0] != 0) tiles = 0;
  for (int t = threadIdx.x; t < tiles; t += kBlock) {
    const int* w = win + (size_t)t * 8;
    if (w[0] > 0) {
      const int64_t WH = (int64_t)w[1] + w[2] + 1;
      const int64_t WW = min((int64_t)w[3] + w[4] + 1, (int64_t)OW);
      if (WH * WW > kUpWindow) too_big = 1;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    flags[0] = too_big ? 0 : 1;
    flags[1] = too_big ? 1 : 0;
  }
}

// ---------------------------------------------------------------------------
// Host-side launch helpers.
// ---------------------------------------------------------------------------
static int check_plane(int64_t h, int64_t w, const char* what) {
  if (h <= 0 || w <= 0 || h * w >= ((int64_t)1 << 31))
    return fail(SDK_ERR_INVALID_ARGUMENT, "%s: plane %lld x %lld must have 1 .. 2^31-1 elements",
                what, (long long)h, (long long)w);
  return SDK_OK;
}

static int check_grid_y(int64_t planes, const char* what) {
  if (ceil_div(planes, kPC) > 65534)   // one grid row is kept for a weight-sum plane
    return fail(SDK_ERR_UNSUPPORTED, "%s: batch*channels = %lld exceeds %d", what,
                (long long)planes, 65534 * kPC);
  return SDK_OK;
}

template <typename T>
static int launch_resample_from_map(const T* image, const T* map, const T* wts, T* out,
                                    int64_t planes, int H, int W, int MP, int P, int interp,
                                    hipStream_t stream) {
  const int pc = gather_planes_per_thread(planes);
#define RFM(PCv)                                                                              \
  SDK_DISPATCH_INTERP(interp, P,                                                              \
                      (launch((resample_from_map_kernel<T, INTERP, WEIGHTED, PCv>),           \
                              dim3((unsigned)ceil_div(MP, kBlock), (unsigned)ceil_div(planes, PCv)), \
                              dim3(kBlock), stream, image, map, wts, out, (int)planes, H, W,  \
                              MP, P)))
  if (pc >= 8) RFM(8); else if (pc >= 4) RFM(4); else if (pc >= 2) RFM(2); else RFM(1);
#undef RFM
  SDK_LAUNCH_CHECK("resample_from_map");
  return SDK_OK;
}

static size_t inverse_layout(int64_t HW, size_t esz, size_t (&off)[4]) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  off[0] = 0;                                   // gate (first int), then cnt: cleared together
  off[1] = 256;                                 // cnt
  off[2] = off[1] + up((size_t)HW * 4);         // src
  off[3] = off[2] + up((size_t)HW * kInvSlots * 4);   // co
  return off[3] + up((size_t)HW * kInvSlots * esz);
}

static UnpoolTiling unpool_tiling(int H, int W);
static size_t unpool_layout(const UnpoolTiling& ut);
static size_t unpool_layout_with_bands(const UnpoolTiling& ut);
static size_t unpool_layout_with_taps(const UnpoolTiling& ut);
static unsigned* unpool_taps_at(void* region, size_t region_bytes, const UnpoolTiling& ut);
template <typename T>
static bool unpool_bands_possible(int H, int W, int OH, int OW, int K, int P, int interp);
template <typename T>
static int build_unpool_windows(const T* map, void* workspace, size_t workspace_bytes, int H, int W,
                                int OH, int OW, int K, int P, int interp, hipStream_t stream,
                                unsigned* seen = nullptr);

// Average unpooling (group = K > 1 samples per pooled pixel, pooled rows of OW pixels) can run
// tiled over the image when the workspace has room for the tile windows behind the lists.
static bool avg_unpool_tiled(int H, int W, int MP, int group, int OW, int P, size_t esz,
                             int64_t planes, size_t lists_bytes, size_t workspace_bytes) {
  if (group <= 1 || OW <= 0 || (MP / group) % OW != 0) return false;
  const UnpoolTiling ut = unpool_tiling(H, W);
  return workspace_bytes >= lists_bytes + unpool_layout(ut) &&
         (int64_t)ut.tiles_x * ut.tiles_y < ((int64_t)1 << 27) && planes < ((int64_t)1 << 31);
}

// Inverts a map into `workspace` (inverse_layout bytes): per target pixel the list of its
// (source, coefficient) pairs, and the gate word that counts sources that found their list full.
// For average unpooling with room for them (avg_unpool_tiled) the tile windows and their flags
// follow the lists, and the lists are filled only where a window is too large for the tiled
// kernel.
template <typename T>
static int build_inverse_lists(const T* map, const T* wts, void* workspace, size_t workspace_bytes,
                               int H, int W, int MP, int P, int interp, int group, int OW,
                               hipStream_t stream) {
  size_t off[4];
  const size_t lists_bytes = inverse_layout((int64_t)H * W, sizeof(T), off);
  char* ws = static_cast<char*>(workspace);
  int* g = reinterpret_cast<int*>(ws + off[0]);
  int* cnt = reinterpret_cast<int*>(ws + off[1]);
  int* src = reinterpret_cast<int*>(ws + off[2]);
  T* co = reinterpret_cast<T*>(ws + off[3]);
  int* flags = nullptr;
  if (avg_unpool_tiled(H, W, MP, group, OW, P, sizeof(T), 0, lists_bytes, workspace_bytes)) {
    flags = reinterpret_cast<int*>(ws + lists_bytes);
    const UnpoolTiling ut = unpool_tiling(H, W);
    const size_t region = workspace_bytes - lists_bytes;
    // the lists' counters, not yet in use, lend themselves to the band table's build
    int rc = zero_fill(ws + off[1], off[2] - off[1], stream);
    if (rc != SDK_OK) return rc;
    rc = build_unpool_windows<T>(map, ws + lists_bytes, region, H, W, MP / group / OW, OW, group,
                                 P, interp, stream, reinterpret_cast<unsigned*>(cnt));
    if (rc != SDK_OK) return rc;
    const int* bands = nullptr;
    if (region >= unpool_layout_with_bands(ut) &&
        unpool_bands_possible<T>(H, W, MP / group / OW, OW, group, P, interp))
      bands = reinterpret_cast<const int*>(ws + lists_bytes + unpool_layout(ut));
    launch(avg_unpool_verdict_kernel, dim3(1), dim3(kBlock), stream, (const int*)(flags + 64),
           ut.tiles_x * ut.tiles_y, OW, flags, g, 0, bands);
    SDK_LAUNCH_CHECK("mapped_avg_unpool(windows)");
  }
  int rc;
  if (flags) {   // the gate, read by the caller whatever happens; the counters where needed
    rc = zero_fill(ws, off[1], stream);
    if (rc == SDK_OK) rc = zero_fill_gated(ws + off[1], off[2] - off[1], stream, flags + 1);
  } else {
    rc = zero_fill(ws, off[2], stream);
  }
  if (rc != SDK_OK) return rc;
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((resample_inverse_fill_kernel<T, INTERP, WEIGHTED>),
                              dim3((unsigned)ceil_div(MP, kBlock)), dim3(kBlock), stream, map,
                              wts, H, W, MP, P, cnt, src, co, g, group,
                              (const int*)(flags ? flags + 1 : nullptr))));
  SDK_LAUNCH_CHECK("resample_to_map(inverse fill)");
  launch(resample_inverse_sort_kernel<T>, dim3((unsigned)ceil_div((int64_t)H * W, kBlock)),
         dim3(kBlock), stream, (const int*)cnt, src, co, H * W, (const int*)g,
         (const int*)(flags ? flags + 1 : nullptr));
  SDK_LAUNCH_CHECK("resample_to_map(inverse sort)");
  if (flags) {
    launch(avg_unpool_verdict_kernel, dim3(1), dim3(kBlock), stream, (const int*)(flags + 64), 0,
           OW, flags, g, 1, (const int*)nullptr);
    SDK_LAUNCH_CHECK("mapped_avg_unpool(gate)");
  }
  return SDK_OK;
}

// prebuilt: `workspace` already holds the lists of this map (build_inverse_lists);
// complete: ... and the caller knows (sdk_resample_plan_complete) that its gate is 0 (bit 0),
// so the fallback launches are left out, and that the tiled average unpooling runs (bit 1), so
// the list gather is left out as well.
// OW > 0 (average unpooling): width of the pooled grid.
template <typename T>
static int launch_resample_to_map(const T* in, const T* map, const T* wts, T* out, T* wsum,
                                  void* workspace, size_t workspace_bytes, int64_t planes, int H,
                                  int W, int MP, int P, int interp, hipStream_t stream,
                                  bool normalize = false, double eps = 0.0, int group = 1,
                                  bool prebuilt = false, int complete = 0, int OW = 0) {
  const int HW = H * W;
  const int* gate = nullptr;   // non-null: device flag, != 0 means "use the atomic scatter"
  size_t off[4];
  const size_t lists_bytes = inverse_layout(HW, sizeof(T), off);
  if (workspace != nullptr && workspace_bytes >= lists_bytes) {
    char* ws = static_cast<char*>(workspace);
    int* g = reinterpret_cast<int*>(ws + off[0]);
    int* cnt = reinterpret_cast<int*>(ws + off[1]);
    int* src = reinterpret_cast<int*>(ws + off[2]);
    T* co = reinterpret_cast<T*>(ws + off[3]);
    const bool tiled = !normalize && wsum == nullptr &&
                       avg_unpool_tiled(H, W, MP, group, OW, P, sizeof(T), planes, lists_bytes, workspace_bytes);
    const int* flags = tiled ? reinterpret_cast<const int*>(ws + lists_bytes) : nullptr;
    // the row-band form of the tiled average unpooling: the table behind the tile windows
    const int* bands = nullptr;
    if (tiled) {
      const UnpoolTiling ut = unpool_tiling(H, W);
      if (workspace_bytes - lists_bytes >= unpool_layout_with_bands(ut) &&
          unpool_bands_possible<T>(H, W, MP / group / OW, OW, group, P, interp))
        bands = reinterpret_cast<const int*>(ws + lists_bytes + unpool_layout(ut));
    }
    if (!prebuilt) {
      const int rc = build_inverse_lists<T>(map, wts, workspace, tiled ? workspace_bytes : lists_bytes,
                                            H, W, MP, P, interp, group, OW, stream);
      if (rc != SDK_OK) return rc;
    }
    if (bands != nullptr && planes > 0) {
      if constexpr (sizeof(T) == 4) {
        unpool_band_launch(true, (const float*)in, nullptr, (const float*)map, (float*)out, bands,
                           unpool_taps_at(ws + lists_bytes, workspace_bytes - lists_bytes,
                                          unpool_tiling(H, W)),
                           nullptr, planes, H, W, MP / group / OW, OW, group, stream);
        SDK_LAUNCH_CHECK("mapped_avg_unpool(bands)");
      }
    }
    if (tiled && planes > 0) {
      const UnpoolTiling ut = unpool_tiling(H, W);
      const int64_t tiles = (int64_t)ut.tiles_x * ut.tiles_y;
      constexpr int PLMAX = kUpBytes / (kUpTile * (int)sizeof(T));
      const int64_t groups = std::max<int64_t>(1, std::min<int64_t>(ceil_div(planes, PLMAX),
                                                                    ceil_div(16384, tiles)));
      const int64_t per_group = ceil_div(ceil_div(planes, groups), PLMAX) * PLMAX;
      const dim3 grid_t((unsigned)tiles, (unsigned)ceil_div(planes, per_group));   // <= 16384 rows
      SDK_DISPATCH_INTERP(interp, P,
                          (launch((avg_unpool_tiles_kernel<T, INTERP, WEIGHTED>), grid_t,
                                  dim3(kBlock), stream, in, map, wts, flags + 64, flags, out, ut,
                                  (int)planes, (int)per_group, MP / group, OW, group, P, bands)));
      SDK_LAUNCH_CHECK("mapped_avg_unpool(tiles)");
    }
    if ((planes > 0 || wsum) && !(tiled && prebuilt && (complete & 2))) {
      const int pc = planes_per_thread(planes);
#define RIG(PCv)                                                                                 \
  launch(resample_inverse_gather_kernel<T, PCv>,                                                 \
         dim3(banded_grid_x(HW), (unsigned)std::max<int64_t>(1, ceil_div(planes, PCv))),         \
         dim3(kBlock), stream, in, (const int*)cnt, (const int*)src, (const T*)co, out, wsum,    \
         (int)planes, HW, MP, (const int*)g, normalize ? 1 : 0, (T)eps, group, flags)
      if (pc == 8) RIG(8); else if (pc == 4) RIG(4); else RIG(2);
#undef RIG
      SDK_LAUNCH_CHECK("resample_to_map(inverse gather)");
    }
    gate = tiled ? flags + 2 : g;
    if (prebuilt && (complete & 1)) return SDK_OK;
  }
  // the scatter: fills, then one launch for all planes and (an extra grid row) the weight sum
  const size_t out_bytes = sizeof(T) * (size_t)planes * H * W, sum_bytes = sizeof(T) * (size_t)H * W;
  if (wsum && out_bytes % 16 == 0 && sum_bytes % 16 == 0 && (uintptr_t)out % 16 == 0 &&
      (uintptr_t)wsum % 16 == 0) {
    const size_t n16 = (out_bytes + sum_bytes) / 16;
    const int blocks = (int)std::min<size_t>(ceil_div((int64_t)n16, kBlock), 256 * 16);
    launch(zero16_pair_kernel, dim3(blocks), dim3(kBlock), stream, (uint4*)out, out_bytes / 16,
           (uint4*)wsum, sum_bytes / 16, gate);
    SDK_LAUNCH_CHECK("resample_to_map(fill)");
  } else {
    int rc = zero_fill_gated(out, out_bytes, stream, gate);
    if (rc != SDK_OK) return rc;
    if (wsum) rc = zero_fill_gated(wsum, sum_bytes, stream, gate);
    if (rc != SDK_OK) return rc;
  }
  if (planes > 0 || wsum) {
    const dim3 grid(banded_grid_x(MP), (unsigned)(ceil_div(planes, kPC) + (wsum ? 1 : 0)));
    SDK_DISPATCH_INTERP(interp, P,
                        (launch((resample_to_map_kernel<T, INTERP, WEIGHTED>), grid, dim3(kBlock),
                                stream, in, map, wts, out, wsum, (int)planes, H, W, MP, P, gate,
                                group)));
    SDK_LAUNCH_CHECK("resample_to_map");
  }
  if (normalize && planes > 0) {   // scatter path only: the gather has divided already
    const size_t total = (size_t)planes * HW;
    const int blocks = (int)std::min<int64_t>(ceil_div((int64_t)total, kBlock), 256 * 16);
    launch(normalize_kernel<T>, dim3(blocks), dim3(kBlock), stream, out, (const T*)wsum, (T)eps,
           (size_t)HW, total, gate);
    SDK_LAUNCH_CHECK("resample_to_map(normalise)");
  }
  return SDK_OK;
}

// INTERP alone (UV maps carry no interpolation weights); same mapping of the enum as
// SDK_DISPATCH_INTERP.
#define SDK_DISPATCH_INTERP_ONLY(interp, CALL)                  \
  do {                                                          \
    if ((interp) == 1) { constexpr int INTERP = 1; CALL; }      \
    else if ((interp) == 2) { constexpr int INTERP = 2; CALL; } \
    else { constexpr int INTERP = 0; CALL; }                    \
  } while (0)

template <typename T>
static int launch_uv_gather(const T* textures, const int64_t* quad, const T* uv, T* out,
                            int64_t planes, int NT, int TH, int TW, int MP, int interp,
                            hipStream_t stream) {
  const int pc = planes_per_thread(planes);
#define UVG(PCv)                                                                              \
  SDK_DISPATCH_INTERP_ONLY(interp,                                                            \
                           (launch((uv_gather_kernel<T, INTERP, PCv>),                        \
                                   dim3(banded_grid_x(MP), (unsigned)ceil_div(planes, PCv)),  \
                                   dim3(kBlock), stream, textures, quad, uv, out, (int)planes, \
                                   NT, TH, TW, MP)))
  if (pc >= 8) UVG(8); else if (pc >= 4) UVG(4); else UVG(2);
#undef UVG
  SDK_LAUNCH_CHECK("resample_from_uv_maps");
  return SDK_OK;
}

// Copies of the bucket counters (a power of two; fewer for many textures, whose pixels
// spread over more addresses anyway and whose scan runs in one workgroup).
static int uv_counter_copies(int64_t NT) {
  int r = 32;
  while (r > 1 && NT * r > 65536) r >>= 1;
  return r;
}

// Workspace of the adjoint by texture: count [R][NT] | offset (NT + 1) | cursor [R][NT] |
// bucket (MP pixels).
static size_t uv_layout(int64_t NT, int64_t MP, size_t (&off)[4]) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const size_t copies = (size_t)uv_counter_copies(NT);
  off[0] = 0;                                       // count
  off[1] = off[0] + up((size_t)NT * copies * 4);    // offset
  off[2] = off[1] + up((size_t)(NT + 1) * 4);       // cursor
  off[3] = off[2] + up((size_t)NT * copies * 4);    // bucket
  return off[3] + up((size_t)MP * 4);
}

static bool uv_by_texture_fits(int64_t NT, int64_t THW, size_t esz) {
  return NT <= kUvMaxTextures && THW * (int64_t)esz <= kUvLdsBytes;
}

// The image pixels bucketed by texture (a function of quad_idx alone) into `workspace`
// (uv_layout bytes): offset[t] .. offset[t + 1] - 1 of `list` are texture t's pixels.
static int build_uv_buckets(const int64_t* quad, void* workspace, int NT, int MP,
                            hipStream_t stream) {
  size_t off[4];
  uv_layout(NT, MP, off);
  char* ws = static_cast<char*>(workspace);
  int* count = reinterpret_cast<int*>(ws + off[0]);
  int* offset = reinterpret_cast<int*>(ws + off[1]);
  int* cursor = reinterpret_cast<int*>(ws + off[2]);
  int* list = reinterpret_cast<int*>(ws + off[3]);
  int rc = zero_fill(count, off[1], stream);
  if (rc != SDK_OK) return rc;
  const dim3 pixel_grid((unsigned)ceil_div(MP, kBlock));
  const int copies = uv_counter_copies(NT);
  launch(uv_count_kernel, pixel_grid, dim3(kBlock), stream, quad, NT, MP, copies, count);
  launch(uv_scan_kernel, dim3(1), dim3(kBlock), stream, (const int*)count, NT, copies, offset,
         cursor);
  launch(uv_fill_kernel, pixel_grid, dim3(kBlock), stream, quad, NT, MP, copies, cursor, list);
  SDK_LAUNCH_CHECK("resample_to_uv_maps(bucket)");
  return SDK_OK;
}

// The adjoint: with a workspace (and textures that fit in LDS) by texture, see
// uv_texture_scatter_kernel; otherwise a zero fill and atomic adds in memory.
// prebuilt: `workspace` already holds the buckets of this quad_idx (build_uv_buckets).
template <typename T>
static int launch_uv_scatter(const T* in, const int64_t* quad, const T* uv, T* textures,
                             void* workspace, size_t workspace_bytes, int64_t planes, int NT,
                             int TH, int TW, int MP, int interp, hipStream_t stream,
                             bool prebuilt = false) {
  const int THW = TH * TW;
  size_t off[4];
  if (workspace != nullptr && uv_by_texture_fits(NT, THW, sizeof(T)) &&
      workspace_bytes >= uv_layout(NT, MP, off)) {
    char* ws = static_cast<char*>(workspace);
    int* offset = reinterpret_cast<int*>(ws + off[1]);
    int* list = reinterpret_cast<int*>(ws + off[3]);
    int rc = prebuilt ? SDK_OK : build_uv_buckets(quad, workspace, NT, MP, stream);
    if (rc != SDK_OK) return rc;
    // planes per workgroup: as many as LDS holds while the grid still fills the GPU; few
    // textures: several workgroups share one and add their parts to a zero-filled output
    int pl = 1;
    while (pl < 4 && (size_t)(2 * pl) * THW * sizeof(T) <= (size_t)kUvLdsBytes &&
           (int64_t)NT * ceil_div(planes, 2 * pl) >= 1024)
      pl *= 2;
    const int64_t groups = (int64_t)NT * ceil_div(planes, pl);
    const int split = (int)std::min<int64_t>(64, std::max<int64_t>(1, 512 / groups));
    if (ceil_div(planes, pl) > 65535)
      return fail(SDK_ERR_UNSUPPORTED, "resample_to_uv_maps: batch*channels = %lld too large",
                  (long long)planes);
    if (split > 1) {
      rc = zero_fill(textures, sizeof(T) * (size_t)planes * NT * THW, stream);
      if (rc != SDK_OK) return rc;
    }
    const dim3 grid((unsigned)NT, (unsigned)ceil_div(planes, pl), (unsigned)split);
#define UVS(PLv)                                                                              \
  SDK_DISPATCH_INTERP_ONLY(interp, (uv_texture_scatter_kernel<T, INTERP, PLv>                 \
                                    <<<grid, dim3(kUvBlock), (size_t)PLv * THW * sizeof(T), stream>>>( \
                                        in, uv, (const int*)offset, (const int*)list, textures, \
                                        (int)planes, NT, TH, TW, MP)))
    if (pl == 4) UVS(4); else if (pl == 2) UVS(2); else UVS(1);
#undef UVS
    SDK_LAUNCH_CHECK("resample_to_uv_maps(by texture)");
    return SDK_OK;
  }
  int rc = zero_fill(textures, sizeof(T) * (size_t)planes * NT * THW, stream);
  if (rc != SDK_OK) return rc;
  SDK_DISPATCH_INTERP_ONLY(interp,
                           (launch((uv_scatter_kernel<T, INTERP>),
                                   dim3(banded_grid_x(MP), (unsigned)ceil_div(planes, kPC)),
                                   dim3(kBlock), stream, in, quad, uv, textures, (int)planes, NT,
                                   TH, TW, MP, (const int*)nullptr)));
  SDK_LAUNCH_CHECK("resample_to_uv_maps");
  return SDK_OK;
}

static UnpoolTiling unpool_tiling(int H, int W) {
  UnpoolTiling ut;
  ut.H = H;
  ut.W = W;
  ut.tw_shift = 7;
  while ((kUpTile >> ut.tw_shift) > H && ut.tw_shift < kUpTileLog2) ++ut.tw_shift;   // flat images: wider tiles
  while (ut.tw_shift > 0 && (1 << (ut.tw_shift - 1)) >= W) --ut.tw_shift;   // narrow ones: taller
  ut.tiles_x = (int)ceil_div(W, ut.TW());
  ut.tiles_y = (int)ceil_div(H, ut.TH());
  return ut;
}

// Workspace of the tiled unpool: gate (first 256 bytes) and the tile windows, cleared together.
static size_t unpool_layout(const UnpoolTiling& ut) {
  return 256 + (size_t)ut.tiles_x * ut.tiles_y * 8 * sizeof(int);
}

// ... followed, when the workspace has room for it, by the table of the row-band kernels
// (pool_band.hpp), whose first word is the device-side verdict "the band kernels do this map".
static size_t unpool_layout_with_bands(const UnpoolTiling& ut) {
  return unpool_layout(ut) + unpool_band_table_bytes(ut.H, ut.W);
}

// ... and, where they fit (unpool_band_taps_bytes), by the bands' packed taps, 256-byte aligned.
static size_t unpool_layout_with_taps(const UnpoolTiling& ut) {
  const size_t t = unpool_band_taps_bytes(ut.H, ut.W);
  const size_t base = unpool_layout_with_bands(ut);
  return t != 0 ? ((base + 255) & ~(size_t)255) + t : base;
}

// The packed taps inside a region laid out as above, nullptr where it has no room for them.
static unsigned* unpool_taps_at(void* region, size_t region_bytes, const UnpoolTiling& ut) {
  if (unpool_band_taps_bytes(ut.H, ut.W) == 0 || region_bytes < unpool_layout_with_taps(ut))
    return nullptr;
  return reinterpret_cast<unsigned*>(static_cast<char*>(region) +
                                     ((unpool_layout_with_bands(ut) + 255) & ~(size_t)255));
}

// Whether the row-band kernels take this element type, interpolation and shape at all.
template <typename T>
static bool unpool_bands_possible(int H, int W, int OH, int OW, int K, int P, int interp) {
  return sizeof(T) == 4 && P == 0 && interp != 1 && interp != 2 &&
         unpool_band_shape(H, W, OH, OW, K);
}

// The tile windows of the tiled unpool (a function of the map alone) into `workspace`
// (unpool_layout bytes), gate word cleared; with workspace_bytes >= unpool_layout_with_bands
// the band table as well; where its verdict is 1 every call on this map runs the band kernels
// and the window kernels return at once.
// seen: scratch for the band table's build (unpool_band_build), or nullptr.
template <typename T>
static int build_unpool_windows(const T* map, void* workspace, size_t workspace_bytes, int H, int W,
                                int OH, int OW, int K, int P, int interp, hipStream_t stream,
                                unsigned* seen) {
  const UnpoolTiling ut = unpool_tiling(H, W);
  char* ws = static_cast<char*>(workspace);
  int* win = reinterpret_cast<int*>(ws + 256);
  const bool with_table = workspace_bytes >= unpool_layout_with_bands(ut);
  int rc = zero_fill(ws, with_table ? unpool_layout_with_bands(ut) : unpool_layout(ut), stream);
  if (rc != SDK_OK) return rc;
  const int* skip = nullptr;
  if (with_table && unpool_bands_possible<T>(H, W, OH, OW, K, P, interp)) {
    int* table = reinterpret_cast<int*>(ws + unpool_layout(ut));
    // (average unpooling is the caller that lends `seen`; its taps are laid out for it)
    unpool_band_build((const float*)map, table, H, W, OH, OW, K, stream, seen,
                      unpool_taps_at(workspace, workspace_bytes, ut), seen != nullptr);
    SDK_LAUNCH_CHECK("mapped_max_unpool(band table)");
    skip = table;
  }
  const int64_t samples = (int64_t)OH * OW * K;
  const dim3 grid_s((unsigned)ceil_div(samples, kBlock));
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((unpool_window_kernel<T, INTERP, WEIGHTED, false>), grid_s,
                              dim3(kBlock), stream, map, samples, P, K, OW, ut, win, skip)));
  SDK_LAUNCH_CHECK("mapped_max_unpool(anchors)");
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((unpool_window_kernel<T, INTERP, WEIGHTED, true>), grid_s,
                              dim3(kBlock), stream, map, samples, P, K, OW, ut, win, skip)));
  SDK_LAUNCH_CHECK("mapped_max_unpool(windows)");
  return SDK_OK;
}

template <typename T>
static int launch_unpool(const T* gout, const int64_t* indices, const T* map, const T* wts, T* gin,
                         void* workspace, size_t workspace_bytes, int64_t planes, int H, int W,
                         int OH, int OW, int K, int P, int interp, hipStream_t stream,
                         bool prebuilt = false, bool bands_known = false) {
  const int64_t HW = (int64_t)H * W, M = (int64_t)OH * OW;
  const int q = pts(P);
  const size_t total = (size_t)planes * M;
  const int64_t map_elems = M * K * q * 2;
  const int* gate = nullptr;   // non-null: device flag, != 0 means "use the atomic scatter"
  const UnpoolTiling ut = unpool_tiling(H, W);
  const int64_t tiles = (int64_t)ut.tiles_x * ut.tiles_y;
  constexpr int PLMAX = kUpBytes / (kUpTile * (int)sizeof(T));
  // plane groups: many short workgroups (the kernel is bound by instruction issue and by the
  // latency of each workgroup's few dependent loads; one or two passes each measured best)
  int64_t groups = std::max<int64_t>(1, std::min<int64_t>(ceil_div(planes, PLMAX),
                                                          ceil_div(16384, tiles)));
  const int64_t per_group = ceil_div(ceil_div(planes, groups), PLMAX) * PLMAX;
  groups = ceil_div(planes, per_group);
  if (workspace != nullptr && workspace_bytes >= unpool_layout(ut) &&
      map_elems < ((int64_t)1 << 31) &&
      tiles < ((int64_t)1 << 27) && groups <= 65535) {
    char* ws = static_cast<char*>(workspace);
    int* g = reinterpret_cast<int*>(ws);
    int* win = reinterpret_cast<int*>(ws + 256);
    // the row-band kernels, where the workspace holds their table and they take the call
    const int* bands = nullptr;
    if (workspace_bytes >= unpool_layout_with_bands(ut) &&
        unpool_bands_possible<T>(H, W, OH, OW, K, P, interp))
      bands = reinterpret_cast<const int*>(ws + unpool_layout(ut));
    int rc;
    if (bands_known) {
      // The caller has read the plan's verdict (sdk_mapped_max_unpool_plan_bands): the band
      // kernel does the call, and the one kernel after it runs only for indices that name
      // another pixel's sample.  The gate word is zero between calls (the plan build clears
      // it, the stray kernel clears it again after use).
      if constexpr (sizeof(T) == 4) {
        if (bands == nullptr)
          return fail(SDK_ERR_INVALID_ARGUMENT, "mapped_max_unpool_planned_bands: no band table for this shape");
        unpool_band_launch(false, (const float*)gout, indices, (const float*)map, (float*)gin,
                           bands, unpool_taps_at(workspace, workspace_bytes, ut), g, planes, H,
                           W, OH, OW, K, stream);
        SDK_LAUNCH_CHECK("mapped_max_unpool(bands)");
        const int64_t blocks = std::min<int64_t>(ceil_div((int64_t)total, kBlock), 4096);
        SDK_DISPATCH_INTERP(interp, P,
                            (launch((mapped_max_unpool_stray_kernel<T, INTERP, WEIGHTED>),
                                    dim3((unsigned)blocks), dim3(kBlock), stream, gout, indices,
                                    map, wts, gin, total, H, W, (int)M, K, P, map_elems, g)));
        SDK_LAUNCH_CHECK("mapped_max_unpool(stray)");
        return SDK_OK;
      } else {
        return fail(SDK_ERR_INVALID_ARGUMENT, "mapped_max_unpool_planned_bands: no band table for this type");
      }
    }
    if (prebuilt) {
      // the windows are there; the gate word is this call's own (the kernels raise it)
      rc = zero_fill(ws, 256, stream);
    } else {
      rc = build_unpool_windows<T>(map, workspace, workspace_bytes, H, W, OH, OW, K, P, interp,
                                   stream);
    }
    if (rc != SDK_OK) return rc;
    if (bands != nullptr) {
      if constexpr (sizeof(T) == 4) {
        unpool_band_launch(false, (const float*)gout, indices, (const float*)map, (float*)gin,
                           bands, unpool_taps_at(workspace, workspace_bytes, ut), g, planes, H,
                           W, OH, OW, K, stream);
        SDK_LAUNCH_CHECK("mapped_max_unpool(bands)");
      }
    }
    const dim3 grid_t((unsigned)tiles, (unsigned)groups);
    SDK_DISPATCH_INTERP(interp, P,
                        (launch((unpool_tiles_kernel<T, INTERP, WEIGHTED>), grid_t, dim3(kBlock),
                                stream, gout, indices, map, wts, (const int*)win, gin, g, ut,
                                (int)planes, (int)per_group, (int)M, OW, K, P, map_elems,
                                bands)));
    SDK_LAUNCH_CHECK("mapped_max_unpool(tiles)");
    gate = g;
  }
  int rc = zero_fill_gated(gin, sizeof(T) * (size_t)planes * HW, stream, gate);
  if (rc != SDK_OK) return rc;
  // as a fallback (seldom run): fewer workgroups, each striding over the elements
  const int64_t blocks = ceil_div((int64_t)total, kBlock);
  const dim3 grid_el((unsigned)(gate != nullptr ? std::min<int64_t>(blocks, 4096) : blocks));
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((mapped_max_unpool_kernel<T, INTERP, WEIGHTED>), grid_el,
                              dim3(kBlock), stream, gout, indices, map, wts, gin, total, H, W,
                              (int)M, P, map_elems, gate)));
  SDK_LAUNCH_CHECK("mapped_max_unpool");
  return SDK_OK;
}

// ---------------------------------------------------------------------------
// The splat of a convolution's column matrix (common/mapped_im2col.h:89-158) as a gather over
// the inverted map, for conv_product.hip (declared in conv_product.hpp).  The map is inverted
// into lists of exact length: per image element u the entries offset[u] .. offset[u + 1] - 1 of
// (sample, coefficient), sample = m * K + k, sorted by sample, so
// every element is written once, with its bias, as a sum in a fixed order; no list can
// overflow.  count -> scan -> fill -> sort build them; they depend on the map alone.
// ---------------------------------------------------------------------------
namespace {

// FILL = false: counts the taps of every image element; true: writes them at the slots the
// scanned counts reserve.  Taps outside the image and taps with a zero coefficient are left
// out (by both passes alike).
template <int INTERP, bool WEIGHTED, bool FILL>
__global__ __launch_bounds__(kBlock) void col2im_invert_kernel(
    const float* __restrict__ map, const float* __restrict__ wts, int H, int W, int M, int K,
    int P, int* __restrict__ counter, int* __restrict__ src, float* __restrict__ co) {
  const int pix = blockIdx.x * kBlock + threadIdx.x;   // sample m * K + k
  if (pix >= M * K) return;
  const int q = WEIGHTED ? P : 1;
  PointTaps<float, INTERP> t;
  for (int p = 0; p < q; ++p) {
    const size_t s = (size_t)pix * q + p;
    t.set(map[s * 2], map[s * 2 + 1], H, W);
    const float wt = WEIGHTED ? wts[s] : 1.0f;
#pragma unroll
    for (int i = 0; i < PointTaps<float, INTERP>::N; ++i) {
      const float c = INTERP == 0 ? wt : t.w[i] * wt;
      if (t.off[i] >= 0 && c != 0.0f) {
        const int slot = atomicAdd(&counter[t.off[i]], 1);
        if constexpr (FILL) {
          src[slot] = pix;
          co[slot] = c;
        }
      }
    }
  }
}

// Exclusive scan of n counters in three launches: per tile of 4096 counters (16 consecutive
// ones per thread) the tile's sum; the sums scanned by one workgroup; every tile again, now
// from its first slot.  offset[i] = cursor[i] = first slot of element i, offset[n] = all slots.
constexpr int kScanPer = 16;
constexpr int kScanTile = kBlock * kScanPer;

// The block's exclusive scan of one value per thread; *total: the block's sum (every thread).
__device__ __forceinline__ int block_exclusive_scan(int mine, int* total) {
  __shared__ int wave_sum[kBlock / 64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int incl = mine;
#pragma unroll
  for (int d = 1; d < 64; d <<= 1) {
    const int below = __shfl_up(incl, d);
    if (lane >= d) incl += below;
  }
  __syncthreads();   // (wave_sum may still be read from the previous call)
  if (lane == 63) wave_sum[wave] = incl;
  __syncthreads();
  int before = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kBlock / 64; ++w) {
    before += w < wave ? wave_sum[w] : 0;
    all += wave_sum[w];
  }
  *total = all;
  return before + incl - mine;
}

__global__ __launch_bounds__(kBlock) void scan_tile_sums_kernel(const int* __restrict__ count,
                                                                int n, int* __restrict__ sums) {
  const int first = blockIdx.x * kScanTile + threadIdx.x * kScanPer;
  int mine = 0;
#pragma unroll
  for (int i = 0; i < kScanPer; ++i) mine += first + i < n ? count[first + i] : 0;
  int total;
  block_exclusive_scan(mine, &total);
  if (threadIdx.x == 0) sums[blockIdx.x] = total;
}

// One workgroup: sums[0 .. tiles) -> their exclusive scan, in place.
__global__ __launch_bounds__(kBlock) void scan_sums_kernel(int* __restrict__ sums, int tiles) {
  int run = 0;
  for (int base = 0; base < tiles; base += kBlock) {
    const int i = base + threadIdx.x;
    const int mine = i < tiles ? sums[i] : 0;
    int total;
    const int before = block_exclusive_scan(mine, &total);
    if (i < tiles) sums[i] = run + before;
    run += total;
  }
}

__global__ __launch_bounds__(kBlock) void scan_apply_kernel(const int* __restrict__ count, int n,
                                                            const int* __restrict__ sums,
                                                            int* __restrict__ offset,
                                                            int* __restrict__ cursor) {
  const int first = blockIdx.x * kScanTile + threadIdx.x * kScanPer;
  int c[kScanPer];
  int mine = 0;
#pragma unroll
  for (int i = 0; i < kScanPer; ++i) {
    c[i] = first + i < n ? count[first + i] : 0;
    mine += c[i];
  }
  int total;
  int run = sums[blockIdx.x] + block_exclusive_scan(mine, &total);
#pragma unroll
  for (int i = 0; i < kScanPer; ++i) {
    if (first + i < n) {
      offset[first + i] = run;
      cursor[first + i] = run;
    }
    run += c[i];
    if (first + i == n - 1) offset[n] = run;
  }
}

// Every element's entries sorted by source, then coefficient (the fill appends in the order
// its atomics are served); selection sort in place, the lists are short.
__global__ __launch_bounds__(kBlock) void col2im_sort_kernel(const int* __restrict__ offset,
                                                             int* __restrict__ src,
                                                             float* __restrict__ co, int HW) {
  const int u = blockIdx.x * kBlock + threadIdx.x;
  if (u >= HW) return;
  const int beg = offset[u], end = offset[u + 1];
  for (int i = beg; i + 1 < end; ++i) {
    int best = i, bs = src[i];
    float bc = co[i];
    const int first_s = bs;
    const float first_c = bc;
    for (int j = i + 1; j < end; ++j) {
      const int sj = src[j];
      const float cj = co[j];
      if (sj < bs || (sj == bs && cj < bc)) {
        best = j;
        bs = sj;
        bc = cj;
      }
    }
    if (best != i) {
      src[best] = first_s;
      co[best] = first_c;
      src[i] = bs;
      co[i] = bc;
    }
  }
}

// col holds the products channels-last, col[b][sample][c]: a wave reads the Cg values of an
// entry's sample as one run (lane = channel) and owns 16 consecutive image elements, whose
// entries are one run of the lists: the lanes fetch that run together (lane l entry l), every
// lane works out which of the 16 elements its entry belongs to, and the wave then walks the
// entries in order, eight value reads in flight at a time, handing a finished element's sums
// to an LDS tile from which the workgroup's 64 elements x 64 channels leave transposed, as
// runs along the image.  grid (blocks of 64 image elements, batch).
constexpr int kC2iTargets = 64;

__global__ __launch_bounds__(kBlock) void col2im_gather_kernel(
    const float* __restrict__ col, const int* __restrict__ offset, const int* __restrict__ src,
    const float* __restrict__ co, const float* __restrict__ bias, float* __restrict__ img, int Cg,
    int HW, size_t samples) {
  __shared__ float tile[kC2iTargets * (kC2iTargets + 1)];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int u0 = blockIdx.x * kC2iTargets;
  const float* col_b = col + (size_t)blockIdx.y * samples * Cg;
  float* img_b = img + (size_t)blockIdx.y * Cg * HW;
  // the 17 list boundaries of the wave's 16 elements (elements past the image: empty lists)
  const int w_first = u0 + 16 * wave;
  const int my_off = offset[min(w_first + min(lane, 16), HW)];
  const int beg_w = __builtin_amdgcn_readlane(my_off, 0);
  const int end_w = __builtin_amdgcn_readlane(my_off, 16);
  for (int c0 = 0; c0 < Cg; c0 += 64) {
    const int cc = min(c0 + lane, Cg - 1);
#pragma unroll
    for (int t = 0; t < 16; ++t) tile[(16 * wave + t) * (kC2iTargets + 1) + lane] = 0.0f;
    float acc = 0.0f;
    int cur = -1;   // element (0..15) the sums belong to
    for (int base = beg_w; base < end_w; base += 64) {
      const int e = base + lane;
      const bool on = e < end_w;
      const int s_l = on ? src[e] : 0;
      const float w_l = on ? co[e] : 0.0f;
      int t_l = 0;   // boundaries 1..16 at or below e: the element of entry e
#pragma unroll
      for (int q = 1; q <= 16; ++q) t_l += __builtin_amdgcn_readlane(my_off, q) <= e ? 1 : 0;
      const int n_here = min(64, end_w - base);   // (uniform)
      for (int i0 = 0; i0 < n_here; i0 += 8) {
        float v[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int s_i = __builtin_amdgcn_readlane(s_l, min(i0 + i, n_here - 1));
          v[i] = col_b[(size_t)s_i * Cg + cc];
        }
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          if (i0 + i < n_here) {
            const int t_i = __builtin_amdgcn_readlane(t_l, i0 + i);
            const float w_i = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w_l), i0 + i));
            if (t_i != cur) {
              if (cur >= 0) tile[(16 * wave + cur) * (kC2iTargets + 1) + lane] = acc;
              acc = 0.0f;
              cur = t_i;
            }
            acc += w_i * v[i];
          }
        }
      }
    }
    if (cur >= 0) tile[(16 * wave + cur) * (kC2iTargets + 1) + lane] = acc;
    __syncthreads();
    // thread (wave, lane): element u0 + lane, channels c0 + wave + 4 i
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int c = c0 + wave + 4 * i;
      if (c < Cg && u0 + lane < HW)
        img_b[(size_t)c * HW + u0 + lane] =
            tile[lane * (kC2iTargets + 1) + wave + 4 * i] + (bias != nullptr ? bias[c] : 0.0f);
    }
    __syncthreads();
  }
}

struct Col2imLists {
  int *count, *offset, *cursor, *sums, *src;
  float* co;
  size_t bytes;
};
Col2imLists col2im_lists_at(void* base, int H, int W, int M, int K, int P, int interp) {
  auto up = [](size_t v) { return (v + 255) & ~(size_t)255; };
  const size_t HW = (size_t)H * W;
  const size_t nnz = (size_t)M * K * (P > 0 ? P : 1) * (interp == 0 ? 1 : 4);
  char* b = static_cast<char*>(base);
  Col2imLists l;
  size_t at = 0;
  l.count = reinterpret_cast<int*>(b + at);
  at += up(HW * 4);
  l.offset = reinterpret_cast<int*>(b + at);
  at += up((HW + 1) * 4);
  l.cursor = reinterpret_cast<int*>(b + at);
  at += up(HW * 4);
  l.sums = reinterpret_cast<int*>(b + at);   // one per 4096 elements (the scan's tile sums)
  at += up((HW / 4096 + 1) * 4);
  l.src = reinterpret_cast<int*>(b + at);
  at += up(nnz * 4);
  l.co = reinterpret_cast<float*>(b + at);
  at += up(nnz * 4);
  l.bytes = at;
  return l;
}

}  // namespace

size_t col2im_lists_bytes(int H, int W, int M, int K, int P, int interp) {
  const int64_t nnz = (int64_t)M * K * (P > 0 ? P : 1) * (interp == 0 ? 1 : 4);
  if ((int64_t)H * W >= ((int64_t)1 << 31) - 1 || nnz >= ((int64_t)1 << 31)) return 0;
  return col2im_lists_at(nullptr, H, W, M, K, P, interp).bytes;
}

int col2im_lists_build(const float* map, const float* wts, void* lists, int H, int W, int M,
                       int K, int P, int interp, hipStream_t stream) {
  const Col2imLists l = col2im_lists_at(lists, H, W, M, K, P, interp);
  const int HW = H * W;
  int rc = zero_fill(l.count, sizeof(int) * (size_t)HW, stream);
  if (rc) return rc;
  const dim3 grid((unsigned)ceil_div((int64_t)M * K, kBlock));
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((col2im_invert_kernel<INTERP, WEIGHTED, false>), grid, dim3(kBlock),
                              stream, map, wts, H, W, M, K, P, l.count, (int*)nullptr,
                              (float*)nullptr)));
  const int tiles = (int)ceil_div(HW, kScanTile);
  launch(scan_tile_sums_kernel, dim3((unsigned)tiles), dim3(kBlock), stream, (const int*)l.count,
         HW, l.sums);
  launch(scan_sums_kernel, dim3(1), dim3(kBlock), stream, l.sums, tiles);
  launch(scan_apply_kernel, dim3((unsigned)tiles), dim3(kBlock), stream, (const int*)l.count, HW,
         (const int*)l.sums, l.offset, l.cursor);
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((col2im_invert_kernel<INTERP, WEIGHTED, true>), grid, dim3(kBlock),
                              stream, map, wts, H, W, M, K, P, l.cursor, l.src, l.co)));
  launch(col2im_sort_kernel, dim3((unsigned)ceil_div(HW, kBlock)), dim3(kBlock), stream,
         (const int*)l.offset, l.src, l.co, HW);
  SDK_LAUNCH_CHECK("mapped_conv(inverted map)");
  return SDK_OK;
}

int col2im_from_lists(const float* col, const float* bias, float* img, const void* lists,
                      int64_t planes, int channels, int H, int W, int M, int K, int P, int interp,
                      hipStream_t stream) {
  const Col2imLists l = col2im_lists_at(const_cast<void*>(lists), H, W, M, K, P, interp);
  const int HW = H * W;
  const int64_t batch = planes / channels;
  if (batch > 65535)
    return fail(SDK_ERR_UNSUPPORTED, "mapped_conv: batch %lld too large", (long long)batch);
  launch(col2im_gather_kernel, dim3((unsigned)ceil_div(HW, kC2iTargets), (unsigned)batch),
         dim3(kBlock), stream, col, (const int*)l.offset, (const int*)l.src, (const float*)l.co,
         bias, img, channels, HW, (size_t)M * K);
  SDK_LAUNCH_CHECK("mapped_conv(col2im)");
  return SDK_OK;
}

// Shared with the convolution drivers (declared in conv_internal.hpp).
template <typename T>
int launch_mapped_im2col(const T* im, const T* map, const T* wts, T* col, int64_t planes, int H,
                         int W, int M, int K, int P, int interp, hipStream_t stream) {
  const dim3 grid(banded_grid_x(M), (unsigned)ceil_div(planes, kPC));
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((mapped_im2col_kernel<T, INTERP, WEIGHTED>), grid,
                                          dim3(kBlock), stream, im, map, wts, col, (int)planes,
                                          H, W, M, K, P)));
  SDK_LAUNCH_CHECK("mapped_im2col");
  return SDK_OK;
}

// `im` must already hold the values to accumulate onto (zeros, or a bias fill).
template <typename T>
int launch_mapped_col2im(const T* col, const T* map, const T* wts, T* im, int64_t planes, int H,
                         int W, int M, int K, int P, int interp, hipStream_t stream) {
  const dim3 grid(banded_grid_x(M), (unsigned)ceil_div(planes, kPC));
  SDK_DISPATCH_INTERP(interp, P,
                      (launch((mapped_col2im_kernel<T, INTERP, WEIGHTED>), grid,
                                          dim3(kBlock), stream, col, map, wts, im, (int)planes,
                                          H, W, M, K, P)));
  SDK_LAUNCH_CHECK("mapped_col2im");
  return SDK_OK;
}

template int launch_mapped_im2col<float>(const float*, const float*, const float*, float*, int64_t,
                                         int, int, int, int, int, int, hipStream_t);
template int launch_mapped_im2col<double>(const double*, const double*, const double*, double*,
                                          int64_t, int, int, int, int, int, int, hipStream_t);
template int launch_mapped_col2im<float>(const float*, const float*, const float*, float*, int64_t,
                                         int, int, int, int, int, int, hipStream_t);
template int launch_mapped_col2im<double>(const double*, const double*, const double*, double*,
                                          int64_t, int, int, int, int, int, int, hipStream_t);

}  // namespace sdk

using namespace sdk;

// ---------------------------------------------------------------------------
// The unpool for callers that cannot allocate: the tile-window scratch of
// sdk_mapped_max_unpool lives in a file-scope device array.  The array's name is
// only a host-side handle: its device address is asked for once per device and
// that pointer is what the fill kernel and the unpool kernels receive.
// ---------------------------------------------------------------------------
static constexpr int kStaticUnpoolTiles = SDK_MAPPED_MAX_UNPOOL_STATIC_MAX_TILES;   // of 2048 pixels
// tile windows, then 48 KB for the row-band table (planes of up to 4000 rows of bands)
static constexpr size_t kStaticUnpoolBytes = 256 + (size_t)kStaticUnpoolTiles * 8 * sizeof(int) +
                                             49152;
static __device__ __align__(256) unsigned char scratch[kStaticUnpoolBytes];

static constexpr int kMaxDevices = 64;
static std::mutex scratch_mutex;
static void* scratch_ptr[kMaxDevices] = {};   // per device: every GPU holds its own copy of the array

// The current device's address of `scratch` (resolved on the first call on that device).
static int static_unpool_scratch(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess)
    return fail(SDK_ERR_DEVICE, "mapped_max_unpool_static: hipGetDevice: %s",
                hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices)
    return fail(SDK_ERR_UNSUPPORTED, "mapped_max_unpool_static: device %d (at most %d devices)",
                dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || p == nullptr)
      return fail(SDK_ERR_DEVICE, "mapped_max_unpool_static: hipGetSymbolAddress: %s",
                  hipGetErrorString(e));
    scratch_ptr[dev] = p;
  }
  *out = scratch_ptr[dev];
  return SDK_OK;
}

// ---------------------------------------------------------------------------
// C entry points.
// ---------------------------------------------------------------------------
extern "C" {

int sdk_resample_from_map(const void* image, const void* sample_map, const void* interp_weights,
                          void* out, int64_t batch, int64_t channels, int64_t height,
                          int64_t width, int64_t map_height, int64_t map_width,
                          int32_t num_interp_pts, int32_t interp, int32_t dtype,
                          sdk_stream_t stream) {
  SDK_REQUIRE(image && sample_map && out, "resample_from_map: NULL pointer");
  SDK_REQUIRE(num_interp_pts >= 0 && (num_interp_pts == 0 || interp_weights),
              "resample_from_map: weighted map needs interp_weights");
  SDK_REQUIRE(batch >= 0 && channels >= 0, "resample_from_map: negative size");
  int rc = check_plane(height, width, "resample_from_map(image)");
  if (rc) return rc;
  rc = check_plane(map_height, map_width, "resample_from_map(map)");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  rc = check_grid_y(planes, "resample_from_map");
  if (rc) return rc;
  SDK_DISPATCH_DTYPE(dtype, return launch_resample_from_map<T>(
                                (const T*)image, (const T*)sample_map, (const T*)interp_weights,
                                (T*)out, planes, (int)height, (int)width,
                                (int)(map_height * map_width), num_interp_pts, interp,
                                (hipStream_t)stream));
  return SDK_OK;
}

size_t sdk_resample_to_map_workspace_bytes(int64_t height, int64_t width, int32_t dtype) {
  if (height < 1 || width < 1 || height * width >= ((int64_t)1 << 31)) return 0;
  size_t off[4];
  // the inverse lists, then the tile windows of the tiled average unpooling
  return inverse_layout(height * width, dtype == SDK_F64 ? 8 : 4, off) +
         unpool_layout_with_taps(unpool_tiling((int)height, (int)width));
}

static int resample_to_map_entry(const void* input, const void* sample_map,
                                 const void* interp_weights, void* out, void* weight_sum,
                                 void* workspace, size_t workspace_bytes, int64_t batch,
                                 int64_t channels, int64_t map_height, int64_t map_width,
                                 int64_t height, int64_t width, int32_t num_interp_pts,
                                 int32_t interp, int32_t dtype, sdk_stream_t stream,
                                 bool normalize, double eps) {
  SDK_REQUIRE(input && sample_map && out, "resample_to_map: NULL pointer");
  SDK_REQUIRE(!normalize || weight_sum, "resample_to_map_normalized: NULL weight_sum");
  SDK_REQUIRE(num_interp_pts >= 0 && (num_interp_pts == 0 || interp_weights),
              "resample_to_map: weighted map needs interp_weights");
  SDK_REQUIRE(batch >= 0 && channels >= 0, "resample_to_map: negative size");
  int rc = check_plane(height, width, "resample_to_map(out)");
  if (rc) return rc;
  rc = check_plane(map_height, map_width, "resample_to_map(map)");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  rc = check_grid_y(planes, "resample_to_map");
  if (rc) return rc;
  if (planes == 0 && !weight_sum) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_resample_to_map<T>(
                                (const T*)input, (const T*)sample_map, (const T*)interp_weights,
                                (T*)out, (T*)weight_sum, workspace, workspace_bytes, planes,
                                (int)height, (int)width, (int)(map_height * map_width),
                                num_interp_pts, interp, (hipStream_t)stream, normalize, eps));
  return SDK_OK;
}

int sdk_resample_to_map(const void* input, const void* sample_map, const void* interp_weights,
                        void* out, void* weight_sum, void* workspace, size_t workspace_bytes,
                        int64_t batch, int64_t channels, int64_t map_height, int64_t map_width,
                        int64_t height, int64_t width, int32_t num_interp_pts, int32_t interp,
                        int32_t dtype, sdk_stream_t stream) {
  return resample_to_map_entry(input, sample_map, interp_weights, out, weight_sum, workspace,
                               workspace_bytes, batch, channels, map_height, map_width, height,
                               width, num_interp_pts, interp, dtype, stream, false, 0.0);
}

int sdk_resample_to_map_normalized(const void* input, const void* sample_map,
                                   const void* interp_weights, void* out, void* weight_sum,
                                   void* workspace, size_t workspace_bytes, double eps,
                                   int64_t batch, int64_t channels, int64_t map_height,
                                   int64_t map_width, int64_t height, int64_t width,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   sdk_stream_t stream) {
  return resample_to_map_entry(input, sample_map, interp_weights, out, weight_sum, workspace,
                               workspace_bytes, batch, channels, map_height, map_width, height,
                               width, num_interp_pts, interp, dtype, stream, true, eps);
}

static int check_uv(const void* a, const void* quad, const void* uv, const void* b,
                    int64_t batch, int64_t channels, int64_t num_textures, int64_t tex_height,
                    int64_t tex_width, int64_t height, int64_t width, const char* what) {
  if (batch < 0 || channels < 0) return fail(SDK_ERR_INVALID_ARGUMENT, "%s: negative size", what);
  // an empty batch has no tensors to point at
  if (batch * channels > 0 && (!a || !quad || !uv || !b))
    return fail(SDK_ERR_INVALID_ARGUMENT, "%s: NULL pointer", what);
  if (num_textures < 1 || num_textures >= ((int64_t)1 << 31))
    return fail(SDK_ERR_INVALID_ARGUMENT, "%s: num_textures = %lld", what, (long long)num_textures);
  int rc = check_plane(tex_height, tex_width, what);
  if (rc) return rc;
  rc = check_plane(num_textures * tex_height, tex_width, what);   // all texels of one plane
  if (rc) return rc;
  rc = check_plane(height, width, what);
  if (rc) return rc;
  return check_grid_y(batch * channels, what);
}

int sdk_resample_from_uv_maps(const void* textures, const int64_t* quad_idx, const void* tex_uv,
                              void* out, int64_t batch, int64_t channels, int64_t num_textures,
                              int64_t tex_height, int64_t tex_width, int64_t height,
                              int64_t width, int32_t interp, int32_t dtype, sdk_stream_t stream) {
  int rc = check_uv(textures, quad_idx, tex_uv, out, batch, channels, num_textures, tex_height,
                    tex_width, height, width, "resample_from_uv_maps");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_uv_gather<T>(
                                (const T*)textures, quad_idx, (const T*)tex_uv, (T*)out, planes,
                                (int)num_textures, (int)tex_height, (int)tex_width,
                                (int)(height * width), interp, (hipStream_t)stream));
  return SDK_OK;
}

size_t sdk_resample_to_uv_maps_workspace_bytes(int64_t num_textures, int64_t tex_height,
                                               int64_t tex_width, int64_t height, int64_t width,
                                               int32_t dtype) {
  if (num_textures < 1 || tex_height < 1 || tex_width < 1 || height < 1 || width < 1 ||
      height * width >= ((int64_t)1 << 31))
    return 0;
  if (!uv_by_texture_fits(num_textures, tex_height * tex_width, dtype == SDK_F64 ? 8 : 4)) return 0;
  size_t off[4];
  return uv_layout(num_textures, height * width, off);
}

int sdk_resample_to_uv_maps(const void* input, const int64_t* quad_idx, const void* tex_uv,
                            void* textures, void* workspace, size_t workspace_bytes,
                            int64_t batch, int64_t channels, int64_t num_textures,
                            int64_t tex_height, int64_t tex_width, int64_t height, int64_t width,
                            int32_t interp, int32_t dtype, sdk_stream_t stream) {
  int rc = check_uv(input, quad_idx, tex_uv, textures, batch, channels, num_textures, tex_height,
                    tex_width, height, width, "resample_to_uv_maps");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_uv_scatter<T>(
                                (const T*)input, quad_idx, (const T*)tex_uv, (T*)textures,
                                workspace, workspace_bytes, planes, (int)num_textures,
                                (int)tex_height, (int)tex_width, (int)(height * width), interp,
                                (hipStream_t)stream));
  return SDK_OK;
}

int sdk_resample_to_uv_maps_plan_build(const int64_t* quad_idx, void* plan, size_t plan_bytes,
                                       int64_t num_textures, int64_t tex_height,
                                       int64_t tex_width, int64_t height, int64_t width,
                                       int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(quad_idx && plan, "resample_to_uv_maps_plan_build: NULL pointer");
  const size_t need = sdk_resample_to_uv_maps_workspace_bytes(num_textures, tex_height, tex_width,
                                                              height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "resample_to_uv_maps_plan_build: plan of %zu bytes, need %zu",
                plan_bytes, need);
  return build_uv_buckets(quad_idx, plan, (int)num_textures, (int)(height * width),
                          (hipStream_t)stream);
}

int sdk_resample_to_uv_maps_planned(const void* input, const int64_t* quad_idx, const void* tex_uv,
                                    void* textures, const void* plan, size_t plan_bytes,
                                    int64_t batch, int64_t channels, int64_t num_textures,
                                    int64_t tex_height, int64_t tex_width, int64_t height,
                                    int64_t width, int32_t interp, int32_t dtype,
                                    sdk_stream_t stream) {
  int rc = check_uv(input, quad_idx, tex_uv, textures, batch, channels, num_textures, tex_height,
                    tex_width, height, width, "resample_to_uv_maps_planned");
  if (rc) return rc;
  SDK_REQUIRE(plan, "resample_to_uv_maps_planned: NULL pointer");
  const size_t need = sdk_resample_to_uv_maps_workspace_bytes(num_textures, tex_height, tex_width,
                                                              height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "resample_to_uv_maps_planned: plan of %zu bytes, need %zu",
                plan_bytes, need);
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_uv_scatter<T>(
                                (const T*)input, quad_idx, (const T*)tex_uv, (T*)textures,
                                const_cast<void*>(plan), plan_bytes, planes, (int)num_textures,
                                (int)tex_height, (int)tex_width, (int)(height * width), interp,
                                (hipStream_t)stream, true));
  return SDK_OK;
}

int sdk_normalize_by_weight_sum(void* data, const void* weight_sum, double eps, int64_t planes,
                                int64_t plane_size, int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(data && weight_sum, "normalize_by_weight_sum: NULL pointer");
  SDK_REQUIRE(planes >= 0 && plane_size >= 0, "normalize_by_weight_sum: negative size");
  const size_t total = (size_t)planes * plane_size;
  if (total == 0) return SDK_OK;
  const int blocks = (int)std::min<int64_t>(ceil_div((int64_t)total, kBlock), 256 * 16);
  SDK_DISPATCH_DTYPE(dtype, (launch(normalize_kernel<T>, dim3(blocks), dim3(kBlock),
                                                (hipStream_t)stream, (T*)data,
                                                (const T*)weight_sum, (T)eps, (size_t)plane_size,
                                                total, (const int*)nullptr)));
  SDK_LAUNCH_CHECK("normalize_by_weight_sum");
  return SDK_OK;
}

static int check_mapped(const void* a, const void* map, const void* wts, const void* b,
                        int64_t batch, int64_t channels, int64_t height, int64_t width,
                        int64_t out_pixels, int64_t K, int32_t P, const char* what) {
  SDK_REQUIRE(a && map && b, "%s: NULL pointer", what);
  SDK_REQUIRE(P >= 0 && (P == 0 || wts), "%s: weighted map needs interp_weights", what);
  SDK_REQUIRE(batch >= 0 && channels >= 0 && K >= 1, "%s: bad size", what);
  SDK_REQUIRE(out_pixels > 0 && out_pixels < ((int64_t)1 << 31), "%s: bad output pixel count",
              what);
  int rc = check_plane(height, width, what);
  if (rc) return rc;
  return check_grid_y(batch * channels, what);
}

int sdk_mapped_im2col(const void* image, const void* sample_map, const void* interp_weights,
                      void* columns, int64_t batch, int64_t channels, int64_t height,
                      int64_t width, int64_t out_pixels, int64_t kernel_size,
                      int32_t num_interp_pts, int32_t interp, int32_t dtype, sdk_stream_t stream) {
  int rc = check_mapped(image, sample_map, interp_weights, columns, batch, channels, height, width,
                        out_pixels, kernel_size, num_interp_pts, "mapped_im2col");
  if (rc) return rc;
  if (batch * channels == 0) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_mapped_im2col<T>(
                                (const T*)image, (const T*)sample_map, (const T*)interp_weights,
                                (T*)columns, batch * channels, (int)height, (int)width,
                                (int)out_pixels, (int)kernel_size, num_interp_pts, interp,
                                (hipStream_t)stream));
  return SDK_OK;
}

int sdk_mapped_col2im(const void* columns, const void* sample_map, const void* interp_weights,
                      void* image, int64_t batch, int64_t channels, int64_t height,
                      int64_t width, int64_t out_pixels, int64_t kernel_size,
                      int32_t num_interp_pts, int32_t interp, int32_t dtype, sdk_stream_t stream) {
  int rc = check_mapped(columns, sample_map, interp_weights, image, batch, channels, height, width,
                        out_pixels, kernel_size, num_interp_pts, "mapped_col2im");
  if (rc) return rc;
  if (batch * channels == 0) return SDK_OK;
  const size_t esz = dtype == SDK_F64 ? 8 : 4;
  rc = zero_fill(image, esz * (size_t)(batch * channels) * height * width, (hipStream_t)stream);
  if (rc) return rc;
  SDK_DISPATCH_DTYPE(dtype, return launch_mapped_col2im<T>(
                                (const T*)columns, (const T*)sample_map,
                                (const T*)interp_weights, (T*)image, batch * channels, (int)height,
                                (int)width, (int)out_pixels, (int)kernel_size, num_interp_pts,
                                interp, (hipStream_t)stream));
  return SDK_OK;
}

int sdk_mapped_max_pool(const void* input, const void* sample_map, const void* interp_weights,
                        void* out, int64_t* indices, int64_t batch, int64_t channels,
                        int64_t height, int64_t width, int64_t out_height, int64_t out_width,
                        int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                        int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(indices, "mapped_max_pool: NULL indices");
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_max_pool: bad output size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(input, sample_map, interp_weights, out, batch, channels, height, width, M,
                        kernel_size, num_interp_pts, "mapped_max_pool");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  if (dtype == SDK_F32 && num_interp_pts == 0 && interp != 1 && interp != 2 &&
      pool_band_launch(false, (const float*)input, (const float*)sample_map, (float*)out, indices,
                       planes, (int)height, (int)width, (int)out_height, (int)out_width,
                       (int)kernel_size, (hipStream_t)stream)) {
    SDK_LAUNCH_CHECK("mapped_max_pool");
    return SDK_OK;
  }
  const dim3 grid(banded_grid_x(M), (unsigned)ceil_div(planes, kPC));
  SDK_DISPATCH_DTYPE(
      dtype,
      SDK_DISPATCH_INTERP(interp, num_interp_pts,
                          (launch((mapped_max_pool_kernel<T, INTERP, WEIGHTED>), grid,
                                              dim3(kBlock), (hipStream_t)stream,
                                              (const T*)input, (const T*)sample_map,
                                              (const T*)interp_weights, (T*)out, indices,
                                              (int)planes, (int)height, (int)width, (int)M,
                                              (int)kernel_size, num_interp_pts))));
  SDK_LAUNCH_CHECK("mapped_max_pool");
  return SDK_OK;
}

int sdk_mapped_avg_pool(const void* input, const void* sample_map, const void* interp_weights,
                        void* out, int64_t batch, int64_t channels, int64_t height, int64_t width,
                        int64_t out_height, int64_t out_width, int64_t kernel_size,
                        int32_t num_interp_pts, int32_t interp, int32_t dtype,
                        sdk_stream_t stream) {
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_avg_pool: bad output size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(input, sample_map, interp_weights, out, batch, channels, height, width, M,
                        kernel_size, num_interp_pts, "mapped_avg_pool");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  if (dtype == SDK_F32 && num_interp_pts == 0 && interp != 1 && interp != 2 &&
      pool_band_launch(true, (const float*)input, (const float*)sample_map, (float*)out, nullptr,
                       planes, (int)height, (int)width, (int)out_height, (int)out_width,
                       (int)kernel_size, (hipStream_t)stream)) {
    SDK_LAUNCH_CHECK("mapped_avg_pool");
    return SDK_OK;
  }
  const dim3 grid(banded_grid_x(M), (unsigned)ceil_div(planes, kPC));
  SDK_DISPATCH_DTYPE(
      dtype,
      SDK_DISPATCH_INTERP(interp, num_interp_pts,
                          (launch((mapped_avg_pool_kernel<T, INTERP, WEIGHTED>), grid,
                                  dim3(kBlock), (hipStream_t)stream, (const T*)input,
                                  (const T*)sample_map, (const T*)interp_weights, (T*)out,
                                  (int)planes, (int)height, (int)width, (int)M, (int)kernel_size,
                                  num_interp_pts))));
  SDK_LAUNCH_CHECK("mapped_avg_pool");
  return SDK_OK;
}

int sdk_mapped_avg_unpool(const void* grad_output, const void* sample_map,
                          const void* interp_weights, void* grad_input, void* workspace,
                          size_t workspace_bytes, int64_t batch, int64_t channels, int64_t height,
                          int64_t width, int64_t out_height, int64_t out_width,
                          int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                          int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_avg_unpool: bad pooled size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(grad_output, sample_map, interp_weights, grad_input, batch, channels,
                        height, width, M, kernel_size, num_interp_pts, "mapped_avg_unpool");
  if (rc) return rc;
  SDK_REQUIRE(M * kernel_size < ((int64_t)1 << 31), "mapped_avg_unpool: too many samples");
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_resample_to_map<T>(
                                (const T*)grad_output, (const T*)sample_map,
                                (const T*)interp_weights, (T*)grad_input, (T*)nullptr, workspace,
                                workspace_bytes, planes, (int)height, (int)width,
                                (int)(M * kernel_size), num_interp_pts, interp,
                                (hipStream_t)stream, false, 0.0, (int)kernel_size, false, 0,
                                (int)out_width));
  return SDK_OK;
}

size_t sdk_mapped_max_unpool_workspace_bytes(int64_t height, int64_t width, int32_t dtype) {
  if (height < 1 || width < 1 || height * width >= ((int64_t)1 << 31)) return 0;
  (void)dtype;
  return unpool_layout_with_taps(unpool_tiling((int)height, (int)width));
}

int sdk_mapped_max_unpool(const void* grad_output, const int64_t* indices, const void* sample_map,
                          const void* interp_weights, void* grad_input, void* workspace,
                          size_t workspace_bytes, int64_t batch, int64_t channels, int64_t height,
                          int64_t width, int64_t out_height, int64_t out_width,
                          int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                          int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(indices, "mapped_max_unpool: NULL indices");
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_max_unpool: bad pooled size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(grad_output, sample_map, interp_weights, grad_input, batch, channels,
                        height, width, M, kernel_size, num_interp_pts, "mapped_max_unpool");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_REQUIRE(ceil_div(planes * M, kBlock) < ((int64_t)1 << 31),
              "mapped_max_unpool: too many elements");
  SDK_DISPATCH_DTYPE(dtype, return launch_unpool<T>(
                                (const T*)grad_output, indices, (const T*)sample_map,
                                (const T*)interp_weights, (T*)grad_input, workspace,
                                workspace_bytes, planes, (int)height, (int)width, (int)out_height,
                                (int)out_width, (int)kernel_size, num_interp_pts, interp,
                                (hipStream_t)stream));
}

int sdk_mapped_max_unpool_static(const void* grad_output, const int64_t* indices,
                                 const void* sample_map, const void* interp_weights,
                                 void* grad_input, int64_t batch, int64_t channels,
                                 int64_t height, int64_t width, int64_t out_height,
                                 int64_t out_width, int64_t kernel_size, int32_t num_interp_pts,
                                 int32_t interp, int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(height >= 1 && width >= 1 && height * width < ((int64_t)1 << 31),
              "mapped_max_unpool_static: bad plane size");
  const size_t need = unpool_layout(unpool_tiling((int)height, (int)width));
  if (need > 256 + (size_t)kStaticUnpoolTiles * 8 * sizeof(int))
    return fail(SDK_ERR_WORKSPACE,
                "mapped_max_unpool_static: a %lld x %lld plane needs %zu bytes of tile windows, "
                "the built-in scratch holds %zu (%d tiles of %d pixels); use sdk_mapped_max_unpool "
                "with a workspace",
                (long long)height, (long long)width, need, kStaticUnpoolBytes, kStaticUnpoolTiles,
                kUpTile);
  void* ws = nullptr;
  int rc = static_unpool_scratch(&ws);
  if (rc) return rc;
  return sdk_mapped_max_unpool(grad_output, indices, sample_map, interp_weights, grad_input, ws,
                               kStaticUnpoolBytes, batch, channels, height, width, out_height,
                               out_width, kernel_size, num_interp_pts, interp, dtype, stream);
}

int sdk_mapped_gather_at_index(const void* image, const int64_t* indices, const void* sample_map,
                               const void* interp_weights, void* out, int64_t batch,
                               int64_t channels, int64_t height, int64_t width,
                               int64_t out_height, int64_t out_width, int64_t kernel_size,
                               int32_t num_interp_pts, int32_t interp, int32_t dtype,
                               sdk_stream_t stream) {
  SDK_REQUIRE(indices, "mapped_gather_at_index: NULL indices");
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_gather_at_index: bad pooled size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(image, sample_map, interp_weights, out, batch, channels, height, width, M,
                        kernel_size, num_interp_pts, "mapped_gather_at_index");
  if (rc) return rc;
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  const size_t total = (size_t)planes * M;
  const int64_t map_elems = M * kernel_size * pts(num_interp_pts) * 2;
  const int blocks = (int)std::min<int64_t>(ceil_div((int64_t)total, kBlock), 256 * 32);
  SDK_DISPATCH_DTYPE(
      dtype, SDK_DISPATCH_INTERP(
                 interp, num_interp_pts,
                 (launch((mapped_gather_at_index_kernel<T, INTERP, WEIGHTED>), dim3(blocks),
                         dim3(kBlock), (hipStream_t)stream, (const T*)image, indices,
                         (const T*)sample_map, (const T*)interp_weights, (T*)out, total,
                         (int)height, (int)width, (int)M, num_interp_pts, map_elems))));
  SDK_LAUNCH_CHECK("mapped_gather_at_index");
  return SDK_OK;
}

// ---------------------------------------------------------------------------
// Plans of the scatter direction: the map-dependent scratch of sdk_resample_to_map,
// sdk_mapped_avg_unpool and sdk_mapped_max_unpool, built once and kept by the caller.
// ---------------------------------------------------------------------------
int sdk_resample_to_map_plan_build(const void* sample_map, const void* interp_weights, void* plan,
                                   size_t plan_bytes, int64_t map_height, int64_t map_width,
                                   int64_t height, int64_t width, int64_t kernel_size,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   sdk_stream_t stream) {
  SDK_REQUIRE(sample_map && plan, "resample_to_map_plan_build: NULL pointer");
  SDK_REQUIRE(num_interp_pts >= 0 && (num_interp_pts == 0 || interp_weights),
              "resample_to_map_plan_build: weighted map needs interp_weights");
  SDK_REQUIRE(kernel_size >= 1, "resample_to_map_plan_build: bad kernel_size");
  int rc = check_plane(height, width, "resample_to_map_plan_build(out)");
  if (rc) return rc;
  SDK_REQUIRE(map_height > 0 && map_width > 0 &&
                  map_height * map_width * kernel_size < ((int64_t)1 << 31),
              "resample_to_map_plan_build: bad map size");
  const size_t need = sdk_resample_to_map_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "resample_to_map_plan_build: plan of %zu bytes, need %zu",
                plan_bytes, need);
  SDK_DISPATCH_DTYPE(dtype, return build_inverse_lists<T>(
                                (const T*)sample_map, (const T*)interp_weights, plan, plan_bytes,
                                (int)height, (int)width,
                                (int)(map_height * map_width * kernel_size), num_interp_pts,
                                interp, (int)kernel_size, (int)map_width, (hipStream_t)stream));
  return SDK_OK;
}

int sdk_resample_plan_complete(const void* plan, size_t plan_bytes, sdk_stream_t stream,
                               int32_t* complete) {
  SDK_REQUIRE(plan && complete && plan_bytes >= 256, "resample_plan_complete: bad argument");
  int gate[2] = {1, 0};   // sources that found a list full; "the tiled average unpooling runs"
  hipError_t e = hipMemcpyAsync(gate, plan, sizeof(gate), hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess)
    return fail(SDK_ERR_DEVICE, "resample_plan_complete: %s", hipGetErrorString(e));
  *complete = (gate[0] == 0 ? 1 : 0) | (gate[1] != 0 ? 2 : 0);
  return SDK_OK;
}

int sdk_resample_to_map_planned(const void* input, const void* sample_map,
                                const void* interp_weights, void* out, void* weight_sum,
                                void* plan, size_t plan_bytes, int32_t plan_complete,
                                int32_t normalize, double eps, int64_t batch, int64_t channels,
                                int64_t map_height, int64_t map_width, int64_t height,
                                int64_t width, int32_t num_interp_pts, int32_t interp,
                                int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(input && out && plan, "resample_to_map_planned: NULL pointer");
  SDK_REQUIRE(plan_complete || sample_map,
              "resample_to_map_planned: the map is needed unless the plan is known complete");
  SDK_REQUIRE(!normalize || weight_sum, "resample_to_map_planned: NULL weight_sum");
  SDK_REQUIRE(num_interp_pts >= 0 && (num_interp_pts == 0 || interp_weights || plan_complete),
              "resample_to_map_planned: weighted map needs interp_weights");
  SDK_REQUIRE(batch >= 0 && channels >= 0, "resample_to_map_planned: negative size");
  int rc = check_plane(height, width, "resample_to_map_planned(out)");
  if (rc) return rc;
  rc = check_plane(map_height, map_width, "resample_to_map_planned(map)");
  if (rc) return rc;
  const size_t need = sdk_resample_to_map_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "resample_to_map_planned: plan of %zu bytes, need %zu",
                plan_bytes, need);
  const int64_t planes = batch * channels;
  rc = check_grid_y(planes, "resample_to_map_planned");
  if (rc) return rc;
  if (planes == 0 && !weight_sum) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_resample_to_map<T>(
                                (const T*)input, (const T*)sample_map, (const T*)interp_weights,
                                (T*)out, (T*)weight_sum, plan, plan_bytes, planes, (int)height,
                                (int)width, (int)(map_height * map_width), num_interp_pts, interp,
                                (hipStream_t)stream, normalize != 0, eps, 1, true,
                                plan_complete != 0));
  return SDK_OK;
}

int sdk_mapped_avg_unpool_planned(const void* grad_output, const void* sample_map,
                                  const void* interp_weights, void* grad_input, void* plan,
                                  size_t plan_bytes, int32_t plan_complete, int64_t batch,
                                  int64_t channels, int64_t height, int64_t width,
                                  int64_t out_height, int64_t out_width, int64_t kernel_size,
                                  int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                  sdk_stream_t stream) {
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_avg_unpool_planned: bad pooled size");
  SDK_REQUIRE(plan, "mapped_avg_unpool_planned: NULL plan");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(grad_output, sample_map, interp_weights, grad_input, batch, channels,
                        height, width, M, kernel_size, num_interp_pts,
                        "mapped_avg_unpool_planned");
  if (rc) return rc;
  SDK_REQUIRE(M * kernel_size < ((int64_t)1 << 31), "mapped_avg_unpool_planned: too many samples");
  const size_t need = sdk_resample_to_map_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "mapped_avg_unpool_planned: plan of %zu bytes, need %zu",
                plan_bytes, need);
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_DISPATCH_DTYPE(dtype, return launch_resample_to_map<T>(
                                (const T*)grad_output, (const T*)sample_map,
                                (const T*)interp_weights, (T*)grad_input, (T*)nullptr, plan,
                                plan_bytes, planes, (int)height, (int)width,
                                (int)(M * kernel_size), num_interp_pts, interp,
                                (hipStream_t)stream, false, 0.0, (int)kernel_size, true,
                                plan_complete, (int)out_width));
  return SDK_OK;
}

int sdk_mapped_max_unpool_plan_build(const void* sample_map, void* plan, size_t plan_bytes,
                                     int64_t height, int64_t width, int64_t out_height,
                                     int64_t out_width, int64_t kernel_size,
                                     int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                     sdk_stream_t stream) {
  SDK_REQUIRE(sample_map && plan, "mapped_max_unpool_plan_build: NULL pointer");
  SDK_REQUIRE(out_height > 0 && out_width > 0 && kernel_size >= 1 && num_interp_pts >= 0,
              "mapped_max_unpool_plan_build: bad size");
  int rc = check_plane(height, width, "mapped_max_unpool_plan_build");
  if (rc) return rc;
  const int64_t M = out_height * out_width;
  SDK_REQUIRE(M < ((int64_t)1 << 31) &&
                  M * kernel_size * pts(num_interp_pts) * 2 < ((int64_t)1 << 31),
              "mapped_max_unpool_plan_build: map too large for a plan");
  const size_t need = sdk_mapped_max_unpool_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "mapped_max_unpool_plan_build: plan of %zu bytes, need %zu",
                plan_bytes, need);
  SDK_DISPATCH_DTYPE(dtype, return build_unpool_windows<T>(
                                (const T*)sample_map, plan, plan_bytes, (int)height, (int)width,
                                (int)out_height, (int)out_width, (int)kernel_size, num_interp_pts,
                                interp, (hipStream_t)stream));
  return SDK_OK;
}

int sdk_mapped_max_unpool_planned(const void* grad_output, const int64_t* indices,
                                  const void* sample_map, const void* interp_weights,
                                  void* grad_input, void* plan, size_t plan_bytes, int64_t batch,
                                  int64_t channels, int64_t height, int64_t width,
                                  int64_t out_height, int64_t out_width, int64_t kernel_size,
                                  int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                  sdk_stream_t stream) {
  SDK_REQUIRE(indices && plan, "mapped_max_unpool_planned: NULL pointer");
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_max_unpool_planned: bad pooled size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(grad_output, sample_map, interp_weights, grad_input, batch, channels,
                        height, width, M, kernel_size, num_interp_pts, "mapped_max_unpool_planned");
  if (rc) return rc;
  const size_t need = sdk_mapped_max_unpool_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "mapped_max_unpool_planned: plan of %zu bytes, need %zu",
                plan_bytes, need);
  SDK_REQUIRE(M * kernel_size * pts(num_interp_pts) * 2 < ((int64_t)1 << 31),
              "mapped_max_unpool_planned: map too large for a plan");
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_REQUIRE(ceil_div(planes * M, kBlock) < ((int64_t)1 << 31),
              "mapped_max_unpool_planned: too many elements");
  SDK_DISPATCH_DTYPE(dtype, return launch_unpool<T>(
                                (const T*)grad_output, indices, (const T*)sample_map,
                                (const T*)interp_weights, (T*)grad_input, plan, plan_bytes, planes,
                                (int)height, (int)width, (int)out_height, (int)out_width,
                                (int)kernel_size, num_interp_pts, interp, (hipStream_t)stream,
                                true));
}

int sdk_mapped_max_unpool_plan_bands(const void* plan, size_t plan_bytes, int64_t height,
                                     int64_t width, int32_t dtype, sdk_stream_t stream,
                                     int32_t* bands) {
  SDK_REQUIRE(plan && bands, "mapped_max_unpool_plan_bands: NULL pointer");
  int rc = check_plane(height, width, "mapped_max_unpool_plan_bands");
  if (rc) return rc;
  const size_t need = sdk_mapped_max_unpool_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "mapped_max_unpool_plan_bands: plan of %zu bytes, need %zu",
                plan_bytes, need);
  *bands = 0;
  const UnpoolTiling ut = unpool_tiling((int)height, (int)width);
  if (dtype != SDK_F32 || plan_bytes < unpool_layout_with_bands(ut)) return SDK_OK;
  int verdict = 0;
  hipError_t e = hipMemcpyAsync(&verdict, static_cast<const char*>(plan) + unpool_layout(ut),
                                sizeof(int), hipMemcpyDeviceToHost, (hipStream_t)stream);
  if (e == hipSuccess) e = hipStreamSynchronize((hipStream_t)stream);
  if (e != hipSuccess)
    return fail(SDK_ERR_DEVICE, "mapped_max_unpool_plan_bands: %s", hipGetErrorString(e));
  *bands = verdict != 0 ? 1 : 0;
  return SDK_OK;
}

int sdk_mapped_max_unpool_planned_bands(const void* grad_output, const int64_t* indices,
                                        const void* sample_map, void* grad_input, void* plan,
                                        size_t plan_bytes, int64_t batch, int64_t channels,
                                        int64_t height, int64_t width, int64_t out_height,
                                        int64_t out_width, int64_t kernel_size, int32_t interp,
                                        int32_t dtype, sdk_stream_t stream) {
  SDK_REQUIRE(indices && plan, "mapped_max_unpool_planned_bands: NULL pointer");
  SDK_REQUIRE(out_height > 0 && out_width > 0, "mapped_max_unpool_planned_bands: bad pooled size");
  const int64_t M = out_height * out_width;
  int rc = check_mapped(grad_output, sample_map, nullptr, grad_input, batch, channels, height,
                        width, M, kernel_size, 0, "mapped_max_unpool_planned_bands");
  if (rc) return rc;
  const size_t need = sdk_mapped_max_unpool_workspace_bytes(height, width, dtype);
  if (need == 0 || plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "mapped_max_unpool_planned_bands: plan of %zu bytes, need %zu",
                plan_bytes, need);
  SDK_REQUIRE(M * kernel_size * 2 < ((int64_t)1 << 31),
              "mapped_max_unpool_planned_bands: map too large for a plan");
  const int64_t planes = batch * channels;
  if (planes == 0) return SDK_OK;
  SDK_REQUIRE(ceil_div(planes * M, kBlock) < ((int64_t)1 << 31),
              "mapped_max_unpool_planned_bands: too many elements");
  SDK_DISPATCH_DTYPE(dtype, return launch_unpool<T>(
                                (const T*)grad_output, indices, (const T*)sample_map,
                                (const T*)nullptr, (T*)grad_input, plan, plan_bytes, planes,
                                (int)height, (int)width, (int)out_height, (int)out_width,
                                (int)kernel_size, 0, interp, (hipStream_t)stream, true, true));
}

}  // extern "C"
