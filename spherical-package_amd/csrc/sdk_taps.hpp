// Device-side interpolation primitives: a sample coordinate is turned once into
// up to four (offset, weight) taps, which are then applied to any number of
// image planes.  Semantics follow the reference's point functions
// (ext_modules/include/core/interpolation.h:97-247, blend order :17-33, splat
// :36-61); translation units including this header must be compiled with
// -ffp-contract=off so products and sums round exactly as on the reference CPU.
//
// One deliberate difference: a tap whose weight is exactly zero is neither read
// nor written.  For finite data the result is identical (the reference adds
// 0*value); only a non-finite value under a zero weight, which the reference
// would turn into NaN, is ignored here.
#pragma once
#include <hip/hip_runtime.h>

namespace sdk {

template <typename T>
__device__ __forceinline__ void atomic_add_noret(T* addr, T v) {
  // Relaxed, device-scope; with -munsafe-fp-atomics this is one
  // global_atomic_add_f32 / _f64 without return value.
  (void)__hip_atomic_fetch_add(addr, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Float add into LDS.  The native ds_add_f32 executes at about one lane every
// three cycles per CU on gfx950; a compare-and-swap loop on the integer view of
// the word is roughly fifteen times faster (measured) and gives the same
// result, retrying only when another lane hit the same word in between.
__device__ __forceinline__ void lds_add_f32(float* addr, float v) {
  int* ip = reinterpret_cast<int*>(addr);
  int old = __hip_atomic_load(ip, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  while (true) {
    const int assumed = old;
    old = atomicCAS(ip, assumed, __float_as_int(__int_as_float(assumed) + v));
    if (old == assumed) break;
  }
}

__device__ __forceinline__ void lds_add_f64(double* addr, double v) {
  unsigned long long* ip = reinterpret_cast<unsigned long long*>(addr);
  unsigned long long old = __hip_atomic_load(ip, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  while (true) {
    const unsigned long long assumed = old;
    old = atomicCAS(ip, assumed, (unsigned long long)__double_as_longlong(
                                     __longlong_as_double((long long)assumed) + v));
    if (old == assumed) break;
  }
}
__device__ __forceinline__ void lds_add(float* addr, float v) { lds_add_f32(addr, v); }
__device__ __forceinline__ void lds_add(double* addr, double v) { lds_add_f64(addr, v); }

// N independent float adds into LDS: all loads, then all compare-and-swaps, are
// issued back to back so their latencies overlap.  A swap that lost a race (two
// lanes of the wave, or another wave, hit the same word) is repeated with the
// value the failed swap returned as the new expectation, again all pending
// words of the lane in one batch; one extra round settles the common case of
// two lanes sharing a word.
template <int N>
__device__ __forceinline__ void lds_add_f32_batch(float* base, const int (&offs)[N],
                                                  const float (&vals)[N]) {
  int old[N], got[N];
#pragma unroll
  for (int i = 0; i < N; ++i)
    old[i] = __hip_atomic_load(reinterpret_cast<int*>(base + offs[i]), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
  for (int i = 0; i < N; ++i)
    got[i] = atomicCAS(reinterpret_cast<int*>(base + offs[i]), old[i],
                       __float_as_int(__int_as_float(old[i]) + vals[i]));
  bool lost = false;
#pragma unroll
  for (int i = 0; i < N; ++i) lost |= got[i] != old[i];
  while (lost) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (got[i] != old[i]) {
        old[i] = got[i];
        got[i] = atomicCAS(reinterpret_cast<int*>(base + offs[i]), old[i],
                           __float_as_int(__int_as_float(old[i]) + vals[i]));
      }
    }
    lost = false;
#pragma unroll
    for (int i = 0; i < N; ++i) lost |= got[i] != old[i];
  }
}

// The same for pairs of floats that share an aligned 8-byte word: one 64-bit
// compare-and-swap adds both, which halves the LDS instructions per value.
__device__ __forceinline__ unsigned long long add_pair(unsigned long long w, float a, float b) {
  const float lo = __uint_as_float((unsigned)w) + a;
  const float hi = __uint_as_float((unsigned)(w >> 32)) + b;
  return (unsigned long long)__float_as_uint(lo) | ((unsigned long long)__float_as_uint(hi) << 32);
}

template <int N>
__device__ __forceinline__ void lds_add_f32x2_batch(float2* base, const int (&offs)[N],
                                                    const float (&va)[N], const float (&vb)[N]) {
  unsigned long long old[N], got[N];
#pragma unroll
  for (int i = 0; i < N; ++i)
    old[i] = __hip_atomic_load(reinterpret_cast<unsigned long long*>(base + offs[i]),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
#pragma unroll
  for (int i = 0; i < N; ++i)
    got[i] = atomicCAS(reinterpret_cast<unsigned long long*>(base + offs[i]), old[i],
                       add_pair(old[i], va[i], vb[i]));
  bool lost = false;
#pragma unroll
  for (int i = 0; i < N; ++i) lost |= got[i] != old[i];
  while (lost) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
      if (got[i] != old[i]) {
        old[i] = got[i];
        got[i] = atomicCAS(reinterpret_cast<unsigned long long*>(base + offs[i]), old[i],
                           add_pair(old[i], va[i], vb[i]));
      }
    }
    lost = false;
#pragma unroll
    for (int i = 0; i < N; ++i) lost |= got[i] != old[i];
  }
}

__device__ __forceinline__ int to_int_clamped(float v) {
  return (int)fminf(fmaxf(v, -2.0e9f), 2.0e9f);
}
__device__ __forceinline__ int to_int_clamped(double v) {
  return (int)fmin(fmax(v, -2.0e9), 2.0e9);
}
__device__ __forceinline__ float floor_t(float v) { return floorf(v); }
__device__ __forceinline__ double floor_t(double v) { return floor(v); }
// Round half away from zero, the rule of llround() used by the reference
// (core/interpolation.h:102-103).
__device__ __forceinline__ float round_t(float v) { return roundf(v); }
__device__ __forceinline__ double round_t(double v) { return round(v); }

// ((v % n) + n) % n for n > 0 (core/util.h:59-62), with the common in-range case first.
__device__ __forceinline__ int wrap_index(int v, int n) {
  if ((unsigned)v < (unsigned)n) return v;
  int r = v % n;
  return r < 0 ? r + n : r;
}

// INTERP: 0 nearest, 1 bilinear, 2 bispherical.
template <typename T, int INTERP>
struct PointTaps {
  static constexpr int N = (INTERP == 0) ? 1 : 4;
  int off[N];  // element offset inside one H x W plane, or -1 (inactive tap)
  int ty[N], tx[N];  // row and column of the tap (meaningful where off >= 0)
  T w[N];

  __device__ __forceinline__ void set(T x, T y, int H, int W) {
    if constexpr (INTERP == 0) {
      const int xi = to_int_clamped(round_t(x));
      const int yi = to_int_clamped(round_t(y));
      const bool ok = (unsigned)xi < (unsigned)W && (unsigned)yi < (unsigned)H;
      off[0] = ok ? yi * W + xi : -1;
      ty[0] = yi;
      tx[0] = xi;
      w[0] = T(1);
    } else {
      const T fx = floor_t(x), fy = floor_t(y);
      const int x1 = to_int_clamped(fx), y1 = to_int_clamped(fy);
      // Weights against the unwrapped integer neighbours x1, x1+1, y1, y1+1.
      const T A = (fy + T(1)) - y, B = (fx + T(1)) - x, C = x - fx, D = y - fy;
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
      w[0] = A * B;
      w[1] = A * C;
      w[2] = D * B;
      w[3] = D * C;
      const int r1 = y1 * W, r2 = r1 + W;
      ty[0] = ty[1] = y1;
      ty[2] = ty[3] = y1 + 1;
      tx[0] = tx[2] = c1;
      tx[1] = tx[3] = c2;
      off[0] = (x1ok && y1ok && w[0] != T(0)) ? r1 + c1 : -1;
      off[1] = (x2ok && y1ok && w[1] != T(0)) ? r1 + c2 : -1;
      off[2] = (x1ok && y2ok && w[2] != T(0)) ? r2 + c1 : -1;
      off[3] = (x2ok && y2ok && w[3] != T(0)) ? r2 + c2 : -1;
    }
  }

  // Branch-free guarded read: inactive taps read element 0 and discard it.
  static __device__ __forceinline__ T read(const T* __restrict__ plane, int o) {
    const T d = plane[o < 0 ? 0 : o];
    return o < 0 ? T(0) : d;
  }

  __device__ __forceinline__ T gather(const T* __restrict__ plane) const {
    if constexpr (INTERP == 0) {
      return read(plane, off[0]);
    } else {
      const T t0 = w[0] * read(plane, off[0]);
      const T t1 = w[1] * read(plane, off[1]);
      const T t2 = w[2] * read(plane, off[2]);
      const T t3 = w[3] * read(plane, off[3]);
      return t0 + t1 + t2 + t3;
    }
  }

  // gather() in two steps, for callers that want the reads of several planes issued before
  // the first of them is used: load() fetches the taps, blend() combines them as gather() does.
  __device__ __forceinline__ void load(const T* __restrict__ plane, T (&raw)[N]) const {
#pragma unroll
    for (int i = 0; i < N; ++i) raw[i] = plane[off[i] < 0 ? 0 : off[i]];
  }
  __device__ __forceinline__ T blend(const T (&raw)[N]) const {
    if constexpr (INTERP == 0) {
      return off[0] < 0 ? T(0) : raw[0];
    } else {
      const T t0 = w[0] * (off[0] < 0 ? T(0) : raw[0]);
      const T t1 = w[1] * (off[1] < 0 ? T(0) : raw[1]);
      const T t2 = w[2] * (off[2] < 0 ? T(0) : raw[2]);
      const T t3 = w[3] * (off[3] < 0 ? T(0) : raw[3]);
      return t0 + t1 + t2 + t3;
    }
  }

  __device__ __forceinline__ void scatter(T* __restrict__ plane, T v) const {
    if constexpr (INTERP == 0) {
      if (off[0] >= 0) atomic_add_noret(plane + off[0], v);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (off[i] >= 0) atomic_add_noret(plane + off[i], w[i] * v);
    }
  }
};

// Applies one map sample (1 point, or P weighted points accumulated in
// ascending order: core/resample.h:144-161) to PC planes that are `stride`
// elements apart.  Planes j >= np are not touched (acc[j] = 0).
// The reads of all PC planes are issued before the first of them is used (load, then blend).
// Left to itself the compiler, where the results feed a chain of compares (the running
// maximum of a pooling window) or a weighted sum, sinks every read next to its use and waits
// for each in turn: up to 32 round trips to memory per sample instead of one.
template <typename T, int INTERP, bool WEIGHTED, int PC>
__device__ __forceinline__ void gather_sample(const T* __restrict__ base, size_t stride, int np,
                                              const T* __restrict__ coords,
                                              const T* __restrict__ wts, int P, int H, int W,
                                              T (&acc)[PC]) {
  PointTaps<T, INTERP> t;
  constexpr int N = PointTaps<T, INTERP>::N;
  const int q = WEIGHTED ? P : 1;
#pragma unroll
  for (int j = 0; j < PC; ++j) acc[j] = T(0);
  for (int p = 0; p < q; ++p) {
    t.set(coords[2 * p], coords[2 * p + 1], H, W);
    T wt = T(1);
    if constexpr (WEIGHTED) wt = wts[p];
    T raw[PC][N];
#pragma unroll
    for (int j = 0; j < PC; ++j) t.load(base + (size_t)(j < np ? j : 0) * stride, raw[j]);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < PC; ++j) {
      const T v = t.blend(raw[j]);
      if constexpr (WEIGHTED) {
        if (j < np) acc[j] += wt * v;
      } else {
        acc[j] = j < np ? v : T(0);
      }
    }
  }
}

// Adjoint of gather_sample (core/resample.h:127-141): splats val[j] into plane j.
template <typename T, int INTERP, bool WEIGHTED, int PC>
__device__ __forceinline__ void scatter_sample(T* __restrict__ base, size_t stride, int np,
                                               const T* __restrict__ coords,
                                               const T* __restrict__ wts, int P, int H, int W,
                                               const T (&val)[PC]) {
  PointTaps<T, INTERP> t;
  if constexpr (!WEIGHTED) {
    t.set(coords[0], coords[1], H, W);
#pragma unroll
    for (int j = 0; j < PC; ++j)
      if (j < np) t.scatter(base + (size_t)j * stride, val[j]);
  } else {
    for (int p = 0; p < P; ++p) {
      t.set(coords[2 * p], coords[2 * p + 1], H, W);
      const T wt = wts[p];
#pragma unroll
      for (int j = 0; j < PC; ++j)
        if (j < np) t.scatter(base + (size_t)j * stride, wt * val[j]);
    }
  }
}

}  // namespace sdk
