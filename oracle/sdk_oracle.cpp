// CPU oracle for the mapped-operation backend.  TEST INFRASTRUCTURE ONLY.
//
// This file restates, in plain C++17/OpenMP with a C ABI, the CPU algorithm of
// the reference package for mapped gather/scatter operations.  It is used by
// the tests, the smoke check and the benchmark's CPU-baseline leg as the
// checker the HIP kernels are compared with.  No product code path may call
// it: the shipped library has no CPU fallback.
//
// Every function cites the reference file:line it follows (paths relative to
// the reference tree).  Arithmetic order matters for bit-exact parity, so the
// interpolation formulas keep the reference's operand and summation order and
// this file must be compiled with -ffp-contract=off.
//
// Pinning (what independently fixes each function's behaviour) is recorded in
// the test-suite next to the tests themselves:
//   gather (nearest / bilinear / bispherical, weighted)  reference known-answer
//       vectors (tests/test_resample.py) + torch grid_sample closed form +
//       compiled-reference fixtures
//   scatter, col2im, unpool   adjoint identity <gather(x),y> = <x,scatter(y)> +
//       compiled-reference fixtures
//   im2col / conv / transposed conv   reference known-answer vectors
//       (tests/test_mapped_convolution.py, test_mapped_transposed_convolution.py)
//       + F.conv2d special case + compiled-reference fixtures
//   max pool values: reference known-answer vectors; argmax index encoding and
//       the CPU initial-value quirk: compiled-reference fixtures.
//   average pool / unpool: reference known-answer vector (tests/test_mapped_pooling.py:110-132)
//       + "mean over k of the pinned im2col rows" + adjoint identity + compiled-reference
//       fixtures (weighted, nearest, bispherical).
//   sample-map generation: closed forms in pixel units (grid, inverse equirectangular), the
//       forward gnomonic projection of every sample giving back its tangent-plane offset,
//       centre sample = the pixel, stride = sub-sampling, float32 against float64.
//   gather at index (gradient of unpooling): adjoint identity with the pinned unpool, and
//       "pooling's value is the gather at pooling's own index".
//   voting resample: compiled-reference fixtures + brute force with numpy's bincount.
//   UV resampling: compiled-reference fixtures + "per texture it is the pinned gather" +
//       adjoint identity (the reference's test-suite holds no vector for it).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>
#include <cfloat>
#include <omp.h>

namespace {

enum Interp : int { NEAREST = 0, BILINEAR = 1, BISPHERICAL = 2 };  // enums.h:12-16

// core/util.h:59-62
inline int64_t wrap_index(int64_t v, int64_t n) { return ((v % n) + n) % n; }

template <typename T>
inline void atomic_accumulate(T* addr, T v) {  // core/util.h:36-43 (CPU branch)
#pragma omp atomic
  *addr += v;
}

// ---------------------------------------------------------------------------
// Point gather.  core/interpolation.h:97-114 (nearest), :137-162 (bilinear),
// :191-218 (bispherical), blend at :17-33; dispatch core/resample.h:63-89.
// ---------------------------------------------------------------------------
template <typename T>
inline T gather_point(const T* plane, T x, T y, int64_t H, int64_t W, int interp) {
  if (interp == BILINEAR || interp == BISPHERICAL) {
    const int64_t x1 = (int64_t)std::floor(x);
    const int64_t y1 = (int64_t)std::floor(y);
    const int64_t x2 = x1 + 1;
    const int64_t y2 = y1 + 1;
    const bool y1ok = y1 >= 0 && y1 <= H - 1;
    const bool y2ok = y2 >= 0 && y2 <= H - 1;
    int64_t c1 = x1, c2 = x2;
    bool x1ok, x2ok;
    if (interp == BISPHERICAL) {
      c1 = wrap_index(x1, W);
      c2 = wrap_index(x2, W);
      x1ok = x2ok = true;
    } else {
      x1ok = x1 >= 0 && x1 <= W - 1;
      x2ok = x2 >= 0 && x2 <= W - 1;
    }
    const T d11 = (x1ok && y1ok) ? plane[y1 * W + c1] : T(0);
    const T d21 = (x2ok && y1ok) ? plane[y1 * W + c2] : T(0);
    const T d12 = (x1ok && y2ok) ? plane[y2 * W + c1] : T(0);
    const T d22 = (x2ok && y2ok) ? plane[y2 * W + c2] : T(0);
    const T A = y2 - y, B = x2 - x, C = x - x1, D = y - y1;
    const T t11 = A * B * d11;
    const T t21 = A * C * d21;
    const T t12 = D * B * d12;
    const T t22 = D * C * d22;
    return t11 + t21 + t12 + t22;
  }
  // NEAREST is also the reference's `default:` branch (core/resample.h:72-76).
  const int64_t xi = std::llround(double(x));
  const int64_t yi = std::llround(double(y));
  const bool ok = xi >= 0 && xi <= W - 1 && yi >= 0 && yi <= H - 1;
  return ok ? plane[yi * W + xi] : T(0);
}

// ---------------------------------------------------------------------------
// Point scatter (adjoint of gather_point).  core/interpolation.h:117-134,
// :165-188, :221-247, splat at :36-61; dispatch core/resample.h:35-60.
// ---------------------------------------------------------------------------
template <typename T>
inline void scatter_point(T v, T* plane, T x, T y, int64_t H, int64_t W, int interp) {
  if (interp == BILINEAR || interp == BISPHERICAL) {
    const int64_t x1 = (int64_t)std::floor(x);
    const int64_t y1 = (int64_t)std::floor(y);
    const int64_t x2 = x1 + 1;
    const int64_t y2 = y1 + 1;
    const bool y1ok = y1 >= 0 && y1 <= H - 1;
    const bool y2ok = y2 >= 0 && y2 <= H - 1;
    int64_t c1 = x1, c2 = x2;
    bool x1ok, x2ok;
    if (interp == BISPHERICAL) {
      c1 = wrap_index(x1, W);
      c2 = wrap_index(x2, W);
      x1ok = x2ok = true;
    } else {
      x1ok = x1 >= 0 && x1 <= W - 1;
      x2ok = x2 >= 0 && x2 <= W - 1;
    }
    const T A = y2 - y, B = x2 - x, C = x - x1, D = y - y1;
    if (x1ok && y1ok) atomic_accumulate(plane + y1 * W + c1, A * B * v);
    if (x2ok && y1ok) atomic_accumulate(plane + y1 * W + c2, A * C * v);
    if (x1ok && y2ok) atomic_accumulate(plane + y2 * W + c1, D * B * v);
    if (x2ok && y2ok) atomic_accumulate(plane + y2 * W + c2, D * C * v);
    return;
  }
  const int64_t xi = std::llround(double(x));
  const int64_t yi = std::llround(double(y));
  if (xi >= 0 && xi <= W - 1 && yi >= 0 && yi <= H - 1)
    atomic_accumulate(plane + yi * W + xi, v);
}

// One map sample = 1 point (P == 0, unweighted) or P weighted points.
// core/resample.h:144-161 (gather: acc += w_i * point, ascending i) and
// :127-141 (scatter: splat w_i * v for each i).
template <typename T>
inline T gather_sample(const T* plane, const T* coords, const T* wts, int P,
                       int64_t H, int64_t W, int interp) {
  if (P == 0) return gather_point(plane, coords[0], coords[1], H, W, interp);
  T acc = T(0);
  for (int i = 0; i < P; ++i)
    acc += wts[i] * gather_point(plane, coords[2 * i], coords[2 * i + 1], H, W, interp);
  return acc;
}

template <typename T>
inline void scatter_sample(T v, T* plane, const T* coords, const T* wts, int P,
                           int64_t H, int64_t W, int interp) {
  if (P == 0) {
    scatter_point(v, plane, coords[0], coords[1], H, W, interp);
    return;
  }
  for (int i = 0; i < P; ++i)
    scatter_point(wts[i] * v, plane, coords[2 * i], coords[2 * i + 1], H, W, interp);
}

inline int pts(int P) { return P == 0 ? 1 : P; }

// ---------------------------------------------------------------------------
// resample_from_map: out[b,c,my,mx] = gather(image[b,c], map[my,mx]).
// common/resample.h:34-52 (:85-107 weighted); loop cpp/resample.h:33-50;
// batch loop src/cpp/resample_layer.cpp:38-69.
// ---------------------------------------------------------------------------
template <typename T>
void resample_from_map(const T* image, const T* map, const T* wts, T* out, int64_t B,
                       int64_t C, int64_t H, int64_t W, int64_t MH, int64_t MW, int P,
                       int interp) {
  const int64_t n = C * MH * MW, mp = MH * MW, q = pts(P);
  for (int64_t b = 0; b < B; ++b) {
    const T* img_b = image + b * C * H * W;
    T* out_b = out + b * n;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
      const int64_t c = i / mp, pix = i % mp;
      out_b[i] = gather_sample(img_b + c * H * W, map + pix * q * 2,
                               wts ? wts + pix * q : nullptr, P, H, W, interp);
    }
  }
}

// resample_to_map: zero-filled out[b,c] receives in[b,c,my,mx] at map[my,mx].
// common/resample.h:11-31 (:55-82 weighted); cpp/resample.h:13-30;
// src/cpp/resample_layer.cpp:7-36 (zero fill :17-18).
template <typename T>
void resample_to_map(const T* in, const T* map, const T* wts, T* out, int64_t B,
                     int64_t C, int64_t MH, int64_t MW, int64_t H, int64_t W, int P,
                     int interp) {
  const int64_t n = C * MH * MW, mp = MH * MW, q = pts(P);
  std::memset(out, 0, sizeof(T) * B * C * H * W);
  for (int64_t b = 0; b < B; ++b) {
    const T* in_b = in + b * n;
    T* out_b = out + b * C * H * W;
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
      const int64_t c = i / mp, pix = i % mp;
      scatter_sample(in_b[i], out_b + c * H * W, map + pix * q * 2,
                     wts ? wts + pix * q : nullptr, P, H, W, interp);
    }
  }
}

// ---------------------------------------------------------------------------
// UV resampling.  Per image pixel: texture quad[y,x] of plane c (plane = NT textures of
// TH x TW), point uv[y,x] interpolated inside that texture alone.
// common/resample.h:132-158 (gather), :160-187 (adjoint); loops cpp/resample.h:124-166;
// batch loops and zero fill src/cpp/uv_resample_layer.cpp:7-72.
// A texture index outside [0, NT) is skipped (the reference would index out of bounds).
// ---------------------------------------------------------------------------
template <typename T>
void resample_from_uv(const T* tex, const int64_t* quad, const T* uv, T* out, int64_t B,
                      int64_t C, int64_t NT, int64_t TH, int64_t TW, int64_t H, int64_t W,
                      int interp) {
  const int64_t hw = H * W, thw = TH * TW;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * hw; ++i) {
    const int64_t pix = i % hw, plane = i / hw, t = quad[pix];
    out[i] = (t < 0 || t >= NT) ? T(0)
                                : gather_point(tex + (plane * NT + t) * thw, uv[pix * 2],
                                               uv[pix * 2 + 1], TH, TW, interp);
  }
}

template <typename T>
void resample_to_uv(const T* in, const int64_t* quad, const T* uv, T* tex, int64_t B, int64_t C,
                    int64_t NT, int64_t TH, int64_t TW, int64_t H, int64_t W, int interp) {
  const int64_t hw = H * W, thw = TH * TW;
  std::memset(tex, 0, sizeof(T) * B * C * NT * thw);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * hw; ++i) {
    const int64_t pix = i % hw, plane = i / hw, t = quad[pix];
    if (t < 0 || t >= NT) continue;
    scatter_point(in[i], tex + (plane * NT + t) * thw, uv[pix * 2], uv[pix * 2 + 1], TH, TW,
                  interp);
  }
}

// ---------------------------------------------------------------------------
// mapped im2col / col2im for ONE batch element.
// col[(c*K + k)*M + pix], map[((pix*K)+k)*q*2], weights[((pix*K)+k)*q].
// common/mapped_im2col.h:11-41, :44-77, :80-116, :119-158; loops
// cpp/mapped_im2col.h:13-108.
// ---------------------------------------------------------------------------
template <typename T>
void mapped_im2col(const T* im, const T* map, const T* wts, T* col, int64_t C, int64_t H,
                   int64_t W, int64_t M, int64_t K, int P, int interp) {
  const int64_t q = pts(P);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < C * M; ++i) {
    const int64_t c = i / M, pix = i % M;
    for (int64_t k = 0; k < K; ++k)
      col[(c * K + k) * M + pix] =
          gather_sample(im + c * H * W, map + (pix * K + k) * q * 2,
                        wts ? wts + (pix * K + k) * q : nullptr, P, H, W, interp);
  }
}

template <typename T>
void mapped_col2im(const T* col, const T* map, const T* wts, T* im, int64_t C, int64_t H,
                   int64_t W, int64_t M, int64_t K, int P, int interp) {
  const int64_t q = pts(P);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < C * M; ++i) {
    const int64_t c = i / M, pix = i % M;
    for (int64_t k = 0; k < K; ++k)
      scatter_sample(col[(c * K + k) * M + pix], im + c * H * W,
                     map + (pix * K + k) * q * 2,
                     wts ? wts + (pix * K + k) * q : nullptr, P, H, W, interp);
  }
}

// ---------------------------------------------------------------------------
// Row-major GEMM helpers standing in for ATen mm (the reference's only
// third-party arithmetic on this path, src/cpp/mapped_convolution_layer.cpp:43-45,
// :72-74, :126-129).  Accumulation is in T, k ascending.
// ---------------------------------------------------------------------------
// C[m,n] (+)= sum_k A[m,k] * Bm[k,n]
template <typename T>
void gemm_nn(const T* A, const T* Bm, T* Cm, int64_t m, int64_t n, int64_t k, bool accumulate) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i) {
    T* crow = Cm + i * n;
    if (!accumulate)
      for (int64_t j = 0; j < n; ++j) crow[j] = T(0);
    for (int64_t l = 0; l < k; ++l) {
      const T a = A[i * k + l];
      const T* brow = Bm + l * n;
      for (int64_t j = 0; j < n; ++j) crow[j] += a * brow[j];
    }
  }
}
// C[m,n] = sum_k A[k,m] * Bm[k,n]   (A transposed)
template <typename T>
void gemm_tn(const T* A, const T* Bm, T* Cm, int64_t m, int64_t n, int64_t k) {
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < m; ++i) {
    T* crow = Cm + i * n;
    for (int64_t j = 0; j < n; ++j) crow[j] = T(0);
    for (int64_t l = 0; l < k; ++l) {
      const T a = A[l * m + i];
      const T* brow = Bm + l * n;
      for (int64_t j = 0; j < n; ++j) crow[j] += a * brow[j];
    }
  }
}
// C[m,n] += sum_k A[m,k] * Bm[n,k]  (B transposed; long reduction)
template <typename T>
void gemm_nt_acc(const T* A, const T* Bm, T* Cm, int64_t m, int64_t n, int64_t k) {
#pragma omp parallel for schedule(static) collapse(2)
  for (int64_t i = 0; i < m; ++i)
    for (int64_t j = 0; j < n; ++j) {
      const T* a = A + i * k;
      const T* b = Bm + j * k;
      T acc = T(0);
      for (int64_t l = 0; l < k; ++l) acc += a[l] * b[l];
      Cm[i * n + j] += acc;
    }
}

// ---------------------------------------------------------------------------
// Mapped convolution.  src/cpp/mapped_convolution_layer.cpp:8-51 (forward),
// :53-89 (backward input), :91-133 (backward weight); weighted twins in
// src/cpp/weighted_mapped_convolution_layer.cpp:8-141.
// weight is [Cout, Cin, K] viewed [Cout, Cin*K].
// ---------------------------------------------------------------------------
template <typename T>
void conv_forward(const T* x, const T* map, const T* wts, const T* weight, const T* bias,
                  T* out, int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout,
                  int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t M = OH * OW, CK = Cin * K;
  std::vector<T> col((size_t)CK * M);
  for (int64_t b = 0; b < B; ++b) {
    mapped_im2col(x + b * Cin * H * W, map, wts, col.data(), Cin, H, W, M, K, P, interp);
    T* ob = out + b * Cout * M;
    gemm_nn(weight, col.data(), ob, Cout, M, CK, false);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < Cout * M; ++i) ob[i] += bias[i / M];
  }
}

template <typename T>
void conv_backward_input(const T* gout, const T* map, const T* wts, const T* weight, T* gin,
                         int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout,
                         int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t M = OH * OW, CK = Cin * K;
  std::vector<T> col((size_t)CK * M);
  std::memset(gin, 0, sizeof(T) * B * Cin * H * W);
  for (int64_t b = 0; b < B; ++b) {
    gemm_tn(weight, gout + b * Cout * M, col.data(), CK, M, Cout);
    mapped_col2im(col.data(), map, wts, gin + b * Cin * H * W, Cin, H, W, M, K, P, interp);
  }
}

template <typename T>
void conv_backward_weight(const T* gout, const T* map, const T* wts, const T* x, T* gweight,
                          int64_t B, int64_t Cin, int64_t H, int64_t W, int64_t Cout,
                          int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t M = OH * OW, CK = Cin * K;
  std::vector<T> col((size_t)CK * M);
  std::memset(gweight, 0, sizeof(T) * Cout * CK);
  for (int64_t b = 0; b < B; ++b) {
    mapped_im2col(x + b * Cin * H * W, map, wts, col.data(), Cin, H, W, M, K, P, interp);
    gemm_nt_acc(gout + b * Cout * M, col.data(), gweight, Cout, CK, M);
  }
}

// grad_bias = grad_output.sum({0,2,3}); include/layers/mapped_convolution_layer.h:130
template <typename T>
void bias_grad(const T* gout, T* gbias, int64_t B, int64_t C, int64_t M) {
  for (int64_t c = 0; c < C; ++c) {
    T acc = T(0);
    for (int64_t b = 0; b < B; ++b)
      for (int64_t i = 0; i < M; ++i) acc += gout[(b * C + c) * M + i];
    gbias[c] = acc;
  }
}

// ---------------------------------------------------------------------------
// Mapped transposed convolution.  src/cpp/mapped_transposed_convolution_layer.cpp
// :8-49 (forward), :51-91 (backward input), :93-131 (backward weight).
// weight is [Cin, Cout, K] viewed [Cin, Cout*K]; the map has the INPUT's
// IH x IW and points into the OH x OW output.
// ---------------------------------------------------------------------------
template <typename T>
void tconv_forward(const T* x, const T* map, const T* wts, const T* weight, const T* bias,
                   T* out, int64_t B, int64_t Cin, int64_t IH, int64_t IW, int64_t Cout,
                   int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t Min = IH * IW, CoK = Cout * K, Mout = OH * OW;
  std::vector<T> col((size_t)CoK * Min);
  std::memset(out, 0, sizeof(T) * B * Cout * Mout);
  for (int64_t b = 0; b < B; ++b) {
    gemm_tn(weight, x + b * Cin * Min, col.data(), CoK, Min, Cin);
    T* ob = out + b * Cout * Mout;
    mapped_col2im(col.data(), map, wts, ob, Cout, OH, OW, Min, K, P, interp);
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < Cout * Mout; ++i) ob[i] += bias[i / Mout];
  }
}

template <typename T>
void tconv_backward_input(const T* gout, const T* map, const T* wts, const T* weight, T* gin,
                          int64_t B, int64_t Cin, int64_t IH, int64_t IW, int64_t Cout,
                          int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t Min = IH * IW, CoK = Cout * K, Mout = OH * OW;
  std::vector<T> col((size_t)CoK * Min);
  for (int64_t b = 0; b < B; ++b) {
    mapped_im2col(gout + b * Cout * Mout, map, wts, col.data(), Cout, OH, OW, Min, K, P, interp);
    gemm_nn(weight, col.data(), gin + b * Cin * Min, Cin, Min, CoK, false);
  }
}

template <typename T>
void tconv_backward_weight(const T* gout, const T* map, const T* wts, const T* x, T* gweight,
                           int64_t B, int64_t Cin, int64_t IH, int64_t IW, int64_t Cout,
                           int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t Min = IH * IW, CoK = Cout * K, Mout = OH * OW;
  std::vector<T> col((size_t)CoK * Min);
  std::memset(gweight, 0, sizeof(T) * Cin * CoK);
  for (int64_t b = 0; b < B; ++b) {
    mapped_im2col(gout + b * Cout * Mout, map, wts, col.data(), Cout, OH, OW, Min, K, P, interp);
    gemm_nt_acc(x + b * Cin * Min, col.data(), gweight, Cin, CoK, Min);
  }
}

// ---------------------------------------------------------------------------
// Mapped max pool.  common/mapped_max_pool.h:13-57 (:81-133 weighted): strict
// `>` so the first maximum wins and NaN never wins; the stored index is the
// flat element offset of the winning sample's x coordinate inside sample_map.
// init_mode 0: running max starts at -FLT_MAX (the reference's device branch,
//              :25-26, for float AND double);
// init_mode 1: starts at numeric_limits<T>::min(), the smallest positive
//              normal (the reference's host branch, :27-28): windows whose
//              samples are all <= that value yield (min(), -1).
// Unpool: common/mapped_max_pool.h:60-78 (:136-171 weighted); a negative stored
// index (no winner) contributes nothing here, where the reference host code
// would read out of bounds.
// ---------------------------------------------------------------------------
template <typename T>
void max_pool(const T* x, const T* map, const T* wts, T* out, int64_t* idx, int64_t B,
              int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW, int64_t K, int P,
              int interp, int init_mode) {
  const int64_t M = OH * OW, q = pts(P);
  const T init = init_mode == 1 ? std::numeric_limits<T>::min() : T(-FLT_MAX);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * M; ++i) {
    const int64_t pix = i % M, plane = i / M;
    T best = init;
    int64_t best_idx = -1;
    for (int64_t k = 0; k < K; ++k) {
      const int64_t s = (pix * K + k) * q;
      const T v = gather_sample(x + plane * H * W, map + s * 2, wts ? wts + s : nullptr, P,
                                H, W, interp);
      if (v > best) {
        best = v;
        best_idx = s * 2;
      }
    }
    out[i] = best;
    idx[i] = best_idx;
  }
}

template <typename T>
void max_unpool(const T* gout, const int64_t* idx, const T* map, const T* wts, T* gin,
                int64_t B, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                int64_t K, int P, int interp) {
  (void)K;
  const int64_t M = OH * OW;
  std::memset(gin, 0, sizeof(T) * B * C * H * W);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * M; ++i) {
    const int64_t plane = i / M;
    const int64_t s = idx[i];
    if (s < 0) continue;
    // s/2 is the flat (pix,k,p=0) sample number, which also indexes the weights.
    scatter_sample(gout[i], gin + plane * H * W, map + s, wts ? wts + s / 2 : nullptr, P, H, W,
                   interp);
  }
}

// The transpose of max_unpool: every pooled element reads the image at the sample its index
// names (0 for a negative index).  No reference counterpart: the reference's unpooling layer
// (layers/functional/mapped_pooling.py:156-199) cannot run; this is what its backward has to be.
template <typename T>
void gather_at_index(const T* image, const int64_t* idx, const T* map, const T* wts, T* out,
                     int64_t B, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW, int P,
                     int interp) {
  const int64_t M = OH * OW;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * M; ++i) {
    const int64_t plane = i / M, s = idx[i];
    out[i] = s < 0 ? T(0)
                   : gather_sample(image + plane * H * W, map + s, wts ? wts + s / 2 : nullptr, P,
                                   H, W, interp);
  }
}

// ---------------------------------------------------------------------------
// Mapped average pool and its adjoint.  common/mapped_avg_pool.h:13-40 (:70-105
// weighted): the K samples are summed in ascending order and the sum is divided
// by K; :42-68 (:107-140 weighted): every sample of a pooled pixel receives
// grad / K (divided first, then splatted).
// ---------------------------------------------------------------------------
template <typename T>
void avg_pool(const T* x, const T* map, const T* wts, T* out, int64_t B, int64_t C, int64_t H,
              int64_t W, int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t M = OH * OW, q = pts(P);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * M; ++i) {
    const int64_t pix = i % M, plane = i / M;
    T accum = T(0);
    for (int64_t k = 0; k < K; ++k) {
      const int64_t s = (pix * K + k) * q;
      accum += gather_sample(x + plane * H * W, map + s * 2, wts ? wts + s : nullptr, P, H, W,
                             interp);
    }
    out[i] = accum / T(K);
  }
}

template <typename T>
void avg_unpool(const T* gout, const T* map, const T* wts, T* gin, int64_t B, int64_t C,
                int64_t H, int64_t W, int64_t OH, int64_t OW, int64_t K, int P, int interp) {
  const int64_t M = OH * OW, q = pts(P);
  std::memset(gin, 0, sizeof(T) * B * C * H * W);
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < B * C * M; ++i) {
    const int64_t pix = i % M, plane = i / M;
    const T value = gout[i] / T(K);
    for (int64_t k = 0; k < K; ++k) {
      const int64_t s = (pix * K + k) * q;
      scatter_sample(value, gin + plane * H * W, map + s * 2, wts ? wts + s : nullptr, P, H, W,
                     interp);
    }
  }
}

}  // namespace

// ---------------------------------------------------------------------------
// C ABI.  dtype: 0 = float32, 1 = float64.  P = 0 selects the unweighted map
// layout [..., 2]; P >= 1 the weighted layout [..., P, 2] with weights [..., P].
// Every function returns 0 on success, 1 on an unsupported dtype.
// ---------------------------------------------------------------------------
// ---------------------------------------------------------------------------
// Sample-map generation.  The reference builds its maps with float32 (default dtype) tensor
// operations; every step below is the corresponding scalar operation in T, in the same order.
// layers/util/grids.py:5-25 (angular resolution, mesh grid; linspace is evaluated from the
// nearer end as the tensor library does), layers/util/conversions.py:24-52 (renormalize,
// spherical -> pixel), layers/util/mapping_functions.py:16-160 (kernel differentials and the
// three projections), layers/util/icosahedron_functions.py:47-103 (gnomonic kernel about
// given points).  Python scalars enter a tensor operation rounded to the tensor's type.
// ---------------------------------------------------------------------------
const double PI = 3.14159265358979323846;

template <typename T>
inline T linspace_at(T lo, T hi, int64_t steps, int64_t i) {
  const T step = (hi - lo) / T(steps - 1);
  return i < steps / 2 ? lo + step * T(i) : hi - step * T(steps - i - 1);
}

template <typename T>
inline T floor_mod(T a, T b) {
  T m = std::fmod(a, b);
  if (m != T(0) && ((b < T(0)) != (m < T(0)))) m += b;
  return m;
}

template <typename T>
inline T lon_to_x(T lon, int64_t W) { return T(W) * (lon - T(-PI)) / T(PI - (-PI)); }
template <typename T>
inline T lat_to_y(T lat, int64_t H) { return T(H - 1) * (lat - T(-PI / 2)) / T(PI / 2 - (-PI / 2)); }

template <typename T>
inline void inverse_gnomonic(T lon, T lat, T dx, T dy, T& out_lon, T& out_lat) {
  const T rho = std::sqrt(dx * dx + dy * dy);
  const T nu = std::atan(rho);
  out_lat = std::asin(std::cos(nu) * std::sin(lat) + dy * std::sin(nu) * std::cos(lat) / rho);
  out_lon = lon + std::atan2(dx * std::sin(nu),
                             rho * std::cos(lat) * std::cos(nu) - dy * std::sin(lat) * std::sin(nu));
}

template <typename T>
void equirect_kernel_map(T* out, int64_t H, int64_t W, int64_t kh, int64_t kw, int64_t stride,
                         int64_t dilation, int proj) {
  const int64_t OH = (H + stride - 1) / stride, OW = (W + stride - 1) / stride, K = kh * kw;
  const double res_lon = 2 * PI / double(W), res_lat = PI / double(H - 1);
#pragma omp parallel for schedule(static)
  for (int64_t idx = 0; idx < OH * OW * K; ++idx) {
    const int64_t k = idx % K, pix = idx / K;
    const int64_t x = (pix % OW) * stride, y = (pix / OW) * stride;
    const int64_t ci = k / kw - kh / 2, cj = k % kw - kw / 2;
    const T dlon = T(double(cj * dilation) * res_lon);
    const T dlat = T(double(ci * dilation) * -res_lat);
    const T lon = linspace_at<T>(T(-PI), T(PI), W + 1, x);
    const T lat = linspace_at<T>(T(-PI / 2), T(PI / 2), H, y);
    T mlon, mlat;
    if (proj == 0) {
      mlat = lat + dlat;
      mlon = lon + dlon;
    } else {
      if (proj == 1) {
        inverse_gnomonic(lon, lat, dlon, dlat, mlon, mlat);
        if (k == K / 2) { mlat = lat; mlon = lon; }
      } else {
        mlat = lat + dlat;
        mlon = lon + dlon / std::cos(mlat);
      }
      mlon = floor_mod(mlon + T(PI), T(2 * PI)) - T(PI);
    }
    out[idx * 2] = lon_to_x(mlon, W);
    out[idx * 2 + 1] = lat_to_y(mlat, H);
  }
}

template <typename T>
void gnomonic_kernel_at(const T* lonlat, T* out, int64_t n, int64_t kh, int64_t kw,
                        double res_lat, double res_lon, int64_t img_h, int64_t img_w) {
  const int64_t K = kh * kw;
#pragma omp parallel for schedule(static)
  for (int64_t idx = 0; idx < n * K; ++idx) {
    const int64_t k = idx % K, p = idx / K, i = k / kw, j = k % kw;
    T dx = T(double(j - kw / 2) * res_lon);
    T dy = T(double(i - kh / 2) * res_lat);
    if (kh % 2 == 0) dy += T(res_lat / 2);
    if (kw % 2 == 0) dx += T(res_lon / 2);
    const T lon = lonlat[p * 2], lat = lonlat[p * 2 + 1];
    T olon, olat;
    inverse_gnomonic(lon, lat, dx, dy, olon, olat);
    const bool centre = k == (kh / 2) * kw + kw / 2;
    if (kh % 2 == 1 && centre) olat = lat;
    if (kw % 2 == 1 && centre) olon = lon;
    olon = floor_mod(olon + T(PI), T(2 * PI)) - T(PI);
    out[idx * 2] = img_h > 0 ? lon_to_x(olon, img_w) : olon;
    out[idx * 2 + 1] = img_h > 0 ? lat_to_y(olat, img_h) : olat;
  }
}

// ---------------------------------------------------------------------------
// Voting resample.  core/interpolation.h:249-265 (one vote per in-range target),
// common/resample.h:109-130 (label and target of an input pixel),
// src/cpp/voting_resample_layer.cpp:8-37 (histogram [C, OH, OW, candidates] per batch element,
// argmax over the last axis: the first of equal counts).  A label outside the range casts no
// vote (the reference would write outside its histogram).  The reference offsets channel c's
// votes by c * OH * OW histogram elements rather than by c whole planes of OH * OW * NC, so
// with more than one channel the histograms overlap; that indexing is kept as it is (label
// images have one channel, for which it is the plain vote).
// ---------------------------------------------------------------------------
void voting_resample(const int64_t* in, const int64_t* map, int64_t* out, int64_t B, int64_t C,
                     int64_t IH, int64_t IW, int64_t OH, int64_t OW, int64_t NC) {
  std::vector<int64_t> votes((size_t)C * OH * OW * NC);
  for (int64_t b = 0; b < B; ++b) {
    std::fill(votes.begin(), votes.end(), 0);
    for (int64_t i = 0; i < C * IH * IW; ++i) {
      const int64_t pix = i % (IH * IW), c = i / (IH * IW);
      const int64_t x = map[pix * 2], y = map[pix * 2 + 1], label = in[b * C * IH * IW + i];
      if (x < 0 || x > OW - 1 || y < 0 || y > OH - 1 || label < 0 || label >= NC) continue;
      // the channel's histogram starts c * OH * OW elements in, not c * OH * OW * NC
      // (common/resample.h:127-129): for C > 1 the channels' histograms overlap
      ++votes[c * OH * OW + (y * OW + x) * NC + label];
    }
    for (int64_t o = 0; o < C * OH * OW; ++o) {
      int64_t arg = 0;
      for (int64_t k = 1; k < NC; ++k)
        if (votes[o * NC + k] > votes[o * NC + arg]) arg = k;
      out[b * C * OH * OW + o] = arg;
    }
  }
}

#define DISPATCH(dtype, CALL)                                       \
  do {                                                              \
    if ((dtype) == 0) { using T = float; CALL; return 0; }          \
    if ((dtype) == 1) { using T = double; CALL; return 0; }         \
    return 1;                                                       \
  } while (0)

extern "C" {

int sdk_oracle_resample_from_map(const void* image, const void* map, const void* wts, void* out,
                                 int64_t B, int64_t C, int64_t H, int64_t W, int64_t MH,
                                 int64_t MW, int P, int interp, int dtype) {
  DISPATCH(dtype, resample_from_map<T>((const T*)image, (const T*)map, (const T*)wts, (T*)out,
                                        B, C, H, W, MH, MW, P, interp));
}

int sdk_oracle_resample_to_map(const void* in, const void* map, const void* wts, void* out,
                               int64_t B, int64_t C, int64_t MH, int64_t MW, int64_t H,
                               int64_t W, int P, int interp, int dtype) {
  DISPATCH(dtype, resample_to_map<T>((const T*)in, (const T*)map, (const T*)wts, (T*)out, B, C,
                                      MH, MW, H, W, P, interp));
}

int sdk_oracle_mapped_im2col(const void* im, const void* map, const void* wts, void* col,
                             int64_t C, int64_t H, int64_t W, int64_t M, int64_t K, int P,
                             int interp, int dtype) {
  DISPATCH(dtype, mapped_im2col<T>((const T*)im, (const T*)map, (const T*)wts, (T*)col, C, H, W,
                                    M, K, P, interp));
}

// `im` must be zero-filled (or hold the values to accumulate onto) by the caller.
int sdk_oracle_mapped_col2im(const void* col, const void* map, const void* wts, void* im,
                             int64_t C, int64_t H, int64_t W, int64_t M, int64_t K, int P,
                             int interp, int dtype) {
  DISPATCH(dtype, mapped_col2im<T>((const T*)col, (const T*)map, (const T*)wts, (T*)im, C, H, W,
                                    M, K, P, interp));
}

int sdk_oracle_mapped_max_pool(const void* x, const void* map, const void* wts, void* out,
                               int64_t* idx, int64_t B, int64_t C, int64_t H, int64_t W,
                               int64_t OH, int64_t OW, int64_t K, int P, int interp, int dtype,
                               int init_mode) {
  DISPATCH(dtype, max_pool<T>((const T*)x, (const T*)map, (const T*)wts, (T*)out, idx, B, C, H,
                               W, OH, OW, K, P, interp, init_mode));
}

int sdk_oracle_mapped_max_unpool(const void* gout, const int64_t* idx, const void* map,
                                 const void* wts, void* gin, int64_t B, int64_t C, int64_t H,
                                 int64_t W, int64_t OH, int64_t OW, int64_t K, int P,
                                 int interp, int dtype) {
  DISPATCH(dtype, max_unpool<T>((const T*)gout, idx, (const T*)map, (const T*)wts, (T*)gin, B,
                                 C, H, W, OH, OW, K, P, interp));
}

int sdk_oracle_mapped_gather_at_index(const void* image, const int64_t* idx, const void* map,
                                      const void* wts, void* out, int64_t B, int64_t C, int64_t H,
                                      int64_t W, int64_t OH, int64_t OW, int P, int interp,
                                      int dtype) {
  DISPATCH(dtype, gather_at_index<T>((const T*)image, idx, (const T*)map, (const T*)wts, (T*)out,
                                      B, C, H, W, OH, OW, P, interp));
}

int sdk_oracle_mapped_avg_pool(const void* x, const void* map, const void* wts, void* out,
                               int64_t B, int64_t C, int64_t H, int64_t W, int64_t OH, int64_t OW,
                               int64_t K, int P, int interp, int dtype) {
  DISPATCH(dtype, avg_pool<T>((const T*)x, (const T*)map, (const T*)wts, (T*)out, B, C, H, W, OH,
                               OW, K, P, interp));
}

int sdk_oracle_mapped_avg_unpool(const void* gout, const void* map, const void* wts, void* gin,
                                 int64_t B, int64_t C, int64_t H, int64_t W, int64_t OH,
                                 int64_t OW, int64_t K, int P, int interp, int dtype) {
  DISPATCH(dtype, avg_unpool<T>((const T*)gout, (const T*)map, (const T*)wts, (T*)gin, B, C, H, W,
                                 OH, OW, K, P, interp));
}

int sdk_oracle_resample_from_uv_maps(const void* tex, const int64_t* quad, const void* uv,
                                     void* out, int64_t B, int64_t C, int64_t NT, int64_t TH,
                                     int64_t TW, int64_t H, int64_t W, int interp, int dtype) {
  DISPATCH(dtype, resample_from_uv<T>((const T*)tex, quad, (const T*)uv, (T*)out, B, C, NT, TH,
                                       TW, H, W, interp));
}

int sdk_oracle_resample_to_uv_maps(const void* in, const int64_t* quad, const void* uv, void* tex,
                                   int64_t B, int64_t C, int64_t NT, int64_t TH, int64_t TW,
                                   int64_t H, int64_t W, int interp, int dtype) {
  DISPATCH(dtype, resample_to_uv<T>((const T*)in, quad, (const T*)uv, (T*)tex, B, C, NT, TH, TW,
                                     H, W, interp));
}

int sdk_oracle_equirect_kernel_map(void* out, int64_t H, int64_t W, int64_t kh, int64_t kw,
                                   int64_t stride, int64_t dilation, int proj, int dtype) {
  DISPATCH(dtype, equirect_kernel_map<T>((T*)out, H, W, kh, kw, stride, dilation, proj));
}

int sdk_oracle_gnomonic_kernel_at(const void* lonlat, void* out, int64_t n, int64_t kh, int64_t kw,
                                  double res_lat, double res_lon, int64_t img_h, int64_t img_w,
                                  int dtype) {
  DISPATCH(dtype, gnomonic_kernel_at<T>((const T*)lonlat, (T*)out, n, kh, kw, res_lat, res_lon,
                                         img_h, img_w));
}

int sdk_oracle_voting_resample(const int64_t* in, const int64_t* map, int64_t* out, int64_t B,
                               int64_t C, int64_t IH, int64_t IW, int64_t OH, int64_t OW,
                               int64_t NC) {
  voting_resample(in, map, out, B, C, IH, IW, OH, OW, NC);
  return 0;
}

int sdk_oracle_mapped_conv_forward(const void* x, const void* map, const void* wts,
                                   const void* weight, const void* bias, void* out, int64_t B,
                                   int64_t Cin, int64_t H, int64_t W, int64_t Cout, int64_t OH,
                                   int64_t OW, int64_t K, int P, int interp, int dtype) {
  DISPATCH(dtype, conv_forward<T>((const T*)x, (const T*)map, (const T*)wts, (const T*)weight,
                                   (const T*)bias, (T*)out, B, Cin, H, W, Cout, OH, OW, K, P,
                                   interp));
}

int sdk_oracle_mapped_conv_backward_input(const void* gout, const void* map, const void* wts,
                                          const void* weight, void* gin, int64_t B, int64_t Cin,
                                          int64_t H, int64_t W, int64_t Cout, int64_t OH,
                                          int64_t OW, int64_t K, int P, int interp, int dtype) {
  DISPATCH(dtype, conv_backward_input<T>((const T*)gout, (const T*)map, (const T*)wts,
                                          (const T*)weight, (T*)gin, B, Cin, H, W, Cout, OH, OW,
                                          K, P, interp));
}

int sdk_oracle_mapped_conv_backward_weight(const void* gout, const void* map, const void* wts,
                                           const void* x, void* gweight, int64_t B, int64_t Cin,
                                           int64_t H, int64_t W, int64_t Cout, int64_t OH,
                                           int64_t OW, int64_t K, int P, int interp, int dtype) {
  DISPATCH(dtype, conv_backward_weight<T>((const T*)gout, (const T*)map, (const T*)wts,
                                           (const T*)x, (T*)gweight, B, Cin, H, W, Cout, OH, OW,
                                           K, P, interp));
}

int sdk_oracle_bias_grad(const void* gout, void* gbias, int64_t B, int64_t C, int64_t M,
                         int dtype) {
  DISPATCH(dtype, bias_grad<T>((const T*)gout, (T*)gbias, B, C, M));
}

int sdk_oracle_mapped_transposed_conv_forward(const void* x, const void* map, const void* wts,
                                              const void* weight, const void* bias, void* out,
                                              int64_t B, int64_t Cin, int64_t IH, int64_t IW,
                                              int64_t Cout, int64_t OH, int64_t OW, int64_t K,
                                              int P, int interp, int dtype) {
  DISPATCH(dtype, tconv_forward<T>((const T*)x, (const T*)map, (const T*)wts, (const T*)weight,
                                    (const T*)bias, (T*)out, B, Cin, IH, IW, Cout, OH, OW, K, P,
                                    interp));
}

int sdk_oracle_mapped_transposed_conv_backward_input(const void* gout, const void* map,
                                                     const void* wts, const void* weight,
                                                     void* gin, int64_t B, int64_t Cin,
                                                     int64_t IH, int64_t IW, int64_t Cout,
                                                     int64_t OH, int64_t OW, int64_t K, int P,
                                                     int interp, int dtype) {
  DISPATCH(dtype, tconv_backward_input<T>((const T*)gout, (const T*)map, (const T*)wts,
                                           (const T*)weight, (T*)gin, B, Cin, IH, IW, Cout, OH,
                                           OW, K, P, interp));
}

int sdk_oracle_mapped_transposed_conv_backward_weight(const void* gout, const void* map,
                                                      const void* wts, const void* x,
                                                      void* gweight, int64_t B, int64_t Cin,
                                                      int64_t IH, int64_t IW, int64_t Cout,
                                                      int64_t OH, int64_t OW, int64_t K, int P,
                                                      int interp, int dtype) {
  DISPATCH(dtype, tconv_backward_weight<T>((const T*)gout, (const T*)map, (const T*)wts,
                                            (const T*)x, (T*)gweight, B, Cin, IH, IW, Cout, OH,
                                            OW, K, P, interp));
}

int sdk_oracle_num_threads(void) { return omp_get_max_threads(); }

}  // extern "C"
