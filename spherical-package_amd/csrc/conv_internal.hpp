// Internal interfaces between the convolution drivers and the kernels they
// chain.  Not part of the C ABI.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "sdk_mapped_ops.h"
#include "sdk_mfma.hpp"

namespace sdk {

// sdk_compute -> matrix arithmetic of the fused kernels that know all three kinds.
inline int matrix_mode(int compute) {
  return compute == SDK_COMPUTE_BF16 ? kMmBf16 : (compute == SDK_COMPUTE_SPLIT ? kMmSplit : kMmF32);
}

int zero_fill(void* ptr, size_t bytes, hipStream_t stream);
// Three buffers (sizes multiples of 4 bytes) cleared by one launch.
int zero_fill3(void* a, size_t a_bytes, void* b, size_t b_bytes, void* c, size_t c_bytes,
               hipStream_t stream);
// grad_bias[c] = sum over batch and pixels (sdk_bias_grad).  beside_contractions: the variant
// that uses no LDS, for a launch that runs concurrently with the contraction kernels.
int bias_grad(const void* grad_output, void* grad_bias, int64_t batch, int64_t channels,
              int64_t pixels, int32_t dtype, hipStream_t stream, bool beside_contractions);
// gate: optional device flag; with one, the fill runs only if *gate != 0.
int zero_fill_gated(void* ptr, size_t bytes, hipStream_t stream, const int* gate);

// Batched mapped im2col / col2im over `planes` image planes (see
// mapped_gather_scatter.hip).  col2im accumulates onto what `im` holds.
template <typename T>
int launch_mapped_im2col(const T* im, const T* map, const T* wts, T* col, int64_t planes, int H,
                         int W, int M, int K, int P, int interp, hipStream_t stream);
template <typename T>
int launch_mapped_col2im(const T* col, const T* map, const T* wts, T* im, int64_t planes, int H,
                         int W, int M, int K, int P, int interp, hipStream_t stream);

// dst[(b*C + c)*n + i] = bias ? bias[c] : 0 for `planes` = B*C planes of n elements; with a gate
// (device flag) only if *gate != 0.
template <typename T>
int plane_fill(T* dst, const T* bias, int64_t planes, int C, size_t n, hipStream_t stream,
               const int* gate = nullptr);

// Geometry of one convolution-shaped call, shared by the generic and the fused
// drivers.  "gather side" is the image the sample map points into, "pixel side"
// the grid the map is defined on:
//   mapped conv:            gather side = input  [Cg = Cin,  H x W],  pixel side = output (Cp = Cout, M = OH*OW)
//   mapped transposed conv: gather side = output [Cg = Cout, OH x OW], pixel side = input (Cp = Cin,  M = IH*IW)
// The weight matrix is always [Cp, Cg*K] row-major.
struct ConvGeom {
  int64_t B;
  int Cg, H, W;  // gather-side channels and plane size
  int Cp, M;     // pixel-side channels and pixel count
  int K, P, interp;
  int OW;        // width of the pixel grid (M = OH * OW)
};

// The three contractions, for the tensors' own floating type, as separate
// im2col/col2im + GEMM launches with `workspace` holding one batch element's
// columns [Cg*K, M].
//   gather_gemm:  pix[b] = Wm x im2col(img[b]) (+ bias per row)       (conv forward, transposed backward-input)
//   gemm_scatter: img[b] (+)= col2im(Wm^T x pix[b]), img pre-filled    (conv backward-input, transposed forward)
//   gather_wgrad: gW = sum_b pix[b] x im2col(img[b])^T                 (both backward-weight)
template <typename T>
int generic_gather_gemm(const ConvGeom& g, const T* img, const T* map, const T* wts, const T* Wm,
                        const T* bias, T* pix, T* workspace, hipStream_t stream);
template <typename T>
int generic_gemm_scatter(const ConvGeom& g, const T* pix, const T* map, const T* wts, const T* Wm,
                         const T* bias, T* img, T* workspace, hipStream_t stream);
template <typename T>
int generic_gather_wgrad(const ConvGeom& g, const T* pix, const T* map, const T* wts, const T* img,
                         T* gW, T* workspace, hipStream_t stream);

}  // namespace sdk
