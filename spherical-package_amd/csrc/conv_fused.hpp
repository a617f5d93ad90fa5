// Fused gather -> MFMA and MFMA -> scatter convolution kernels (float32 tensors).
#pragma once
#include <hip/hip_runtime.h>

#include "conv_internal.hpp"

namespace sdk {

// True when the fused kernels cover this geometry.
bool fused_supported(const ConvGeom& g);

int fused_gather_gemm(const ConvGeom& g, int compute, const float* img, const float* map,
                      const float* wts, const float* Wm, const float* bias, float* pix,
                      hipStream_t stream);
int fused_gemm_scatter(const ConvGeom& g, int compute, const float* pix, const float* map,
                       const float* wts, const float* Wm, const float* bias, float* img,
                       hipStream_t stream);
int fused_gather_wgrad(const ConvGeom& g, int compute, const float* pix, const float* map,
                       const float* wts, const float* img, float* gW, hipStream_t stream);

}  // namespace sdk
