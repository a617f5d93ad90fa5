// Mapped convolution over images of at most four channels (conv_small.hip), float32.
#pragma once
#include <hip/hip_runtime.h>

#include "conv_internal.hpp"

namespace sdk {

// Geometries the packed kernels cover: Cg <= 4, K <= 25, Cp <= 128.
bool small_conv_supported(const ConvGeom& g);
// ... and whose weight gradient fits the accumulators of one wave.
bool small_wgrad_supported(const ConvGeom& g);

// pix[b] = Wm x im2col(img[b]) (+ bias per row); Wm[n][c][k] as the caller passes it.
int small_forward(const ConvGeom& g, const float* img, const float* map, const float* wts,
                  const float* Wm, const float* bias, float* pix, hipStream_t stream);
// img[b] += col2im(Wm^T x pix[b]) with float atomics; img must hold the values to add to.
int small_scatter(const ConvGeom& g, const float* pix, const float* map, const float* wts,
                  const float* Wm, float* img, hipStream_t stream);
// gW += sum_b pix[b] x im2col(img[b])^T; gW must hold the values to add to (zeros).
// gbias (optional, [Cp], zeros): receives the sum of pix over batch and pixels as well.
int small_wgrad(const ConvGeom& g, const float* pix, const float* map, const float* wts,
                const float* img, float* gW, hipStream_t stream, float* gbias = nullptr);

}  // namespace sdk
