// Mapped max / average pooling of float32 planes from an LDS window, driven by a tap plan
// (pool_window.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "conv_plan.hpp"

namespace sdk {

// out[plane][m] (and, for max pooling, idx[plane][m]) for the pixels of the plan's tiles
// listed in tl.inside (tiles whose taps all lie inside their window); unweighted maps only.
// idx == nullptr: average pooling.  The values are formed as the per-pixel kernels form them
// (mapped_gather_scatter.hip): products and sums in tap order, first maximum wins.
int window_pool(const float* in, const Plan& plan, const TileLists& tl, float* out, int64_t* idx,
                int64_t planes, int H, int W, int K, hipStream_t stream);

}  // namespace sdk
