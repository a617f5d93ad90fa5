// Row-band pooling kernels (pool_band.hip): launcher shared with the pooling entry points.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace sdk {

// Max (avg = false: values and int64 indices) or average pooling of float32 planes through a
// map of single nearest taps.  Returns false, having launched nothing, when the shape is not
// one the band kernels take (the caller then runs the per-pixel kernel).
bool pool_band_launch(bool avg, const float* in, const float* map, float* out, int64_t* idx,
                      int64_t planes, int H, int W, int OH, int OW, int K, hipStream_t stream);

}  // namespace sdk
