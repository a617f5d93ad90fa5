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

// Unpooling by image row bands (float32, single nearest taps, K = 4 or 9, image width a
// multiple of 4 and at most 4096).  unpool_band_shape says whether
// the kernels take the shape at all.  The table (unpool_band_table_bytes, zero-filled by the
// caller, then unpool_band_build) depends on the map alone; its first word is the device-side
// verdict: 1 when the band kernels will do the call, 0 when they return at once and the
// caller's other route has to run (it stays 0 when unpool_band_build is never called).
bool unpool_band_shape(int H, int W, int OH, int OW, int K);
size_t unpool_band_table_bytes(int H, int W);
// Bytes of the packed taps a plan may hold behind the table (every band's pooled pixels with
// their taps resolved, so that the band kernels read them instead of decoding the map in every
// workgroup); 0 for shapes where they would take more than 32 MiB.
size_t unpool_band_taps_bytes(int H, int W);
// seen: nullptr, or scratch of one zeroed 32-bit word per image pixel (not needed afterwards):
// the build then also finds out whether average unpooling may add sample by sample without
// atomics (no two pooled pixels with the same sample at one image pixel).
// taps: nullptr, or unpool_band_taps_bytes of room for the packed taps (perm: in the layout of
// average unpooling, which keeps even and odd columns apart in LDS).
void unpool_band_build(const float* map, int* table, int H, int W, int OH, int OW, int K,
                       hipStream_t stream, unsigned* seen = nullptr, unsigned* taps = nullptr,
                       bool perm = false);
// avg: every sample of a pooled pixel receives grad_output / K (idx unused); else the sample the
// index names receives grad_output.  gate: raised when an index names a sample of another
// pooled pixel than its own (the caller then redoes the call with its atomic route).
// taps: what unpool_band_build wrote for this map with perm = avg, or nullptr.
void unpool_band_launch(bool avg, const float* gout, const int64_t* idx, const float* map,
                        float* gin, const int* table, const unsigned* taps, int* gate,
                        int64_t planes, int H, int W, int OH, int OW, int K, hipStream_t stream);

}  // namespace sdk
