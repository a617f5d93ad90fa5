// Runs of neighbouring lanes that hold the same key, found with one ballot.
#pragma once
#include <hip/hip_runtime.h>

namespace sdk {

// Runs of equal keys over the lanes of a wave: distance of each lane to the first lane of its
// run and whether it is the last one.  `same` = this lane continues the run of the lane below.
struct LaneRuns {
  int dist;
  bool tail;
  __device__ __forceinline__ LaneRuns(bool same) {
    const int lane = threadIdx.x & 63;
    const unsigned long long heads = __ballot(lane == 0 || !same);
    const unsigned long long upto = heads & (~0ull >> (63 - lane));
    dist = lane - (63 - __clzll((long long)upto));
    tail = lane == 63 || (((heads >> 1) >> lane) & 1ull);
  }
  // inclusive sum of v over the lanes of the run up to this one
  template <typename T>
  __device__ __forceinline__ T sum(T v) const {
    for (int d = 1; d < 64; d <<= 1) {
      if (!__any(dist >= d)) break;
      const T below = __shfl_up(v, d);
      if (dist >= d) v += below;
    }
    return v;
  }
};

}  // namespace sdk
