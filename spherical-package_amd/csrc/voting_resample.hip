// Voting resample: integer labels scattered through an integer sample map; every output pixel
// keeps the label most of its sources carry.  Reference: votes with 64-bit atomic adds into a
// [C, OH, OW, candidates] int64 histogram per batch element, then argmax over the last axis
// (ext_modules/include/core/interpolation.h:249-265, core/resample.h:163-172,
// common/resample.h:109-130, src/cpp/voting_resample_layer.cpp:8-37).  Here the histogram is a
// caller-provided workspace of 32-bit counters (a pixel cannot collect 2^31 votes), reused
// pass after pass for as many batch elements as it holds; the first label with the most votes wins, label 0 where nobody voted.
// With more than one channel the reference's histograms overlap (its channel offset lacks the
// factor `candidates`); label images have one channel, and the overlap is reproduced as it is.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "sdk_host.hpp"
#include "sdk_lane_runs.hpp"

namespace sdk {

constexpr int kVoteBlock = 256;

__global__ __launch_bounds__(kVoteBlock) void vote_clear_kernel(uint4* __restrict__ p, size_t n16) {
  const size_t stride = (size_t)gridDim.x * kVoteBlock;
  for (size_t i = (size_t)blockIdx.x * kVoteBlock + threadIdx.x; i < n16; i += stride)
    p[i] = make_uint4(0, 0, 0, 0);
}

// One thread per input pixel, grid.y over (batch element of this pass, channel): the plane
// arithmetic is per workgroup, and the pixel's target (16 bytes of the map) and its label are
// requested together.  A label outside [0, candidates) casts no vote (the reference would
// write outside its histogram).  Neighbouring lanes often vote for the same cell (pixels of a
// label image that share a target): a run of them casts its votes with one atomic, from its
// last lane.
__global__ __launch_bounds__(kVoteBlock) void vote_kernel(
    const int64_t* __restrict__ labels, const int64_t* __restrict__ map,
    unsigned* __restrict__ votes, int in_pixels, int channels, int OH, int OW, int candidates,
    size_t element_stride) {
  const int pix = blockIdx.x * kVoteBlock + threadIdx.x;
  const unsigned plane = blockIdx.y;
  const unsigned e = plane / (unsigned)channels, c = plane - e * (unsigned)channels;
  const int at = min(pix, in_pixels - 1);
  const long long x = map[(size_t)at * 2], y = map[(size_t)at * 2 + 1];
  const long long label = labels[(size_t)plane * in_pixels + at];
  const bool ok = pix < in_pixels && x >= 0 && x <= OW - 1 && y >= 0 && y <= OH - 1 &&
                  label >= 0 && label < candidates;
  // channel offset in histogram elements as the reference has it (common/resample.h:127-129):
  // c * OH * OW, not c whole histograms, so the histograms of several channels overlap
  const long long cell = ok ? (long long)(e * element_stride + (size_t)c * OH * OW +
                                          ((size_t)y * OW + (size_t)x) * candidates +
                                          (size_t)label)
                            : -1;
  const long long below = __shfl_up(cell, 1);
  const LaneRuns runs(below == cell);
  if (ok && runs.tail) atomicAdd(&votes[cell], (unsigned)(runs.dist + 1));
}

// One thread per output pixel, grid.y over (batch element of this pass, channel): index of
// the first largest count.  The counts are read eight at a time, all eight requested before
// the first is compared.
__global__ __launch_bounds__(kVoteBlock) void vote_argmax_kernel(
    const unsigned* __restrict__ votes, int64_t* __restrict__ out, int out_pixels, int channels,
    int candidates, size_t element_stride) {
  const int pix = blockIdx.x * kVoteBlock + threadIdx.x;
  if (pix >= out_pixels) return;
  const unsigned plane = blockIdx.y;
  const unsigned e = plane / (unsigned)channels, c = plane - e * (unsigned)channels;
  const unsigned* v =
      votes + e * element_stride + ((size_t)c * out_pixels + pix) * (size_t)candidates;
  unsigned best = 0;
  int arg = 0;
  for (int k0 = 0; k0 < candidates; k0 += 8) {
    unsigned n[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) n[i] = v[min(k0 + i, candidates - 1)];
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (k0 + i < candidates && n[i] > best) {   // strict: the first of equal counts stays
        best = n[i];
        arg = k0 + i;
      }
  }
  out[(size_t)plane * out_pixels + pix] = arg;
}

static size_t vote_bytes(int64_t channels, int64_t oh, int64_t ow, int64_t candidates) {
  const size_t n = (size_t)channels * oh * ow * candidates * sizeof(unsigned);
  return (n + 255) & ~(size_t)255;
}

}  // namespace sdk

using namespace sdk;

extern "C" {

size_t sdk_voting_resample_workspace_bytes(int64_t channels, int64_t out_height,
                                           int64_t out_width, int64_t num_candidates) {
  if (channels < 1 || out_height < 1 || out_width < 1 || num_candidates < 1) return 0;
  return vote_bytes(channels, out_height, out_width, num_candidates);
}

int sdk_voting_resample_to_map(const int64_t* input, const int64_t* sample_map, int64_t* out,
                               void* workspace, size_t workspace_bytes, int64_t batch,
                               int64_t channels, int64_t in_height, int64_t in_width,
                               int64_t out_height, int64_t out_width, int64_t num_candidates,
                               sdk_stream_t stream) {
  SDK_REQUIRE(batch >= 0 && channels >= 0, "voting_resample_to_map: negative size");
  SDK_REQUIRE(in_height >= 1 && in_width >= 1 && in_height * in_width < ((int64_t)1 << 31) &&
                  out_height >= 1 && out_width >= 1 &&
                  out_height * out_width < ((int64_t)1 << 31),
              "voting_resample_to_map: planes must have 1 .. 2^31-1 elements");
  SDK_REQUIRE(num_candidates >= 1 && num_candidates < ((int64_t)1 << 31),
              "voting_resample_to_map: num_candidates = %lld", (long long)num_candidates);
  if (batch * channels == 0) return SDK_OK;
  SDK_REQUIRE(input && sample_map && out, "voting_resample_to_map: NULL pointer");
  const size_t need = vote_bytes(channels, out_height, out_width, num_candidates);
  if (workspace == nullptr || workspace_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "voting_resample_to_map: workspace of %zu bytes needed, got %zu",
                need, workspace_bytes);
  SDK_REQUIRE((uintptr_t)workspace % 16 == 0, "voting_resample_to_map: workspace not 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  unsigned* votes = static_cast<unsigned*>(workspace);
  const int in_pixels = (int)(in_height * in_width);
  const int out_pixels = (int)(out_height * out_width);
  const size_t n_in = (size_t)channels * in_pixels;
  const size_t n_out = (size_t)channels * out_height * out_width;
  SDK_REQUIRE(channels <= 65535, "voting_resample_to_map: more than 65535 channels");
  // as many batch elements per pass as the workspace holds histograms (and grid.y planes)
  const int64_t per_pass = std::min<int64_t>(
      std::min<int64_t>(batch, (int64_t)(workspace_bytes / need)), 65535 / channels);
  for (int64_t b = 0; b < batch; b += per_pass) {
    const int64_t nb = std::min<int64_t>(per_pass, batch - b);
    const size_t n16 = need / 16 * (size_t)nb;
    const int clear_blocks = (int)std::min<int64_t>(ceil_div((int64_t)n16, kVoteBlock), 4096);
    launch(vote_clear_kernel, dim3(clear_blocks), dim3(kVoteBlock), s, (uint4*)workspace, n16);
    const unsigned planes = (unsigned)(nb * channels);
    launch(vote_kernel, dim3((unsigned)ceil_div(in_pixels, kVoteBlock), planes), dim3(kVoteBlock),
           s, input + (size_t)b * n_in, sample_map, votes, in_pixels, (int)channels,
           (int)out_height, (int)out_width, (int)num_candidates, need / sizeof(unsigned));
    launch(vote_argmax_kernel, dim3((unsigned)ceil_div(out_pixels, kVoteBlock), planes),
           dim3(kVoteBlock), s, (const unsigned*)votes, out + (size_t)b * n_out, out_pixels,
           (int)channels, (int)num_candidates, need / sizeof(unsigned));
  }
  SDK_LAUNCH_CHECK("voting_resample_to_map");
  return SDK_OK;
}

}  // extern "C"
