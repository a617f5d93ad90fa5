// Fused gather -> MFMA and MFMA -> scatter convolution kernels (float32 tensors).
#pragma once
#include <hip/hip_runtime.h>

#include "conv_internal.hpp"
#include "conv_plan.hpp"

namespace sdk {

// A tap plan handed from one contraction of a call to the next (backward-input builds it,
// backward-weight of the same call reuses it).
struct SharedPlan {
  bool valid = false;
  Plan plan;
  // The caller has cleared the scatter's image and the weight gradient already (the combined
  // backward of a layer with at most four image channels, whose seven launches are its time).
  bool cleared = false;
  // ... and wants the bias gradient (the sum of the weight gradient's pixel-side operand over
  // batch and pixels) from the weight-gradient kernel, into this cleared buffer.
  float* bias_sum = nullptr;
};

// Everything the fused kernels derive from the sample map alone, built once into a
// caller-owned buffer and reused by every call on that map (any batch size, channel counts,
// weights): the tap plan with its tile lists and the inverse plan with its tile lists.
struct CachedPlan {
  Plan plan;
  TileLists lists, lists4;      // all tiles by window fit; ... and at most four rows per sample
  bool has_inverse = false;
  InversePlan inverse;
  TileLists inverse_lists;
  const void* col2im_lists = nullptr;   // the inverted map of the product route, where kept
};
// g: only H, W, M, OW, K, P and interp matter.  0 bytes: no plan for this geometry.
size_t cached_plan_bytes(const ConvGeom& g);
int build_cached_plan(const ConvGeom& g, const float* map, const float* wts, void* buffer,
                      hipStream_t stream);
// Pointers into a buffer build_cached_plan filled for the same geometry.
void load_cached_plan(const ConvGeom& g, void* buffer, CachedPlan* out);

// True when the fused kernels cover this geometry.
bool fused_supported(const ConvGeom& g);

// Bytes of device scratch the fused kernels need for this geometry (re-laid-out weights).
size_t fused_workspace_bytes(const ConvGeom& g);

// cached (optional, all three): a plan built by build_cached_plan for this map and geometry.
int fused_gather_gemm(const ConvGeom& g, int compute, const float* img, const float* map,
                      const float* wts, const float* Wm, const float* bias, float* pix,
                      float* workspace, hipStream_t stream, const CachedPlan* cached = nullptr);
// shared (optional): gemm_scatter stores the plan it built there; gather_wgrad uses a valid one
// instead of building its own (same map, weights and geometry, same workspace still alive).
int fused_gemm_scatter(const ConvGeom& g, int compute, const float* pix, const float* map,
                       const float* wts, const float* Wm, const float* bias, float* img,
                       float* workspace, hipStream_t stream, SharedPlan* shared = nullptr,
                       const CachedPlan* cached = nullptr);
int fused_gather_wgrad(const ConvGeom& g, int compute, const float* pix, const float* map,
                       const float* wts, const float* img, float* gW, float* workspace,
                       hipStream_t stream, const SharedPlan* shared = nullptr,
                       const CachedPlan* cached = nullptr);

// Bytes of the permuted weight copy the plan-driven scatter kernel reads.
size_t staged_workspace_bytes(const ConvGeom& g);

// Plan-driven variant (conv_plan.hpp); workspace = permuted weights + plan.  With a gate
// (device counter) the kernel runs only if *gate != 0.
bool planned_scatter_supported(const ConvGeom& g);
int planned_gemm_scatter(const ConvGeom& g, bool bf16, const float* pix, const float* map,
                         const float* wts, const float* Wm, float* img, float* workspace,
                         const int* gate, hipStream_t stream, SharedPlan* shared = nullptr);

}  // namespace sdk
