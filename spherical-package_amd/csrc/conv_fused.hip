#include "conv_fused.hpp"

#include "sdk_host.hpp"

namespace sdk {
bool fused_supported(const ConvGeom&) { return false; }
int fused_gather_gemm(const ConvGeom&, int, const float*, const float*, const float*, const float*,
                      const float*, float*, hipStream_t) {
  return fail(SDK_ERR_UNSUPPORTED, "fused path not built");
}
int fused_gemm_scatter(const ConvGeom&, int, const float*, const float*, const float*,
                       const float*, const float*, float*, hipStream_t) {
  return fail(SDK_ERR_UNSUPPORTED, "fused path not built");
}
int fused_gather_wgrad(const ConvGeom&, int, const float*, const float*, const float*,
                       const float*, float*, hipStream_t) {
  return fail(SDK_ERR_UNSUPPORTED, "fused path not built");
}
}  // namespace sdk
