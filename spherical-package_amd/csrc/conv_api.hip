// C entry points of mapped convolution and mapped transposed convolution.
// Each call is reduced to one of three contractions over a ConvGeom (see
// conv_internal.hpp) and routed to the fused MFMA kernels when they cover the
// request, otherwise to the generic im2col/col2im + GEMM path.
#include <hip/hip_runtime.h>

#include <mutex>

#include "conv_fused.hpp"
#include "conv_small.hpp"
#include "conv_internal.hpp"
#include "sdk_host.hpp"

using namespace sdk;

namespace {

size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

size_t generic_workspace_bytes(int64_t gather_channels, int64_t K, int64_t M, int dtype) {
  return align256((size_t)gather_channels * K * M * (dtype == SDK_F64 ? 8 : 4));
}

int check_common(const char* what, int64_t B, int64_t Cg, int64_t H, int64_t W, int64_t Cp,
                 int64_t M, int64_t K, int32_t P, const void* wts, int32_t dtype,
                 int32_t compute) {
  SDK_REQUIRE(B >= 0 && Cg >= 1 && Cp >= 1 && K >= 1, "%s: bad size", what);
  SDK_REQUIRE(H >= 1 && W >= 1 && H * W < ((int64_t)1 << 31), "%s: bad plane size", what);
  SDK_REQUIRE(M >= 1 && M < ((int64_t)1 << 31), "%s: bad pixel count", what);
  SDK_REQUIRE(Cg * K < ((int64_t)1 << 24) && Cp < ((int64_t)1 << 24), "%s: too many channels",
              what);
  SDK_REQUIRE(P >= 0 && (P == 0 || wts), "%s: weighted map needs interp_weights", what);
  SDK_REQUIRE(dtype == SDK_F32 || dtype == SDK_F64, "%s: unknown dtype %d", what, dtype);
  SDK_REQUIRE(compute == SDK_COMPUTE_NATIVE || compute == SDK_COMPUTE_BF16 ||
                  compute == SDK_COMPUTE_UNFUSED || compute == SDK_COMPUTE_SPLIT,
              "%s: unknown compute mode %d", what, compute);
  if (compute == SDK_COMPUTE_BF16 && dtype != SDK_F32)
    return fail(SDK_ERR_UNSUPPORTED, "%s: bf16 compute needs float32 tensors", what);
  return SDK_OK;
}

int check_workspace(const char* what, size_t need, void* ws, size_t ws_bytes) {
  if (!ws || ws_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "%s: needs %zu bytes of workspace, got %zu", what, need,
                ws ? ws_bytes : (size_t)0);
  return SDK_OK;
}

enum Op { GATHER_GEMM, GEMM_SCATTER, GATHER_WGRAD };

// a: pixel-side tensor for GEMM_SCATTER / GATHER_WGRAD inputs, image otherwise (see call sites).
// A plan buffer handed in by the caller (sdk_mapped_conv_plan_build), or none.
struct PlanArg {
  void* buffer = nullptr;
  size_t bytes = 0;
};

// The size check of a caller's plan buffer, also made up front by the combined backward calls
// so that a refused call has launched nothing.
int check_plan(const char* what, const ConvGeom& g, int dtype, int compute, PlanArg plan) {
  if (plan.buffer == nullptr || dtype != SDK_F32 || compute == SDK_COMPUTE_UNFUSED ||
      !fused_supported(g))
    return SDK_OK;
  const size_t need = cached_plan_bytes(g);
  if (need == 0 || plan.bytes < need)
    return fail(SDK_ERR_WORKSPACE, "%s: the plan buffer has %zu bytes, this geometry's plan %zu",
                what, plan.bytes, need);
  return SDK_OK;
}

int run(const char* what, Op op, const ConvGeom& g, int dtype, int compute, const void* in0,
        const void* map, const void* wts, const void* in1, const void* bias, void* out, void* ws,
        size_t ws_bytes, hipStream_t stream, SharedPlan* shared, PlanArg plan) {
  if (g.B == 0 && op != GATHER_WGRAD) return SDK_OK;
  if (dtype == SDK_F32 && compute != SDK_COMPUTE_UNFUSED && fused_supported(g)) {
    int rc = check_workspace(what, fused_workspace_bytes(g), ws, ws_bytes);
    if (rc) return rc;
    CachedPlan cached;
    const CachedPlan* cp = nullptr;
    if (plan.buffer != nullptr) {
      rc = check_plan(what, g, dtype, compute, plan);
      if (rc) return rc;
      load_cached_plan(g, plan.buffer, &cached);
      cp = &cached;
    }
    const float* m = (const float*)map;
    const float* w = (const float*)wts;
    switch (op) {
      case GATHER_GEMM:
        return fused_gather_gemm(g, compute, (const float*)in0, m, w, (const float*)in1,
                                 (const float*)bias, (float*)out, (float*)ws, stream, cp);
      case GEMM_SCATTER:
        return fused_gemm_scatter(g, compute, (const float*)in0, m, w, (const float*)in1,
                                  (const float*)bias, (float*)out, (float*)ws, stream, shared, cp);
      case GATHER_WGRAD:
        return fused_gather_wgrad(g, compute, (const float*)in0, m, w, (const float*)in1,
                                  (float*)out, (float*)ws, stream, shared, cp);
    }
  }
  if (compute == SDK_COMPUTE_BF16)
    return fail(SDK_ERR_UNSUPPORTED, "%s: bf16 compute is not available for this shape", what);
  int rc = check_workspace(what, generic_workspace_bytes(g.Cg, g.K, g.M, dtype), ws, ws_bytes);
  if (rc) return rc;
  SDK_DISPATCH_DTYPE(dtype, {
    switch (op) {
      case GATHER_GEMM:
        return generic_gather_gemm<T>(g, (const T*)in0, (const T*)map, (const T*)wts,
                                      (const T*)in1, (const T*)bias, (T*)out, (T*)ws, stream);
      case GEMM_SCATTER:
        return generic_gemm_scatter<T>(g, (const T*)in0, (const T*)map, (const T*)wts,
                                       (const T*)in1, (const T*)bias, (T*)out, (T*)ws, stream);
      case GATHER_WGRAD:
        return generic_gather_wgrad<T>(g, (const T*)in0, (const T*)map, (const T*)wts,
                                       (const T*)in1, (T*)out, (T*)ws, stream);
    }
  });
  return SDK_OK;
}

}  // namespace

// ---------------------------------------------------------------------------
// The bias gradient of a combined backward call reads grad_output once and is bound by HBM; the
// two contractions beside it are bound by the matrix unit and leave HBM idle.  It runs on a
// stream of the library's own (default priority), forked from the caller's stream before the
// contractions and joined behind them, so that its waves take the slots the contraction
// workgroups leave free.  One side stream and event pair per device, created at the first
// call; if that fails (or the call is being captured into a graph) the bias gradient simply
// runs on the caller's stream, as it does when grad_output is small.
// ---------------------------------------------------------------------------
namespace {
// grad_output of at least this many bytes (a bias gradient of about 0.1 ms) goes to the side stream
constexpr int64_t kSideStreamBytes = (int64_t)384 << 20;
inline bool side_worth(int64_t batch, int64_t channels, int64_t pixels, int32_t dtype) {
  return batch * channels * pixels * (dtype == SDK_F64 ? 8 : 4) >= kSideStreamBytes;
}
struct SideStream {
  bool tried = false, ok = false;
  hipStream_t s = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
};
constexpr int kMaxDevices = 64;
SideStream g_side[kMaxDevices];
std::mutex g_side_mutex;

// Runs `work(stream_to_use)` forked from `stream`; returns with *joined = the event the caller's
// stream must wait for afterwards (nullptr: the work ran on the caller's stream).
// worth: whether the work is long enough to pay for the fork and the join (about 50 us of
// stream synchronisation, measured on a 64 us convolution step and on a 1.8 ms one).
template <typename Work>
int fork_side(hipStream_t stream, hipEvent_t* joined, bool worth, Work work) {
  *joined = nullptr;
  if (!worth) return work(stream);
  int dev = -1;
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices ||
      hipStreamIsCapturing(stream, &cap) != hipSuccess || cap != hipStreamCaptureStatusNone) {
    (void)hipGetLastError();
    return work(stream);
  }
  std::lock_guard<std::mutex> lock(g_side_mutex);
  SideStream& ss = g_side[dev];
  if (!ss.tried) {
    ss.tried = true;
    ss.ok = hipStreamCreateWithFlags(&ss.s, hipStreamNonBlocking) == hipSuccess &&
            hipEventCreateWithFlags(&ss.fork, hipEventDisableTiming) == hipSuccess &&
            hipEventCreateWithFlags(&ss.join, hipEventDisableTiming) == hipSuccess;
    if (!ss.ok) (void)hipGetLastError();
  }
  if (!ss.ok || hipEventRecord(ss.fork, stream) != hipSuccess ||
      hipStreamWaitEvent(ss.s, ss.fork, 0) != hipSuccess) {
    (void)hipGetLastError();
    return work(stream);
  }
  const int rc = work(ss.s);
  if (hipEventRecord(ss.join, ss.s) != hipSuccess)
    return fail(SDK_ERR_DEVICE, "backward: cannot record the side stream's event");
  *joined = ss.join;
  return rc;
}
}  // namespace

extern "C" {

size_t sdk_mapped_conv_workspace_bytes(int64_t batch, int64_t in_channels, int64_t out_channels,
                                       int64_t image_height, int64_t image_width,
                                       int64_t map_height, int64_t map_width,
                                       int64_t kernel_size, int32_t num_interp_pts,
                                       int32_t interp, int32_t dtype, int32_t compute) {
  if (map_height < 1 || map_width < 1 || map_height * map_width >= ((int64_t)1 << 31)) return 0;
  if (image_height < 1 || image_width < 1 || image_height * image_width >= ((int64_t)1 << 31))
    return 0;
  const int64_t gather_pixels = map_height * map_width;
  // Upper bound over the conv (gather side = in_channels) and transposed conv
  // (gather side = out_channels) roles, so one query serves a whole layer call.
  ConvGeom a{batch, (int)in_channels, (int)image_height, (int)image_width, (int)out_channels,
             (int)gather_pixels, (int)kernel_size, num_interp_pts, interp, (int)map_width};
  ConvGeom b{batch, (int)out_channels, (int)image_height, (int)image_width, (int)in_channels,
             (int)gather_pixels, (int)kernel_size, num_interp_pts, interp, (int)map_width};
  if (dtype == SDK_F32 && compute != SDK_COMPUTE_UNFUSED && fused_supported(a) &&
      fused_supported(b))
    return align256(std::max(fused_workspace_bytes(a), fused_workspace_bytes(b)));
  return generic_workspace_bytes(std::max(in_channels, out_channels), kernel_size, gather_pixels,
                                 dtype);
}

static int impl_mapped_conv_forward(const void* input, const void* sample_map, const void* interp_weights,
                            const void* weight, const void* bias, void* output, void* workspace,
                            size_t workspace_bytes, int64_t batch, int64_t in_channels,
                            int64_t height, int64_t width, int64_t out_channels,
                            int64_t out_height, int64_t out_width, int64_t kernel_size,
                            int32_t num_interp_pts, int32_t interp, int32_t dtype,
                            int32_t compute, sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_conv_forward";
  SDK_REQUIRE(input && sample_map && weight && bias && output, "%s: NULL pointer", what);
  SDK_REQUIRE(out_height >= 1 && out_width >= 1, "%s: bad output size", what);
  const int64_t M = out_height * out_width;
  int rc = check_common(what, batch, in_channels, height, width, out_channels, M, kernel_size,
                        num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)in_channels, (int)height, (int)width, (int)out_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)out_width};
  return run(what, GATHER_GEMM, g, dtype, compute, input, sample_map, interp_weights, weight, bias,
             output, workspace, workspace_bytes, (hipStream_t)stream, nullptr, plan);
}

static int impl_mapped_conv_backward_input(const void* grad_output, const void* sample_map,
                                   const void* interp_weights, const void* weight,
                                   void* grad_input, void* workspace, size_t workspace_bytes,
                                   int64_t batch, int64_t in_channels, int64_t height,
                                   int64_t width, int64_t out_channels, int64_t out_height,
                                   int64_t out_width, int64_t kernel_size,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   int32_t compute, sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_conv_backward_input";
  SDK_REQUIRE(grad_output && sample_map && weight && grad_input, "%s: NULL pointer", what);
  SDK_REQUIRE(out_height >= 1 && out_width >= 1, "%s: bad output size", what);
  const int64_t M = out_height * out_width;
  int rc = check_common(what, batch, in_channels, height, width, out_channels, M, kernel_size,
                        num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)in_channels, (int)height, (int)width, (int)out_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)out_width};
  return run(what, GEMM_SCATTER, g, dtype, compute, grad_output, sample_map, interp_weights,
             weight, nullptr, grad_input, workspace, workspace_bytes, (hipStream_t)stream, nullptr,
             plan);
}

static int impl_mapped_conv_backward_weight(const void* grad_output, const void* sample_map,
                                    const void* interp_weights, const void* input,
                                    void* grad_weight, void* workspace, size_t workspace_bytes,
                                    int64_t batch, int64_t in_channels, int64_t height,
                                    int64_t width, int64_t out_channels, int64_t out_height,
                                    int64_t out_width, int64_t kernel_size,
                                    int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                    int32_t compute, sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_conv_backward_weight";
  SDK_REQUIRE(grad_output && sample_map && input && grad_weight, "%s: NULL pointer", what);
  SDK_REQUIRE(out_height >= 1 && out_width >= 1, "%s: bad output size", what);
  const int64_t M = out_height * out_width;
  int rc = check_common(what, batch, in_channels, height, width, out_channels, M, kernel_size,
                        num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)in_channels, (int)height, (int)width, (int)out_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)out_width};
  return run(what, GATHER_WGRAD, g, dtype, compute, grad_output, sample_map, interp_weights, input,
             nullptr, grad_weight, workspace, workspace_bytes, (hipStream_t)stream, nullptr, plan);
}

static int impl_mapped_transposed_conv_forward(const void* input, const void* sample_map,
                                       const void* interp_weights, const void* weight,
                                       const void* bias, void* output, void* workspace,
                                       size_t workspace_bytes, int64_t batch,
                                       int64_t in_channels, int64_t in_height, int64_t in_width,
                                       int64_t out_channels, int64_t out_height,
                                       int64_t out_width, int64_t kernel_size,
                                       int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                       int32_t compute, sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_transposed_conv_forward";
  SDK_REQUIRE(input && sample_map && weight && bias && output, "%s: NULL pointer", what);
  SDK_REQUIRE(in_height >= 1 && in_width >= 1, "%s: bad input size", what);
  const int64_t M = in_height * in_width;
  int rc = check_common(what, batch, out_channels, out_height, out_width, in_channels, M,
                        kernel_size, num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)out_channels, (int)out_height, (int)out_width, (int)in_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)in_width};
  return run(what, GEMM_SCATTER, g, dtype, compute, input, sample_map, interp_weights, weight,
             bias, output, workspace, workspace_bytes, (hipStream_t)stream, nullptr, plan);
}

static int impl_mapped_transposed_conv_backward_input(const void* grad_output, const void* sample_map,
                                              const void* interp_weights, const void* weight,
                                              void* grad_input, void* workspace,
                                              size_t workspace_bytes, int64_t batch,
                                              int64_t in_channels, int64_t in_height,
                                              int64_t in_width, int64_t out_channels,
                                              int64_t out_height, int64_t out_width,
                                              int64_t kernel_size, int32_t num_interp_pts,
                                              int32_t interp, int32_t dtype, int32_t compute,
                                              sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_transposed_conv_backward_input";
  SDK_REQUIRE(grad_output && sample_map && weight && grad_input, "%s: NULL pointer", what);
  SDK_REQUIRE(in_height >= 1 && in_width >= 1, "%s: bad input size", what);
  const int64_t M = in_height * in_width;
  int rc = check_common(what, batch, out_channels, out_height, out_width, in_channels, M,
                        kernel_size, num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)out_channels, (int)out_height, (int)out_width, (int)in_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)in_width};
  return run(what, GATHER_GEMM, g, dtype, compute, grad_output, sample_map, interp_weights, weight,
             nullptr, grad_input, workspace, workspace_bytes, (hipStream_t)stream, nullptr, plan);
}

static int impl_mapped_transposed_conv_backward_weight(const void* grad_output, const void* sample_map,
                                               const void* interp_weights, const void* input,
                                               void* grad_weight, void* workspace,
                                               size_t workspace_bytes, int64_t batch,
                                               int64_t in_channels, int64_t in_height,
                                               int64_t in_width, int64_t out_channels,
                                               int64_t out_height, int64_t out_width,
                                               int64_t kernel_size, int32_t num_interp_pts,
                                               int32_t interp, int32_t dtype, int32_t compute,
                                               sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_transposed_conv_backward_weight";
  SDK_REQUIRE(grad_output && sample_map && input && grad_weight, "%s: NULL pointer", what);
  SDK_REQUIRE(in_height >= 1 && in_width >= 1, "%s: bad input size", what);
  const int64_t M = in_height * in_width;
  int rc = check_common(what, batch, out_channels, out_height, out_width, in_channels, M,
                        kernel_size, num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)out_channels, (int)out_height, (int)out_width, (int)in_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)in_width};
  return run(what, GATHER_WGRAD, g, dtype, compute, input, sample_map, interp_weights,
             grad_output, nullptr, grad_weight, workspace, workspace_bytes, (hipStream_t)stream,
             nullptr, plan);
}

static int impl_mapped_conv_backward(const void* grad_output, const void* sample_map,
                             const void* interp_weights, const void* input, const void* weight,
                             void* grad_input, void* grad_weight, void* grad_bias,
                             void* workspace, size_t workspace_bytes, int64_t batch,
                             int64_t in_channels, int64_t height, int64_t width,
                             int64_t out_channels, int64_t out_height, int64_t out_width,
                             int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                             int32_t dtype, int32_t compute, sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_conv_backward";
  SDK_REQUIRE(grad_output && sample_map && input && weight && grad_input && grad_weight &&
                  grad_bias,
              "%s: NULL pointer", what);
  SDK_REQUIRE(out_height >= 1 && out_width >= 1, "%s: bad output size", what);
  const int64_t M = out_height * out_width;
  int rc = check_common(what, batch, in_channels, height, width, out_channels, M, kernel_size,
                        num_interp_pts, interp_weights, dtype, compute);
  if (rc) return rc;
  ConvGeom g{batch, (int)in_channels, (int)height, (int)width, (int)out_channels, (int)M,
             (int)kernel_size, num_interp_pts, interp, (int)out_width};
  rc = check_plan(what, g, dtype, compute, plan);
  if (rc) return rc;
  SharedPlan shared;   // the tap plan of the map is built once for both contractions
  // A layer with at most four image channels runs three small kernels, each adding into a
  // target that has to start from zero: the three targets are cleared by one launch.
  if (dtype == SDK_F32 && compute != SDK_COMPUTE_UNFUSED && batch > 0 && fused_supported(g) &&
      small_conv_supported(g) && small_wgrad_supported(g) &&
      !side_worth(batch, out_channels, M, dtype)) {
    rc = zero_fill3(grad_bias, sizeof(float) * (size_t)out_channels, grad_input,
                    sizeof(float) * (size_t)batch * in_channels * height * width, grad_weight,
                    sizeof(float) * (size_t)out_channels * in_channels * kernel_size,
                    (hipStream_t)stream);
    if (rc) return rc;
    shared.cleared = true;
    shared.bias_sum = static_cast<float*>(grad_bias);   // summed by the weight-gradient kernel
  }
  hipEvent_t joined = nullptr;
  if (!shared.cleared)
    rc = fork_side((hipStream_t)stream, &joined, side_worth(batch, out_channels, M, dtype),
                   [&](hipStream_t s) {
      return bias_grad(grad_output, grad_bias, batch, out_channels, M, dtype, s,
                       s != (hipStream_t)stream);
    });
  if (rc == SDK_OK)
    rc = run(what, GEMM_SCATTER, g, dtype, compute, grad_output, sample_map, interp_weights,
             weight, nullptr, grad_input, workspace, workspace_bytes, (hipStream_t)stream, &shared,
             plan);
  if (rc == SDK_OK)
    rc = run(what, GATHER_WGRAD, g, dtype, compute, grad_output, sample_map, interp_weights, input,
             nullptr, grad_weight, workspace, workspace_bytes, (hipStream_t)stream, &shared, plan);
  // (joined also after an error: the caller's stream must not run ahead of the side stream)
  if (joined != nullptr && hipStreamWaitEvent((hipStream_t)stream, joined, 0) != hipSuccess)
    return fail(SDK_ERR_DEVICE, "%s: cannot join the side stream", what);
  return rc;
}

static int impl_mapped_transposed_conv_backward(const void* grad_output, const void* sample_map,
                                        const void* interp_weights, const void* input,
                                        const void* weight, void* grad_input, void* grad_weight,
                                        void* grad_bias, void* workspace, size_t workspace_bytes,
                                        int64_t batch, int64_t in_channels, int64_t in_height,
                                        int64_t in_width, int64_t out_channels,
                                        int64_t out_height, int64_t out_width,
                                        int64_t kernel_size, int32_t num_interp_pts,
                                        int32_t interp, int32_t dtype, int32_t compute,
                                        sdk_stream_t stream, PlanArg plan) {
  const char* what = "mapped_transposed_conv_backward";
  SDK_REQUIRE(grad_output && grad_bias, "%s: NULL pointer", what);
  SDK_REQUIRE(out_height >= 1 && out_width >= 1 && out_height * out_width < ((int64_t)1 << 31),
              "%s: bad output size", what);
  SDK_REQUIRE(in_height >= 1 && in_width >= 1, "%s: bad input size", what);
  int rc = check_common(what, batch, out_channels, out_height, out_width, in_channels,
                        in_height * in_width, kernel_size, num_interp_pts, interp_weights, dtype,
                        compute);
  if (rc) return rc;
  {
    ConvGeom g{batch, (int)out_channels, (int)out_height, (int)out_width, (int)in_channels,
               (int)(in_height * in_width), (int)kernel_size, num_interp_pts, interp,
               (int)in_width};
    rc = check_plan(what, g, dtype, compute, plan);
    if (rc) return rc;
  }
  hipEvent_t joined = nullptr;
  rc = fork_side((hipStream_t)stream, &joined,
                     side_worth(batch, out_channels, out_height * out_width, dtype),
                     [&](hipStream_t s) {
    return bias_grad(grad_output, grad_bias, batch, out_channels, out_height * out_width, dtype, s,
                     s != (hipStream_t)stream);
  });
  if (rc == SDK_OK)
    rc = impl_mapped_transposed_conv_backward_input(
        grad_output, sample_map, interp_weights, weight, grad_input, workspace, workspace_bytes,
        batch, in_channels, in_height, in_width, out_channels, out_height, out_width,
        kernel_size, num_interp_pts, interp, dtype, compute, stream, plan);
  if (rc == SDK_OK)
    rc = impl_mapped_transposed_conv_backward_weight(
        grad_output, sample_map, interp_weights, input, grad_weight, workspace, workspace_bytes,
        batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size,
        num_interp_pts, interp, dtype, compute, stream, plan);
  if (joined != nullptr && hipStreamWaitEvent((hipStream_t)stream, joined, 0) != hipSuccess)
    return fail(SDK_ERR_DEVICE, "%s: cannot join the side stream", what);
  return rc;
}


size_t sdk_mapped_conv_plan_bytes(int64_t image_height, int64_t image_width, int64_t map_height,
                                  int64_t map_width, int64_t kernel_size, int32_t num_interp_pts,
                                  int32_t interp, int32_t dtype) {
  if (dtype != SDK_F32 || map_height < 1 || map_width < 1 || image_height < 1 || image_width < 1 ||
      kernel_size < 1 || num_interp_pts < 0 ||
      map_height * map_width >= ((int64_t)1 << 31) || image_height * image_width >= ((int64_t)1 << 31))
    return 0;
  ConvGeom g{1, 1, (int)image_height, (int)image_width, 1, (int)(map_height * map_width),
             (int)kernel_size, num_interp_pts, interp, (int)map_width};
  if (!fused_supported(g)) return 0;
  return cached_plan_bytes(g);
}

int sdk_mapped_conv_plan_build(const void* sample_map, const void* interp_weights, void* plan,
                               size_t plan_bytes, int64_t image_height, int64_t image_width,
                               int64_t map_height, int64_t map_width, int64_t kernel_size,
                               int32_t num_interp_pts, int32_t interp, int32_t dtype,
                               sdk_stream_t stream) {
  const char* what = "mapped_conv_plan_build";
  SDK_REQUIRE(sample_map && plan, "%s: NULL pointer", what);
  SDK_REQUIRE(num_interp_pts >= 0 && (num_interp_pts == 0 || interp_weights),
              "%s: weighted map needs interp_weights", what);
  const size_t need = sdk_mapped_conv_plan_bytes(image_height, image_width, map_height, map_width,
                                                 kernel_size, num_interp_pts, interp, dtype);
  if (need == 0)
    return fail(SDK_ERR_UNSUPPORTED, "%s: no plan for this geometry (ask sdk_mapped_conv_plan_bytes)",
                what);
  if (plan_bytes < need)
    return fail(SDK_ERR_WORKSPACE, "%s: needs %zu bytes, got %zu", what, need, plan_bytes);
  ConvGeom g{1, 1, (int)image_height, (int)image_width, 1, (int)(map_height * map_width),
             (int)kernel_size, num_interp_pts, interp, (int)map_width};
  return build_cached_plan(g, (const float*)sample_map, (const float*)interp_weights, plan,
                           (hipStream_t)stream);
}

int sdk_mapped_conv_forward(const void* input, const void* sample_map, const void* interp_weights,
                            const void* weight, const void* bias, void* output, void* workspace,
                            size_t workspace_bytes, int64_t batch, int64_t in_channels,
                            int64_t height, int64_t width, int64_t out_channels,
                            int64_t out_height, int64_t out_width, int64_t kernel_size,
                            int32_t num_interp_pts, int32_t interp, int32_t dtype,
                            int32_t compute, sdk_stream_t stream) {
  return impl_mapped_conv_forward(input, sample_map, interp_weights, weight, bias, output, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_conv_forward_planned(const void* input, const void* sample_map, const void* interp_weights,
                            const void* weight, const void* bias, void* output, void* workspace,
                            size_t workspace_bytes, void* plan,
    size_t plan_bytes, int64_t batch, int64_t in_channels,
                            int64_t height, int64_t width, int64_t out_channels,
                            int64_t out_height, int64_t out_width, int64_t kernel_size,
                            int32_t num_interp_pts, int32_t interp, int32_t dtype,
                            int32_t compute, sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_conv_forward(input, sample_map, interp_weights, weight, bias, output, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_conv_backward_input(const void* grad_output, const void* sample_map,
                                   const void* interp_weights, const void* weight,
                                   void* grad_input, void* workspace, size_t workspace_bytes,
                                   int64_t batch, int64_t in_channels, int64_t height,
                                   int64_t width, int64_t out_channels, int64_t out_height,
                                   int64_t out_width, int64_t kernel_size,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   int32_t compute, sdk_stream_t stream) {
  return impl_mapped_conv_backward_input(grad_output, sample_map, interp_weights, weight, grad_input, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_conv_backward_input_planned(const void* grad_output, const void* sample_map,
                                   const void* interp_weights, const void* weight,
                                   void* grad_input, void* workspace, size_t workspace_bytes, void* plan,
    size_t plan_bytes,
                                   int64_t batch, int64_t in_channels, int64_t height,
                                   int64_t width, int64_t out_channels, int64_t out_height,
                                   int64_t out_width, int64_t kernel_size,
                                   int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                   int32_t compute, sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_conv_backward_input(grad_output, sample_map, interp_weights, weight, grad_input, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_conv_backward_weight(const void* grad_output, const void* sample_map,
                                    const void* interp_weights, const void* input,
                                    void* grad_weight, void* workspace, size_t workspace_bytes,
                                    int64_t batch, int64_t in_channels, int64_t height,
                                    int64_t width, int64_t out_channels, int64_t out_height,
                                    int64_t out_width, int64_t kernel_size,
                                    int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                    int32_t compute, sdk_stream_t stream) {
  return impl_mapped_conv_backward_weight(grad_output, sample_map, interp_weights, input, grad_weight, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_conv_backward_weight_planned(const void* grad_output, const void* sample_map,
                                    const void* interp_weights, const void* input,
                                    void* grad_weight, void* workspace, size_t workspace_bytes, void* plan,
    size_t plan_bytes,
                                    int64_t batch, int64_t in_channels, int64_t height,
                                    int64_t width, int64_t out_channels, int64_t out_height,
                                    int64_t out_width, int64_t kernel_size,
                                    int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                    int32_t compute, sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_conv_backward_weight(grad_output, sample_map, interp_weights, input, grad_weight, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_transposed_conv_forward(const void* input, const void* sample_map,
                                       const void* interp_weights, const void* weight,
                                       const void* bias, void* output, void* workspace,
                                       size_t workspace_bytes, int64_t batch,
                                       int64_t in_channels, int64_t in_height, int64_t in_width,
                                       int64_t out_channels, int64_t out_height,
                                       int64_t out_width, int64_t kernel_size,
                                       int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                       int32_t compute, sdk_stream_t stream) {
  return impl_mapped_transposed_conv_forward(input, sample_map, interp_weights, weight, bias, output, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_transposed_conv_forward_planned(const void* input, const void* sample_map,
                                       const void* interp_weights, const void* weight,
                                       const void* bias, void* output, void* workspace,
                                       size_t workspace_bytes, void* plan,
    size_t plan_bytes, int64_t batch,
                                       int64_t in_channels, int64_t in_height, int64_t in_width,
                                       int64_t out_channels, int64_t out_height,
                                       int64_t out_width, int64_t kernel_size,
                                       int32_t num_interp_pts, int32_t interp, int32_t dtype,
                                       int32_t compute, sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_transposed_conv_forward(input, sample_map, interp_weights, weight, bias, output, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_transposed_conv_backward_input(const void* grad_output, const void* sample_map,
                                              const void* interp_weights, const void* weight,
                                              void* grad_input, void* workspace,
                                              size_t workspace_bytes, int64_t batch,
                                              int64_t in_channels, int64_t in_height,
                                              int64_t in_width, int64_t out_channels,
                                              int64_t out_height, int64_t out_width,
                                              int64_t kernel_size, int32_t num_interp_pts,
                                              int32_t interp, int32_t dtype, int32_t compute,
                                              sdk_stream_t stream) {
  return impl_mapped_transposed_conv_backward_input(grad_output, sample_map, interp_weights, weight, grad_input, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_transposed_conv_backward_input_planned(const void* grad_output, const void* sample_map,
                                              const void* interp_weights, const void* weight,
                                              void* grad_input, void* workspace,
                                              size_t workspace_bytes, void* plan,
    size_t plan_bytes, int64_t batch,
                                              int64_t in_channels, int64_t in_height,
                                              int64_t in_width, int64_t out_channels,
                                              int64_t out_height, int64_t out_width,
                                              int64_t kernel_size, int32_t num_interp_pts,
                                              int32_t interp, int32_t dtype, int32_t compute,
                                              sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_transposed_conv_backward_input(grad_output, sample_map, interp_weights, weight, grad_input, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_transposed_conv_backward_weight(const void* grad_output, const void* sample_map,
                                               const void* interp_weights, const void* input,
                                               void* grad_weight, void* workspace,
                                               size_t workspace_bytes, int64_t batch,
                                               int64_t in_channels, int64_t in_height,
                                               int64_t in_width, int64_t out_channels,
                                               int64_t out_height, int64_t out_width,
                                               int64_t kernel_size, int32_t num_interp_pts,
                                               int32_t interp, int32_t dtype, int32_t compute,
                                               sdk_stream_t stream) {
  return impl_mapped_transposed_conv_backward_weight(grad_output, sample_map, interp_weights, input, grad_weight, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_transposed_conv_backward_weight_planned(const void* grad_output, const void* sample_map,
                                               const void* interp_weights, const void* input,
                                               void* grad_weight, void* workspace,
                                               size_t workspace_bytes, void* plan,
    size_t plan_bytes, int64_t batch,
                                               int64_t in_channels, int64_t in_height,
                                               int64_t in_width, int64_t out_channels,
                                               int64_t out_height, int64_t out_width,
                                               int64_t kernel_size, int32_t num_interp_pts,
                                               int32_t interp, int32_t dtype, int32_t compute,
                                               sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_transposed_conv_backward_weight(grad_output, sample_map, interp_weights, input, grad_weight, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_conv_backward(const void* grad_output, const void* sample_map,
                             const void* interp_weights, const void* input, const void* weight,
                             void* grad_input, void* grad_weight, void* grad_bias,
                             void* workspace, size_t workspace_bytes, int64_t batch,
                             int64_t in_channels, int64_t height, int64_t width,
                             int64_t out_channels, int64_t out_height, int64_t out_width,
                             int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                             int32_t dtype, int32_t compute, sdk_stream_t stream) {
  return impl_mapped_conv_backward(grad_output, sample_map, interp_weights, input, weight, grad_input, grad_weight, grad_bias, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_conv_backward_planned(const void* grad_output, const void* sample_map,
                             const void* interp_weights, const void* input, const void* weight,
                             void* grad_input, void* grad_weight, void* grad_bias,
                             void* workspace, size_t workspace_bytes, void* plan,
    size_t plan_bytes, int64_t batch,
                             int64_t in_channels, int64_t height, int64_t width,
                             int64_t out_channels, int64_t out_height, int64_t out_width,
                             int64_t kernel_size, int32_t num_interp_pts, int32_t interp,
                             int32_t dtype, int32_t compute, sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_conv_backward(grad_output, sample_map, interp_weights, input, weight, grad_input, grad_weight, grad_bias, workspace, workspace_bytes, batch, in_channels, height, width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

int sdk_mapped_transposed_conv_backward(const void* grad_output, const void* sample_map,
                                        const void* interp_weights, const void* input,
                                        const void* weight, void* grad_input, void* grad_weight,
                                        void* grad_bias, void* workspace, size_t workspace_bytes,
                                        int64_t batch, int64_t in_channels, int64_t in_height,
                                        int64_t in_width, int64_t out_channels,
                                        int64_t out_height, int64_t out_width,
                                        int64_t kernel_size, int32_t num_interp_pts,
                                        int32_t interp, int32_t dtype, int32_t compute,
                                        sdk_stream_t stream) {
  return impl_mapped_transposed_conv_backward(grad_output, sample_map, interp_weights, input, weight, grad_input, grad_weight, grad_bias, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, PlanArg());
}

int sdk_mapped_transposed_conv_backward_planned(const void* grad_output, const void* sample_map,
                                        const void* interp_weights, const void* input,
                                        const void* weight, void* grad_input, void* grad_weight,
                                        void* grad_bias, void* workspace, size_t workspace_bytes, void* plan,
    size_t plan_bytes,
                                        int64_t batch, int64_t in_channels, int64_t in_height,
                                        int64_t in_width, int64_t out_channels,
                                        int64_t out_height, int64_t out_width,
                                        int64_t kernel_size, int32_t num_interp_pts,
                                        int32_t interp, int32_t dtype, int32_t compute,
                                        sdk_stream_t stream) {
  PlanArg pa;
  pa.buffer = plan;
  pa.bytes = plan_bytes;
  return impl_mapped_transposed_conv_backward(grad_output, sample_map, interp_weights, input, weight, grad_input, grad_weight, grad_bias, workspace, workspace_bytes, batch, in_channels, in_height, in_width, out_channels, out_height, out_width, kernel_size, num_interp_pts, interp, dtype, compute, stream, pa);
}

}  // extern "C"
