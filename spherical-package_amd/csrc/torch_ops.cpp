// Compiled PyTorch-ROCm operator layer over the C ABI of libsdk_mapped_ops.so.
//
// Registers, for the CUDA (= HIP on ROCm) dispatch key, the operators of the `sdk_mapped_ops`
// namespace whose per-call cost matters: each checks its tensors the way the reference's
// pybind entry points do (contiguous, all on the GPU: ext_modules/include/cuda_helper.h:12-18;
// ext_modules/include/layers/mapped_convolution_layer.h:62-143 is the shape of such an entry
// point), allocates the outputs, fetches the current HIP stream, looks up or builds the plan of
// the map and makes one call into the C ABI.  The schemas are defined from Python
// (_spherical_distortion_ext/_ops.py), which loads this library when it is built and registers
// its own implementations of the same operators when it is not; both keep the same plan cache
// rules: keyed on the map's storage, offset, version counter, shape and the geometry; least
// recently used entry dropped first; maps without a version counter (inference tensors) and
// keys that miss during a stream capture go to the entry points that build what they need
// inside the call.
//
// Built with the host compiler against the torch headers; no device code here.
#include <ATen/ATen.h>
#include <c10/core/DeviceGuard.h>
#include <c10/hip/HIPStream.h>
#include <hip/hip_runtime_api.h>
#include <torch/library.h>

#include <cstdint>
#include <list>
#include <mutex>
#include <string>
#include <vector>

#include "sdk_mapped_ops.h"

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;

// ----------------------------------------------------------------------------- state
std::mutex g_mu;
int g_default_mode = SDK_COMPUTE_NATIVE;
thread_local int t_mode = -1;   // -1: no override on this thread
bool g_cache_enabled = true;
size_t g_cache_max = 16;
bool g_unpool_workspace = true;

int current_mode() { return t_mode >= 0 ? t_mode : g_default_mode; }

struct TensorKey {
  bool present = false;
  const void* storage = nullptr;
  int64_t offset = 0, version = 0;
  std::vector<int64_t> shape;
  bool operator==(const TensorKey& o) const {
    return present == o.present && storage == o.storage && offset == o.offset &&
           version == o.version && shape == o.shape;
  }
};

// false: the tensor's changes cannot be tracked (no version counter)
bool tensor_key(const OptTensor& t, TensorKey* k) {
  if (!t.has_value() || !t->defined()) return true;
  if (t->is_inference()) return false;
  k->present = true;
  k->storage = t->storage().data();
  k->offset = t->storage_offset();
  k->version = (int64_t)t->_version();
  k->shape = t->sizes().vec();
  return true;
}

enum Kind { kConv = 0, kResample = 1, kAvgUnpool = 2, kMaxUnpool = 3 };

struct Key {
  int kind = 0, device = 0, dtype = 0;
  TensorKey map, wts;
  int64_t a = 0, b = 0, K = 0, P = 0, interp = 0;
  bool operator==(const Key& o) const {
    return kind == o.kind && device == o.device && dtype == o.dtype && map == o.map &&
           wts == o.wts && a == o.a && b == o.b && K == o.K && P == o.P && interp == o.interp;
  }
};

struct Entry {
  Key key;
  Tensor plan;
  size_t nbytes = 0;
  c10::Storage keep_map, keep_wts;   // an address cannot be reused while its entry lives
  hipStream_t stream = nullptr;      // last user: a call on another stream is ordered behind it
  int complete = 0;
};
std::list<Entry> g_cache;   // most recently used last

struct PlanRef {
  Tensor plan;   // undefined: none
  size_t nbytes = 0;
  int complete = 0;
  void* ptr() const { return plan.defined() ? plan.data_ptr() : nullptr; }
};

void order_behind(hipStream_t cur, hipStream_t last) {
  if (cur == last) return;
  hipEvent_t ev = nullptr;
  if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) return;
  if (hipEventRecord(ev, last) == hipSuccess) (void)hipStreamWaitEvent(cur, ev, 0);
  (void)hipEventDestroy(ev);
}

bool capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}

void fail_call(const char* name, int rc) {
  TORCH_CHECK(false, name, " failed (status ", rc, "): ", sdk_last_error());
}
#define SDK_CALL(name, ...)              \
  do {                                   \
    const int rc__ = name(__VA_ARGS__);  \
    if (rc__ != 0) fail_call(#name, rc__); \
  } while (0)

const void* cptr(const OptTensor& t) {
  return (t.has_value() && t->defined()) ? t->data_ptr() : nullptr;
}

int dtype_code(const Tensor& ref) {
  if (ref.scalar_type() == at::kFloat) return SDK_F32;
  if (ref.scalar_type() == at::kDouble) return SDK_F64;
  TORCH_CHECK(false, "unsupported dtype ", ref.scalar_type(), " (float32 and float64 only)");
}

void check_first(const Tensor& ref) {
  TORCH_CHECK(ref.is_cuda(), "this backend runs on the GPU only: tensors must be CUDA/HIP tensors");
  (void)dtype_code(ref);
}
void check_one(const Tensor& ref, const char* name, const Tensor& t, bool any_dtype = false) {
  TORCH_CHECK(t.is_contiguous(), name, " must be contiguous");
  TORCH_CHECK(t.is_cuda() && t.device() == ref.device(), name, " must be a CUDA tensor on ",
              ref.device());
  TORCH_CHECK(any_dtype || t.scalar_type() == ref.scalar_type(), name, " must have dtype ",
              ref.scalar_type(), " (got ", t.scalar_type(), ")");
}
void check_opt(const Tensor& ref, const char* name, const OptTensor& t) {
  if (t.has_value() && t->defined()) check_one(ref, name, *t);
}

// 0 for the unweighted map layout, P for the weighted one.
int64_t npts(const Tensor& map, const OptTensor& w, int64_t rank_unweighted) {
  if (!w.has_value() || !w->defined()) {
    TORCH_CHECK(map.dim() == rank_unweighted && map.size(-1) == 2, "sample_map must have ",
                rank_unweighted, " dimensions ending in 2, got ", map.sizes());
    return 0;
  }
  TORCH_CHECK(map.dim() == rank_unweighted + 1 && map.size(-1) == 2,
              "weighted sample_map must have ", rank_unweighted + 1,
              " dimensions ending in 2, got ", map.sizes());
  TORCH_CHECK(w->sizes() == map.sizes().slice(0, map.dim() - 1), "interp_weights shape ",
              w->sizes(), " does not match sample_map ", map.sizes());
  return w->size(-1);
}

hipStream_t stream_of(const Tensor& ref) {
  return c10::hip::getCurrentHIPStream(ref.device().index()).stream();
}

Tensor bytes_on(const Tensor& ref, size_t n) {
  return at::empty({(int64_t)n}, ref.options().dtype(at::kByte));
}

// The kept plan of `key`, or one built by `build` (which returns the plan's size, 0 for none,
// and fills the buffer it is handed on `stream`).
template <typename Size, typename Build>
PlanRef plan_for(Key key, const Tensor& ref, const Tensor& map, const OptTensor& wts,
                 hipStream_t stream, Size size, Build build) {
  PlanRef out;
  if (!g_cache_enabled) return out;
  if (!tensor_key(map, &key.map) || !tensor_key(wts, &key.wts)) return out;
  std::lock_guard<std::mutex> lock(g_mu);
  for (auto it = g_cache.begin(); it != g_cache.end(); ++it) {
    if (it->key == key) {
      g_cache.splice(g_cache.end(), g_cache, it);   // most recently used
      Entry& e = g_cache.back();
      order_behind(stream, e.stream);
      e.stream = stream;
      out.plan = e.plan;
      out.nbytes = e.nbytes;
      out.complete = e.complete;
      return out;
    }
  }
  if (capturing(stream)) return out;
  const size_t n = size();
  if (n == 0) return out;
  Entry e;
  e.key = key;
  e.plan = bytes_on(ref, n);
  e.nbytes = n;
  e.complete = build(e.plan.data_ptr(), n);
  e.keep_map = map.storage();
  if (wts.has_value() && wts->defined()) e.keep_wts = wts->storage();
  e.stream = stream;
  while (g_cache.size() >= g_cache_max) g_cache.pop_front();
  g_cache.push_back(std::move(e));
  out.plan = g_cache.back().plan;
  out.nbytes = n;
  out.complete = g_cache.back().complete;
  return out;
}

PlanRef conv_plan(const Tensor& ref, const Tensor& map, const OptTensor& wts, int64_t img_h,
                  int64_t img_w, int64_t K, int64_t P, int64_t interp, hipStream_t stream) {
  if (ref.scalar_type() != at::kFloat) return PlanRef();
  const int64_t MH = map.size(0), MW = map.size(1);
  Key key;
  key.kind = kConv;
  key.device = ref.device().index();
  key.a = img_h;
  key.b = img_w;
  key.K = K;
  key.P = P;
  key.interp = interp;
  return plan_for(
      key, ref, map, wts, stream,
      [&] { return sdk_mapped_conv_plan_bytes(img_h, img_w, MH, MW, K, (int32_t)P, (int32_t)interp, SDK_F32); },
      [&](void* buf, size_t n) {
        SDK_CALL(sdk_mapped_conv_plan_build, map.data_ptr(), cptr(wts), buf, n, img_h, img_w, MH,
                 MW, K, (int32_t)P, (int32_t)interp, SDK_F32, stream);
        return 0;
      });
}

PlanRef scatter_plan(Kind kind, const Tensor& ref, const Tensor& map, const OptTensor& wts,
                     int64_t out_h, int64_t out_w, int64_t K, int64_t P, int64_t interp,
                     hipStream_t stream) {
  const int dt = dtype_code(ref);
  const int64_t MH = map.size(0), MW = map.size(1);
  Key key;
  key.kind = kind;
  key.device = ref.device().index();
  key.dtype = dt;
  key.a = out_h;
  key.b = out_w;
  key.K = K;
  key.P = P;
  key.interp = interp;
  return plan_for(
      key, ref, map, wts, stream,
      [&] {
        return kind == kMaxUnpool ? sdk_mapped_max_unpool_workspace_bytes(out_h, out_w, dt)
                                  : sdk_resample_to_map_workspace_bytes(out_h, out_w, dt);
      },
      [&](void* buf, size_t n) {
        if (kind == kMaxUnpool) {
          SDK_CALL(sdk_mapped_max_unpool_plan_build, map.data_ptr(), buf, n, out_h, out_w, MH, MW,
                   K, (int32_t)P, (int32_t)interp, dt, stream);
          int32_t bands = 0;
          SDK_CALL(sdk_mapped_max_unpool_plan_bands, buf, n, out_h, out_w, dt, stream, &bands);
          return (int)bands;
        }
        SDK_CALL(sdk_resample_to_map_plan_build, map.data_ptr(), cptr(wts), buf, n, MH, MW, out_h,
                 out_w, K, (int32_t)P, (int32_t)interp, dt, stream);
        int32_t flag = 0;
        SDK_CALL(sdk_resample_plan_complete, buf, n, stream, &flag);
        return (int)flag;
      });
}

// ----------------------------------------------------------------------------- resample
Tensor resample_from_map(const Tensor& x, const Tensor& map, const OptTensor& wts, int64_t interp) {
  check_first(x);
  check_one(x, "x", x);
  check_one(x, "sample_map", map);
  check_opt(x, "interp_weights", wts);
  const int64_t P = npts(map, wts, 3);
  TORCH_CHECK(x.dim() == 4, "x must be [B, C, H, W]");
  const int64_t B = x.size(0), C = x.size(1), H = x.size(2), W = x.size(3);
  const int64_t MH = map.size(0), MW = map.size(1);
  Tensor out = at::empty({B, C, MH, MW}, x.options());
  c10::DeviceGuard guard(x.device());
  SDK_CALL(sdk_resample_from_map, x.data_ptr(), map.data_ptr(), cptr(wts), out.data_ptr(), B, C, H,
           W, MH, MW, (int32_t)P, (int32_t)interp, dtype_code(x), stream_of(x));
  return out;
}

std::tuple<Tensor, Tensor> resample_to_map_impl(const Tensor& x, const Tensor& map,
                                                const OptTensor& wts, int64_t out_h,
                                                int64_t out_w, int64_t interp, bool normalize,
                                                double eps) {
  check_first(x);
  check_one(x, "x", x);
  check_one(x, "sample_map", map);
  check_opt(x, "interp_weights", wts);
  const int64_t P = npts(map, wts, 3);
  TORCH_CHECK(x.dim() == 4, "x must be [B, C, MH, MW]");
  const int64_t B = x.size(0), C = x.size(1), MH = x.size(2), MW = x.size(3);
  TORCH_CHECK(map.size(0) == MH && map.size(1) == MW, "sample_map grid ",
              map.sizes().slice(0, 2), " must match the input's ", x.sizes().slice(2));
  const int dt = dtype_code(x);
  Tensor out = at::empty({B, C, out_h, out_w}, x.options());
  Tensor wsum;
  if (normalize) wsum = at::empty({out_h, out_w}, x.options());
  c10::DeviceGuard guard(x.device());
  hipStream_t s = stream_of(x);
  PlanRef plan = scatter_plan(kResample, x, map, wts, out_h, out_w, 1, P, interp, s);
  if (plan.plan.defined()) {
    SDK_CALL(sdk_resample_to_map_planned, x.data_ptr(), map.data_ptr(), cptr(wts), out.data_ptr(),
             normalize ? wsum.data_ptr() : nullptr, plan.ptr(), plan.nbytes, plan.complete,
             normalize ? 1 : 0, eps, B, C, MH, MW, out_h, out_w, (int32_t)P, (int32_t)interp, dt, s);
    return {out, wsum};
  }
  const size_t nws = sdk_resample_to_map_workspace_bytes(out_h, out_w, dt);
  Tensor ws;
  if (nws) ws = bytes_on(x, nws);
  if (normalize)
    SDK_CALL(sdk_resample_to_map_normalized, x.data_ptr(), map.data_ptr(), cptr(wts),
             out.data_ptr(), wsum.data_ptr(), nws ? ws.data_ptr() : nullptr, nws, eps, B, C, MH, MW,
             out_h, out_w, (int32_t)P, (int32_t)interp, dt, s);
  else
    SDK_CALL(sdk_resample_to_map, x.data_ptr(), map.data_ptr(), cptr(wts), out.data_ptr(), nullptr,
             nws ? ws.data_ptr() : nullptr, nws, B, C, MH, MW, out_h, out_w, (int32_t)P,
             (int32_t)interp, dt, s);
  return {out, wsum};
}

Tensor resample_to_map(const Tensor& x, const Tensor& map, const OptTensor& wts, int64_t out_h,
                       int64_t out_w, int64_t interp) {
  return std::get<0>(resample_to_map_impl(x, map, wts, out_h, out_w, interp, false, 0.0));
}
std::tuple<Tensor, Tensor> resample_to_map_normalized(const Tensor& x, const Tensor& map,
                                                      const OptTensor& wts, int64_t out_h,
                                                      int64_t out_w, int64_t interp, double eps) {
  return resample_to_map_impl(x, map, wts, out_h, out_w, interp, true, eps);
}

// ----------------------------------------------------------------------------- pooling
void check_kernel(const Tensor& map, int64_t kernel_size) {
  TORCH_CHECK(map.dim() >= 3 && map.size(2) == kernel_size, "kernel_size ", kernel_size,
              " does not match sample_map ", map.sizes());
}

std::tuple<Tensor, Tensor> mapped_max_pool(const Tensor& x, const Tensor& map, const OptTensor& wts,
                                           int64_t kernel_size, int64_t interp) {
  check_first(x);
  check_one(x, "x", x);
  check_one(x, "sample_map", map);
  check_opt(x, "interp_weights", wts);
  const int64_t P = npts(map, wts, 4);
  TORCH_CHECK(x.dim() == 4, "x must be [B, C, H, W]");
  check_kernel(map, kernel_size);
  const int64_t B = x.size(0), C = x.size(1), H = x.size(2), W = x.size(3);
  const int64_t OH = map.size(0), OW = map.size(1);
  Tensor out = at::empty({B, C, OH, OW}, x.options());
  Tensor idx = at::empty({B, C, OH, OW}, x.options().dtype(at::kLong));
  c10::DeviceGuard guard(x.device());
  SDK_CALL(sdk_mapped_max_pool, x.data_ptr(), map.data_ptr(), cptr(wts), out.data_ptr(),
           idx.data_ptr<int64_t>(), B, C, H, W, OH, OW, kernel_size, (int32_t)P, (int32_t)interp,
           dtype_code(x), stream_of(x));
  return {out, idx};
}

Tensor mapped_avg_pool(const Tensor& x, const Tensor& map, const OptTensor& wts,
                       int64_t kernel_size, int64_t interp) {
  check_first(x);
  check_one(x, "x", x);
  check_one(x, "sample_map", map);
  check_opt(x, "interp_weights", wts);
  const int64_t P = npts(map, wts, 4);
  TORCH_CHECK(x.dim() == 4, "x must be [B, C, H, W]");
  check_kernel(map, kernel_size);
  const int64_t B = x.size(0), C = x.size(1), H = x.size(2), W = x.size(3);
  const int64_t OH = map.size(0), OW = map.size(1);
  Tensor out = at::empty({B, C, OH, OW}, x.options());
  c10::DeviceGuard guard(x.device());
  SDK_CALL(sdk_mapped_avg_pool, x.data_ptr(), map.data_ptr(), cptr(wts), out.data_ptr(), B, C, H, W,
           OH, OW, kernel_size, (int32_t)P, (int32_t)interp, dtype_code(x), stream_of(x));
  return out;
}

Tensor mapped_max_unpool(const Tensor& g, const Tensor& idx, const Tensor& map,
                         const OptTensor& wts, int64_t in_h, int64_t in_w, int64_t kernel_size,
                         int64_t interp) {
  check_first(g);
  check_one(g, "grad_output", g);
  check_one(g, "idx_mask", idx, true);
  check_one(g, "sample_map", map);
  check_opt(g, "interp_weights", wts);
  TORCH_CHECK(idx.scalar_type() == at::kLong && idx.sizes() == g.sizes(),
              "idx_mask must be an int64 tensor shaped like grad_output");
  const int64_t P = npts(map, wts, 4);
  TORCH_CHECK(g.dim() == 4, "grad_output must be [B, C, OH, OW]");
  const int64_t B = g.size(0), C = g.size(1), OH = g.size(2), OW = g.size(3);
  TORCH_CHECK(map.size(0) == OH && map.size(1) == OW && map.size(2) == kernel_size, "sample_map ",
              map.sizes(), " does not match grad_output ", g.sizes(), " / kernel_size ",
              kernel_size);
  const int dt = dtype_code(g);
  Tensor gin = at::empty({B, C, in_h, in_w}, g.options());
  c10::DeviceGuard guard(g.device());
  hipStream_t s = stream_of(g);
  if (g_unpool_workspace) {
    PlanRef plan = scatter_plan(kMaxUnpool, g, map, wts, in_h, in_w, kernel_size, P, interp, s);
    if (plan.plan.defined() && plan.complete) {
      SDK_CALL(sdk_mapped_max_unpool_planned_bands, g.data_ptr(), idx.data_ptr<int64_t>(),
               map.data_ptr(), gin.data_ptr(), plan.ptr(), plan.nbytes, B, C, in_h, in_w, OH, OW,
               kernel_size, (int32_t)interp, dt, s);
      return gin;
    }
    if (plan.plan.defined()) {
      SDK_CALL(sdk_mapped_max_unpool_planned, g.data_ptr(), idx.data_ptr<int64_t>(), map.data_ptr(),
               cptr(wts), gin.data_ptr(), plan.ptr(), plan.nbytes, B, C, in_h, in_w, OH, OW,
               kernel_size, (int32_t)P, (int32_t)interp, dt, s);
      return gin;
    }
  }
  const size_t nws = g_unpool_workspace ? sdk_mapped_max_unpool_workspace_bytes(in_h, in_w, dt) : 0;
  Tensor ws;
  if (nws) ws = bytes_on(g, nws);
  SDK_CALL(sdk_mapped_max_unpool, g.data_ptr(), idx.data_ptr<int64_t>(), map.data_ptr(), cptr(wts),
           gin.data_ptr(), nws ? ws.data_ptr() : nullptr, nws, B, C, in_h, in_w, OH, OW,
           kernel_size, (int32_t)P, (int32_t)interp, dt, s);
  return gin;
}

Tensor mapped_avg_unpool(const Tensor& g, const Tensor& map, const OptTensor& wts, int64_t in_h,
                         int64_t in_w, int64_t kernel_size, int64_t interp) {
  check_first(g);
  check_one(g, "grad_output", g);
  check_one(g, "sample_map", map);
  check_opt(g, "interp_weights", wts);
  const int64_t P = npts(map, wts, 4);
  TORCH_CHECK(g.dim() == 4, "grad_output must be [B, C, OH, OW]");
  const int64_t B = g.size(0), C = g.size(1), OH = g.size(2), OW = g.size(3);
  TORCH_CHECK(map.size(0) == OH && map.size(1) == OW && map.size(2) == kernel_size, "sample_map ",
              map.sizes(), " does not match grad_output ", g.sizes(), " / kernel_size ",
              kernel_size);
  const int dt = dtype_code(g);
  Tensor gin = at::empty({B, C, in_h, in_w}, g.options());
  c10::DeviceGuard guard(g.device());
  hipStream_t s = stream_of(g);
  PlanRef plan = scatter_plan(kAvgUnpool, g, map, wts, in_h, in_w, kernel_size, P, interp, s);
  if (plan.plan.defined()) {
    SDK_CALL(sdk_mapped_avg_unpool_planned, g.data_ptr(), map.data_ptr(), cptr(wts), gin.data_ptr(),
             plan.ptr(), plan.nbytes, plan.complete, B, C, in_h, in_w, OH, OW, kernel_size,
             (int32_t)P, (int32_t)interp, dt, s);
    return gin;
  }
  const size_t nws = sdk_resample_to_map_workspace_bytes(in_h, in_w, dt);
  Tensor ws;
  if (nws) ws = bytes_on(g, nws);
  SDK_CALL(sdk_mapped_avg_unpool, g.data_ptr(), map.data_ptr(), cptr(wts), gin.data_ptr(),
           nws ? ws.data_ptr() : nullptr, nws, B, C, in_h, in_w, OH, OW, kernel_size, (int32_t)P,
           (int32_t)interp, dt, s);
  return gin;
}

// ----------------------------------------------------------------------------- convolution
struct ConvDims {
  int64_t B, Cin, Cout, K;
};
ConvDims conv_dims(const Tensor& x, const Tensor& weight, const Tensor& map, int64_t kernel_size,
                   bool transposed) {
  TORCH_CHECK(x.dim() == 4 && weight.dim() == 3 && map.dim() >= 4, "bad tensor ranks");
  TORCH_CHECK(map.size(2) == kernel_size && weight.size(2) == kernel_size, "kernel_size ",
              kernel_size, " does not match sample_map ", map.sizes(), " / weight ",
              weight.sizes());
  ConvDims d;
  d.B = x.size(0);
  d.Cin = x.size(1);
  d.K = kernel_size;
  TORCH_CHECK(weight.size(transposed ? 0 : 1) == d.Cin, "weight ", weight.sizes(),
              " does not match ", d.Cin, " input channels");
  d.Cout = weight.size(transposed ? 1 : 0);
  return d;
}

Tensor workspace(const Tensor& ref, const ConvDims& d, int64_t img_h, int64_t img_w, int64_t map_h,
                 int64_t map_w, int64_t P, int64_t interp, size_t* n) {
  *n = sdk_mapped_conv_workspace_bytes(d.B, d.Cin, d.Cout, img_h, img_w, map_h, map_w, d.K,
                                       (int32_t)P, (int32_t)interp, dtype_code(ref), current_mode());
  return *n ? bytes_on(ref, *n) : Tensor();
}

Tensor mapped_conv_forward(const Tensor& x, const Tensor& map, const OptTensor& wts,
                           const Tensor& weight, const Tensor& bias, int64_t kernel_size,
                           int64_t interp) {
  check_first(x);
  check_one(x, "input", x);
  check_one(x, "sample_map", map);
  check_opt(x, "interp_weights", wts);
  check_one(x, "weight", weight);
  check_one(x, "bias", bias);
  const int64_t P = npts(map, wts, 4);
  const ConvDims d = conv_dims(x, weight, map, kernel_size, false);
  const int64_t H = x.size(2), W = x.size(3), OH = map.size(0), OW = map.size(1);
  Tensor out = at::empty({d.B, d.Cout, OH, OW}, x.options());
  c10::DeviceGuard guard(x.device());
  hipStream_t s = stream_of(x);
  size_t nws = 0;
  Tensor ws = workspace(x, d, H, W, OH, OW, P, interp, &nws);
  PlanRef plan = conv_plan(x, map, wts, H, W, d.K, P, interp, s);
  const int dt = dtype_code(x), mode = current_mode();
  void* wsp = nws ? ws.data_ptr() : nullptr;
  if (!plan.plan.defined())
    SDK_CALL(sdk_mapped_conv_forward, x.data_ptr(), map.data_ptr(), cptr(wts), weight.data_ptr(),
             bias.data_ptr(), out.data_ptr(), wsp, nws, d.B, d.Cin, H, W, d.Cout, OH, OW, d.K,
             (int32_t)P, (int32_t)interp, dt, mode, s);
  else
    SDK_CALL(sdk_mapped_conv_forward_planned, x.data_ptr(), map.data_ptr(), cptr(wts),
             weight.data_ptr(), bias.data_ptr(), out.data_ptr(), wsp, nws, plan.ptr(), plan.nbytes,
             d.B, d.Cin, H, W, d.Cout, OH, OW, d.K, (int32_t)P, (int32_t)interp, dt, mode, s);
  return out;
}

std::tuple<Tensor, Tensor, Tensor> mapped_conv_backward(const Tensor& grad_output,
                                                        const Tensor& map, const OptTensor& wts,
                                                        const Tensor& x, const Tensor& weight,
                                                        const Tensor& bias, int64_t kernel_size,
                                                        int64_t interp) {
  // The reference checks input, sample_map, weight and bias here, not grad_output
  // (include/layers/mapped_convolution_layer.h:93-96); the kernels need it dense too.
  const Tensor g = grad_output.contiguous();
  check_first(g);
  check_one(g, "grad_output", g);
  check_one(g, "input", x);
  check_one(g, "sample_map", map);
  check_opt(g, "interp_weights", wts);
  check_one(g, "weight", weight);
  check_one(g, "bias", bias);
  const int64_t P = npts(map, wts, 4);
  const ConvDims d = conv_dims(x, weight, map, kernel_size, false);
  const int64_t H = x.size(2), W = x.size(3), OH = map.size(0), OW = map.size(1);
  Tensor gi = at::empty_like(x), gw = at::empty_like(weight);
  Tensor gb = at::empty({d.Cout}, x.options());
  c10::DeviceGuard guard(x.device());
  hipStream_t s = stream_of(x);
  size_t nws = 0;
  Tensor ws = workspace(x, d, H, W, OH, OW, P, interp, &nws);
  PlanRef plan = conv_plan(x, map, wts, H, W, d.K, P, interp, s);
  const int dt = dtype_code(x), mode = current_mode();
  void* wsp = nws ? ws.data_ptr() : nullptr;
  if (!plan.plan.defined())
    SDK_CALL(sdk_mapped_conv_backward, g.data_ptr(), map.data_ptr(), cptr(wts), x.data_ptr(),
             weight.data_ptr(), gi.data_ptr(), gw.data_ptr(), gb.data_ptr(), wsp, nws, d.B, d.Cin,
             H, W, d.Cout, OH, OW, d.K, (int32_t)P, (int32_t)interp, dt, mode, s);
  else
    SDK_CALL(sdk_mapped_conv_backward_planned, g.data_ptr(), map.data_ptr(), cptr(wts),
             x.data_ptr(), weight.data_ptr(), gi.data_ptr(), gw.data_ptr(), gb.data_ptr(), wsp, nws,
             plan.ptr(), plan.nbytes, d.B, d.Cin, H, W, d.Cout, OH, OW, d.K, (int32_t)P,
             (int32_t)interp, dt, mode, s);
  return {gi, gw, gb};
}

Tensor mapped_transposed_conv_forward(const Tensor& x, const Tensor& map, const OptTensor& wts,
                                      const Tensor& weight, const Tensor& bias, int64_t out_h,
                                      int64_t out_w, int64_t kernel_size, int64_t interp) {
  check_first(x);
  check_one(x, "input", x);
  check_one(x, "sample_map", map);
  check_opt(x, "interp_weights", wts);
  check_one(x, "weight", weight);
  check_one(x, "bias", bias);
  const int64_t P = npts(map, wts, 4);
  const ConvDims d = conv_dims(x, weight, map, kernel_size, true);
  const int64_t IH = x.size(2), IW = x.size(3);
  TORCH_CHECK(map.size(0) == IH && map.size(1) == IW, "sample_map grid ", map.sizes().slice(0, 2),
              " must match the input's ", x.sizes().slice(2));
  Tensor out = at::empty({d.B, d.Cout, out_h, out_w}, x.options());
  c10::DeviceGuard guard(x.device());
  hipStream_t s = stream_of(x);
  size_t nws = 0;
  Tensor ws = workspace(x, d, out_h, out_w, IH, IW, P, interp, &nws);
  PlanRef plan = conv_plan(x, map, wts, out_h, out_w, d.K, P, interp, s);
  const int dt = dtype_code(x), mode = current_mode();
  void* wsp = nws ? ws.data_ptr() : nullptr;
  if (!plan.plan.defined())
    SDK_CALL(sdk_mapped_transposed_conv_forward, x.data_ptr(), map.data_ptr(), cptr(wts),
             weight.data_ptr(), bias.data_ptr(), out.data_ptr(), wsp, nws, d.B, d.Cin, IH, IW,
             d.Cout, out_h, out_w, d.K, (int32_t)P, (int32_t)interp, dt, mode, s);
  else
    SDK_CALL(sdk_mapped_transposed_conv_forward_planned, x.data_ptr(), map.data_ptr(), cptr(wts),
             weight.data_ptr(), bias.data_ptr(), out.data_ptr(), wsp, nws, plan.ptr(), plan.nbytes,
             d.B, d.Cin, IH, IW, d.Cout, out_h, out_w, d.K, (int32_t)P, (int32_t)interp, dt, mode,
             s);
  return out;
}

std::tuple<Tensor, Tensor, Tensor> mapped_transposed_conv_backward(
    const Tensor& grad_output, const Tensor& map, const OptTensor& wts, const Tensor& x,
    const Tensor& weight, const Tensor& bias, int64_t kernel_size, int64_t interp) {
  const Tensor g = grad_output.contiguous();
  check_first(g);
  check_one(g, "grad_output", g);
  check_one(g, "input", x);
  check_one(g, "sample_map", map);
  check_opt(g, "interp_weights", wts);
  check_one(g, "weight", weight);
  check_one(g, "bias", bias);
  const int64_t P = npts(map, wts, 4);
  const ConvDims d = conv_dims(x, weight, map, kernel_size, true);
  TORCH_CHECK(g.dim() == 4, "grad_output must be [B, C, OH, OW]");
  const int64_t IH = x.size(2), IW = x.size(3), OH = g.size(2), OW = g.size(3);
  Tensor gi = at::empty_like(x), gw = at::empty_like(weight);
  Tensor gb = at::empty({d.Cout}, x.options());
  c10::DeviceGuard guard(x.device());
  hipStream_t s = stream_of(x);
  size_t nws = 0;
  Tensor ws = workspace(x, d, OH, OW, IH, IW, P, interp, &nws);
  PlanRef plan = conv_plan(x, map, wts, OH, OW, d.K, P, interp, s);
  const int dt = dtype_code(x), mode = current_mode();
  void* wsp = nws ? ws.data_ptr() : nullptr;
  if (!plan.plan.defined())
    SDK_CALL(sdk_mapped_transposed_conv_backward, g.data_ptr(), map.data_ptr(), cptr(wts),
             x.data_ptr(), weight.data_ptr(), gi.data_ptr(), gw.data_ptr(), gb.data_ptr(), wsp, nws,
             d.B, d.Cin, IH, IW, d.Cout, OH, OW, d.K, (int32_t)P, (int32_t)interp, dt, mode, s);
  else
    SDK_CALL(sdk_mapped_transposed_conv_backward_planned, g.data_ptr(), map.data_ptr(), cptr(wts),
             x.data_ptr(), weight.data_ptr(), gi.data_ptr(), gw.data_ptr(), gb.data_ptr(), wsp, nws,
             plan.ptr(), plan.nbytes, d.B, d.Cin, IH, IW, d.Cout, OH, OW, d.K, (int32_t)P,
             (int32_t)interp, dt, mode, s);
  return {gi, gw, gb};
}

}  // namespace

TORCH_LIBRARY_IMPL(sdk_mapped_ops, CUDA, m) {
  m.impl("resample_from_map", &resample_from_map);
  m.impl("resample_to_map", &resample_to_map);
  m.impl("resample_to_map_normalized", &resample_to_map_normalized);
  m.impl("mapped_max_pool", &mapped_max_pool);
  m.impl("mapped_max_unpool", &mapped_max_unpool);
  m.impl("mapped_avg_pool", &mapped_avg_pool);
  m.impl("mapped_avg_unpool", &mapped_avg_unpool);
  m.impl("mapped_conv_forward", &mapped_conv_forward);
  m.impl("mapped_conv_backward", &mapped_conv_backward);
  m.impl("mapped_transposed_conv_forward", &mapped_transposed_conv_forward);
  m.impl("mapped_transposed_conv_backward", &mapped_transposed_conv_backward);
}

// Controls, called from Python (ctypes): the compute mode (process default and per-thread
// override), the plan cache and the unpool workspace switch.
extern "C" {
const char* sdk_torch_native_ops(void) {
  return "resample_from_map,resample_to_map,resample_to_map_normalized,mapped_max_pool,"
         "mapped_max_unpool,mapped_avg_pool,mapped_avg_unpool,mapped_conv_forward,"
         "mapped_conv_backward,mapped_transposed_conv_forward,mapped_transposed_conv_backward";
}
void sdk_torch_set_default_mode(int mode) { g_default_mode = mode; }
// mode < 0 removes the override; returns the previous override (-1: none)
int sdk_torch_set_thread_mode(int mode) {
  const int prev = t_mode;
  t_mode = mode;
  return prev;
}
int sdk_torch_current_mode(void) { return current_mode(); }
void sdk_torch_set_plan_cache(int enabled, int max_entries) {
  std::lock_guard<std::mutex> lock(g_mu);
  g_cache_enabled = enabled != 0;
  if (max_entries > 0) g_cache_max = (size_t)max_entries;
  if (!g_cache_enabled) g_cache.clear();
  while (g_cache.size() > g_cache_max) g_cache.pop_front();
}
int sdk_torch_plan_cache_size(void) {
  std::lock_guard<std::mutex> lock(g_mu);
  return (int)g_cache.size();
}
void sdk_torch_set_unpool_workspace(int enabled) { g_unpool_workspace = enabled != 0; }
}
