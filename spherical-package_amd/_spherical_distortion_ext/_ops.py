"""PyTorch-ROCm custom operators over the C ABI.

Every operator here checks its tensors the way the reference's pybind entry
points do (contiguous, all on the GPU: ext_modules/include/cuda_helper.h:12-18),
allocates the outputs with torch, fetches the current HIP stream and makes one
call into libsdk_mapped_ops.so.  The operators are registered in the
``sdk_mapped_ops`` namespace of torch.library for the CUDA (= HIP on ROCm)
dispatch key only: calling them with CPU tensors raises, there is no CPU path.

The schemas are defined here.  Where libsdk_torch_ops.so is built (csrc/torch_ops.cpp, the
same checks, allocation, stream fetch and plan cache in C++), it is loaded and implements the
operators it names; the functions below implement the others, and all of them when that
library is absent or the environment says SDK_TORCH_OPS=python.  The compute mode, the plan
cache switches and the unpool workspace switch set here reach both.
"""
import contextlib
import ctypes
import os
import threading

import torch

from . import _capi

_NS = "sdk_mapped_ops"
_DTYPES = {torch.float32: _capi.SDK_F32, torch.float64: _capi.SDK_F64}

# Arithmetic of the dense contraction inside the convolution operators: "native"
# (the tensors' type), "bf16" (bf16 operands, fp32 accumulate), "split" (fp32 operands as
# three bf16 pieces each: fp32 accuracy from the bf16 matrix unit) or "unfused"
# (separate im2col/col2im + GEMM kernels, the cross-check path).
_MODES = {"native": _capi.SDK_COMPUTE_NATIVE, "fp32": _capi.SDK_COMPUTE_NATIVE,
          "bf16": _capi.SDK_COMPUTE_BF16, "unfused": _capi.SDK_COMPUTE_UNFUSED,
          "split": _capi.SDK_COMPUTE_SPLIT}
_default_mode = _capi.SDK_COMPUTE_NATIVE   # process-wide default
_tls = threading.local()                   # per-thread override (conv_compute)


def _mode_value(mode):
    if mode not in _MODES:
        raise ValueError("compute mode must be one of %s" % sorted(_MODES))
    return _MODES[mode]


# libsdk_torch_ops.so as a ctypes handle (its control functions) once it is loaded, else None
_native = None
_NATIVE_OPS = frozenset()


def set_conv_compute(mode):
    """Sets the process-wide default arithmetic of the mapped (transposed) convolutions:
    "native" (fp32 MFMA), "split" (fp32 operands as three bf16 pieces), "bf16" (operands
    rounded to bf16), "unfused" (im2col + GEMM kernels)."""
    global _default_mode
    _default_mode = _mode_value(mode)
    if _native is not None:
        _native.sdk_torch_set_default_mode(_default_mode)


def _current_mode():
    # SDK_COMPUTE_NATIVE is 0: an override is "set" when it is not None, whatever its value
    mode = getattr(_tls, "mode", None)
    return _default_mode if mode is None else mode


def get_conv_compute():
    """The mode a convolution called now on this thread would use."""
    return {_capi.SDK_COMPUTE_BF16: "bf16", _capi.SDK_COMPUTE_UNFUSED: "unfused",
            _capi.SDK_COMPUTE_SPLIT: "split"}.get(_current_mode(), "native")


@contextlib.contextmanager
def conv_compute(mode):
    """Overrides the compute mode for the calls made inside the block on this thread; None
    leaves the default in force.  The autograd functions run their backward under the mode
    their forward saw, and the nn modules take a `compute` argument that ends up here."""
    if mode is None:
        yield
        return
    value = _mode_value(mode)
    previous = getattr(_tls, "mode", None)
    _tls.mode = value
    if _native is not None:
        _native.sdk_torch_set_thread_mode(value)
    try:
        yield
    finally:
        _tls.mode = previous
        if _native is not None:
            _native.sdk_torch_set_thread_mode(-1 if previous is None else previous)


def _check(ref, **tensors):
    """ref: the tensor that decides device and dtype (first argument of the op)."""
    if not ref.is_cuda:
        raise RuntimeError("this backend runs on the GPU only: tensors must be CUDA/HIP tensors")
    if ref.dtype not in _DTYPES:
        raise RuntimeError("unsupported dtype %s (float32 and float64 only)" % ref.dtype)
    for name, t in tensors.items():
        if t is None:
            continue
        if not t.is_contiguous():
            raise RuntimeError("%s must be contiguous" % name)
        if not t.is_cuda or t.device != ref.device:
            raise RuntimeError("%s must be a CUDA tensor on %s" % (name, ref.device))
        if t.dtype != ref.dtype and name not in ("idx_mask", "quad_idx"):
            raise RuntimeError("%s must have dtype %s (got %s)" % (name, ref.dtype, t.dtype))


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(ref):
    return ctypes.c_void_p(torch.cuda.current_stream(ref.device).cuda_stream)


def _npts(sample_map, interp_weights, map_rank_unweighted):
    """0 for the unweighted map layout, P for the weighted one."""
    if interp_weights is None:
        if sample_map.dim() != map_rank_unweighted or sample_map.shape[-1] != 2:
            raise RuntimeError("sample_map must have %d dimensions ending in 2, got %s"
                               % (map_rank_unweighted, tuple(sample_map.shape)))
        return 0
    if sample_map.dim() != map_rank_unweighted + 1 or sample_map.shape[-1] != 2:
        raise RuntimeError("weighted sample_map must have %d dimensions ending in 2, got %s"
                           % (map_rank_unweighted + 1, tuple(sample_map.shape)))
    if tuple(interp_weights.shape) != tuple(sample_map.shape[:-1]):
        raise RuntimeError("interp_weights shape %s does not match sample_map %s"
                           % (tuple(interp_weights.shape), tuple(sample_map.shape)))
    return int(interp_weights.shape[-1])


def _workspace(ref, batch, cin, cout, img_h, img_w, map_h, map_w, K, P, interp):
    n = _capi.load().sdk_mapped_conv_workspace_bytes(
        batch, cin, cout, img_h, img_w, map_h, map_w, K, P, interp, _DTYPES[ref.dtype],
        _current_mode())
    if n == 0:
        return None, 0
    return torch.empty(n, dtype=torch.uint8, device=ref.device), n


# --------------------------------------------------------------------------- conv plans
# What the convolution kernels derive from a sample map alone (include/sdk_mapped_ops.h, "Plans")
# is built once per map and reused by every later call on it.  An entry is keyed on the map's
# (and the point weights') storage address, offset, version counter, shape and the geometry, and
# holds the storages, so an address cannot be handed to another tensor while its entry lives;
# in-place changes of a map bump its version and miss.
#
# The cache evicts the least recently used entry beyond `_PLAN_CACHE_MAX` (a hit moves its
# entry to the end).  Three kinds of call go past it, to the entry points that build what they
# need in the call's own workspace: a map without a version counter (a tensor created under
# torch.inference_mode(): an in-place change of it could not be seen), a key that misses while
# the current stream is being captured into a graph (the build would only be recorded, the
# entry would look built to an eager call before the first replay, and its buffer would belong
# to the graph's private pool), and everything when the cache is switched off.
_PLAN_CACHE = {}
_PLAN_CACHE_MAX = 16
_plan_cache_enabled = True
_NO_KEY = object()   # _tensor_key of a tensor whose changes cannot be tracked


class _PlanEntry:
    """A kept plan: the buffer, its size, the storages of the map it was built from, the
    stream that used it last (every call reads the plan, and the max-unpool call rewrites the
    plan's gate word, so a call on another stream is ordered behind the last user) and the
    `complete` verdict of a scatter plan."""
    __slots__ = ("plan", "nbytes", "keep", "stream", "complete")

    def __init__(self, plan, nbytes, keep, stream, complete=0):
        self.plan, self.nbytes, self.keep, self.stream, self.complete = \
            plan, nbytes, keep, stream, complete


def set_conv_plan_cache(enabled, max_entries=None):
    """Keeps (default) or rebuilds per call what the operators derive from a map alone: the
    plans of the mapped (transposed) convolutions, the inverted maps of resample_to_map and
    average unpooling, the tile windows of max unpooling.  max_entries: how many plans are
    kept (least recently used dropped first; default 16, one per (map, geometry) in use)."""
    global _plan_cache_enabled, _PLAN_CACHE_MAX
    _plan_cache_enabled = bool(enabled)
    if max_entries is not None:
        if int(max_entries) < 1:
            raise ValueError("max_entries must be at least 1")
        _PLAN_CACHE_MAX = int(max_entries)
    if not enabled:
        _PLAN_CACHE.clear()
    while len(_PLAN_CACHE) > _PLAN_CACHE_MAX:
        _PLAN_CACHE.pop(next(iter(_PLAN_CACHE)))
    if _native is not None:
        _native.sdk_torch_set_plan_cache(1 if enabled else 0, _PLAN_CACHE_MAX)


def plan_cache_size():
    """Plans kept at the moment, by the compiled operator layer and by this module."""
    n = len(_PLAN_CACHE)
    if _native is not None:
        n += int(_native.sdk_torch_plan_cache_size())
    return n


def _tensor_key(t):
    if t is None:
        return None
    if t.is_inference():
        return _NO_KEY
    return (t.untyped_storage().data_ptr(), t.storage_offset(), t._version, tuple(t.shape))


def _cache_lookup(key, cur):
    """The entry of `key`, made the most recently used one and ordered behind its last user
    on another stream; None on a miss."""
    ent = _PLAN_CACHE.pop(key, None)
    if ent is None:
        return None
    _PLAN_CACHE[key] = ent
    if ent.stream != cur:
        cur.wait_stream(ent.stream)
        ent.stream = cur
    return ent


def _cache_insert(key, ent):
    while len(_PLAN_CACHE) >= _PLAN_CACHE_MAX:
        _PLAN_CACHE.pop(next(iter(_PLAN_CACHE)))
    _PLAN_CACHE[key] = ent


def _uncacheable(*keys):
    return any(k is _NO_KEY for k in keys)


def _conv_plan(ref, sample_map, interp_weights, img_h, img_w, K, P, interp):
    """(plan tensor, bytes) for this map and geometry, built on first use; (None, 0) when the
    library has no plan for it or the cache is off."""
    if not _plan_cache_enabled or ref.dtype != torch.float32:
        return None, 0
    MH, MW = int(sample_map.shape[0]), int(sample_map.shape[1])
    km, kw = _tensor_key(sample_map), _tensor_key(interp_weights)
    if _uncacheable(km, kw):
        return None, 0
    key = (ref.device, km, kw, int(img_h), int(img_w), int(K), int(P), int(interp))
    cur = torch.cuda.current_stream(ref.device)
    ent = _cache_lookup(key, cur)
    if ent is not None:
        return ent.plan, ent.nbytes
    if torch.cuda.is_current_stream_capturing():
        return None, 0
    n = _capi.load().sdk_mapped_conv_plan_bytes(int(img_h), int(img_w), MH, MW, int(K), int(P),
                                                int(interp), _capi.SDK_F32)
    if n == 0:
        return None, 0
    plan = torch.empty(n, dtype=torch.uint8, device=ref.device)
    _capi.call("sdk_mapped_conv_plan_build", _ptr(sample_map), _ptr(interp_weights), _ptr(plan), n,
               int(img_h), int(img_w), MH, MW, int(K), int(P), int(interp), _capi.SDK_F32,
               _stream(ref))
    keep = (sample_map.untyped_storage(),
            None if interp_weights is None else interp_weights.untyped_storage())
    _cache_insert(key, _PlanEntry(plan, n, keep, cur))
    return plan, n


def _scatter_plan(kind, ref, sample_map, interp_weights, out_h, out_w, K, P, interp):
    """(plan tensor, bytes, complete) of a scatter-direction operator for this map, built on
    first use and kept like the convolution plans; (None, 0, 0) when the cache is off.

    kind "resample" / "avg_unpool": the inverted map (sdk_resample_to_map_plan_build; K = 1 for
    a resampling map), complete = 1 when every target's list holds all its sources, checked
    once after the build (not under stream capture, where the check's synchronisation is not
    allowed).  kind "max_unpool": the tile windows (sdk_mapped_max_unpool_plan_build), complete = 1
    when the row-band kernel does every call on the plan (sdk_mapped_max_unpool_plan_bands)."""
    if not _plan_cache_enabled:
        return None, 0, 0
    dt = _DTYPES[ref.dtype]
    km, kw = _tensor_key(sample_map), _tensor_key(interp_weights)
    if _uncacheable(km, kw):
        return None, 0, 0
    key = (kind, ref.device, dt, km, kw, int(out_h), int(out_w), int(K), int(P), int(interp))
    cur = torch.cuda.current_stream(ref.device)
    ent = _cache_lookup(key, cur)
    if ent is not None:
        return ent.plan, ent.nbytes, ent.complete
    if torch.cuda.is_current_stream_capturing():
        return None, 0, 0
    lib = _capi.load()
    query = ("sdk_mapped_max_unpool_workspace_bytes" if kind == "max_unpool"
             else "sdk_resample_to_map_workspace_bytes")
    n = getattr(lib, query)(int(out_h), int(out_w), dt)
    if n == 0:
        return None, 0, 0
    plan = torch.empty(n, dtype=torch.uint8, device=ref.device)
    MH, MW = int(sample_map.shape[0]), int(sample_map.shape[1])
    complete = 0
    if kind == "max_unpool":
        _capi.call("sdk_mapped_max_unpool_plan_build", _ptr(sample_map), _ptr(plan), n, int(out_h),
                   int(out_w), MH, MW, int(K), int(P), int(interp), dt, _stream(ref))
        flag = ctypes.c_int32(0)
        _capi.call("sdk_mapped_max_unpool_plan_bands", _ptr(plan), n, int(out_h), int(out_w), dt,
                   _stream(ref), ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
        complete = int(flag.value)
    else:
        _capi.call("sdk_resample_to_map_plan_build", _ptr(sample_map), _ptr(interp_weights),
                   _ptr(plan), n, MH, MW, int(out_h), int(out_w), int(K), int(P), int(interp), dt,
                   _stream(ref))
        flag = ctypes.c_int32(0)
        _capi.call("sdk_resample_plan_complete", _ptr(plan), n, _stream(ref),
                   ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
        complete = int(flag.value)
    keep = (sample_map.untyped_storage(),
            None if interp_weights is None else interp_weights.untyped_storage())
    _cache_insert(key, _PlanEntry(plan, n, keep, cur, complete))
    return plan, n, complete


def _scatter_workspace(ref, out_h, out_w, query="sdk_resample_to_map_workspace_bytes"):
    n = getattr(_capi.load(), query)(int(out_h), int(out_w), _DTYPES[ref.dtype])
    if n == 0:
        return None, 0
    return torch.empty(n, dtype=torch.uint8, device=ref.device), n


# --------------------------------------------------------------------------- resample
def resample_from_map(x, sample_map, interp_weights, interp):
    _check(x, x=x, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 3)
    B, C, H, W = x.shape
    MH, MW = sample_map.shape[:2]
    out = torch.empty((B, C, MH, MW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _capi.call("sdk_resample_from_map", _ptr(x), _ptr(sample_map), _ptr(interp_weights),
                   _ptr(out), B, C, H, W, MH, MW, P, int(interp), _DTYPES[x.dtype], _stream(x))
    return out


def resample_to_map(x, sample_map, interp_weights, out_h, out_w, interp):
    _check(x, x=x, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 3)
    B, C, MH, MW = x.shape
    if tuple(sample_map.shape[:2]) != (MH, MW):
        raise RuntimeError("sample_map grid %s must match the input's %s"
                           % (tuple(sample_map.shape[:2]), (MH, MW)))
    out = torch.empty((B, C, int(out_h), int(out_w)), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        plan, nplan, complete = _scatter_plan("resample", x, sample_map, interp_weights, out_h,
                                              out_w, 1, P, interp)
        if plan is not None:
            _capi.call("sdk_resample_to_map_planned", _ptr(x), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(out), ctypes.c_void_p(0), _ptr(plan), nplan,
                       complete, 0, 0.0, B, C, MH, MW, int(out_h), int(out_w), P, int(interp),
                       _DTYPES[x.dtype], _stream(x))
            return out
        ws, nws = _scatter_workspace(x, out_h, out_w)
        _capi.call("sdk_resample_to_map", _ptr(x), _ptr(sample_map), _ptr(interp_weights),
                   _ptr(out), ctypes.c_void_p(0), _ptr(ws), nws, B, C, MH, MW, int(out_h),
                   int(out_w), P, int(interp), _DTYPES[x.dtype], _stream(x))
    return out


def resample_to_map_normalized(x, sample_map, interp_weights, out_h, out_w, interp, eps):
    """resample_to_map(x) / (resample_to_map(ones) + eps) with one weight-sum plane."""
    _check(x, x=x, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 3)
    B, C, MH, MW = x.shape
    if tuple(sample_map.shape[:2]) != (MH, MW):
        raise RuntimeError("sample_map grid must match the input's")
    out = torch.empty((B, C, int(out_h), int(out_w)), dtype=x.dtype, device=x.device)
    wsum = torch.empty((int(out_h), int(out_w)), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        plan, nplan, complete = _scatter_plan("resample", x, sample_map, interp_weights, out_h,
                                              out_w, 1, P, interp)
        if plan is not None:
            _capi.call("sdk_resample_to_map_planned", _ptr(x), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(out), _ptr(wsum), _ptr(plan), nplan, complete,
                       1, float(eps), B, C, MH, MW, int(out_h), int(out_w), P, int(interp),
                       _DTYPES[x.dtype], _stream(x))
            return out, wsum
        ws, nws = _scatter_workspace(x, out_h, out_w)
        _capi.call("sdk_resample_to_map_normalized", _ptr(x), _ptr(sample_map),
                   _ptr(interp_weights), _ptr(out), _ptr(wsum), _ptr(ws), nws, float(eps), B, C,
                   MH, MW, int(out_h), int(out_w), P, int(interp), _DTYPES[x.dtype], _stream(x))
    return out, wsum


# --------------------------------------------------------------------------- im2col / col2im
def mapped_im2col(x, sample_map, interp_weights, interp):
    _check(x, x=x, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 4)
    B, C, H, W = x.shape
    OH, OW, K = sample_map.shape[:3]
    col = torch.empty((B, C * K, OH * OW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _capi.call("sdk_mapped_im2col", _ptr(x), _ptr(sample_map), _ptr(interp_weights),
                   _ptr(col), B, C, H, W, OH * OW, K, P, int(interp), _DTYPES[x.dtype],
                   _stream(x))
    return col


def mapped_col2im(col, sample_map, interp_weights, height, width, interp):
    _check(col, col=col, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 4)
    OH, OW, K = sample_map.shape[:3]
    B, CK, M = col.shape
    if M != OH * OW or CK % K:
        raise RuntimeError("columns %s do not match sample_map %s"
                           % (tuple(col.shape), tuple(sample_map.shape)))
    C = CK // K
    im = torch.empty((B, C, int(height), int(width)), dtype=col.dtype, device=col.device)
    with torch.cuda.device(col.device):
        _capi.call("sdk_mapped_col2im", _ptr(col), _ptr(sample_map), _ptr(interp_weights),
                   _ptr(im), B, C, int(height), int(width), M, K, P, int(interp),
                   _DTYPES[col.dtype], _stream(col))
    return im


# --------------------------------------------------------------------------- pooling
_UNPOOL_WORKSPACE = True


def set_unpool_workspace(enabled):
    """mapped_max_unpool with (default) or without the scratch buffer that lets the call run
    as a gather; without it the call is the zero fill + atomic scatter."""
    global _UNPOOL_WORKSPACE
    _UNPOOL_WORKSPACE = bool(enabled)
    if _native is not None:
        _native.sdk_torch_set_unpool_workspace(1 if enabled else 0)


def mapped_max_pool(x, sample_map, interp_weights, kernel_size, interp):
    _check(x, x=x, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 4)
    B, C, H, W = x.shape
    OH, OW, K = sample_map.shape[:3]
    if K != int(kernel_size):
        raise RuntimeError("kernel_size %d does not match sample_map %s"
                           % (int(kernel_size), tuple(sample_map.shape)))
    out = torch.empty((B, C, OH, OW), dtype=x.dtype, device=x.device)
    idx = torch.empty((B, C, OH, OW), dtype=torch.int64, device=x.device)
    with torch.cuda.device(x.device):
        _capi.call("sdk_mapped_max_pool", _ptr(x), _ptr(sample_map), _ptr(interp_weights),
                   _ptr(out), _ptr(idx), B, C, H, W, OH, OW, K, P, int(interp),
                   _DTYPES[x.dtype], _stream(x))
    return out, idx


def mapped_max_unpool(grad_output, idx_mask, sample_map, interp_weights, in_h, in_w,
                      kernel_size, interp):
    _check(grad_output, grad_output=grad_output, idx_mask=idx_mask, sample_map=sample_map,
           interp_weights=interp_weights)
    if idx_mask.dtype != torch.int64 or idx_mask.shape != grad_output.shape:
        raise RuntimeError("idx_mask must be an int64 tensor shaped like grad_output")
    P = _npts(sample_map, interp_weights, 4)
    B, C, OH, OW = grad_output.shape
    if tuple(sample_map.shape[:3]) != (OH, OW, int(kernel_size)):
        raise RuntimeError("sample_map %s does not match grad_output %s / kernel_size %d"
                           % (tuple(sample_map.shape), tuple(grad_output.shape), int(kernel_size)))
    gin = torch.empty((B, C, int(in_h), int(in_w)), dtype=grad_output.dtype,
                      device=grad_output.device)
    with torch.cuda.device(grad_output.device):
        if _UNPOOL_WORKSPACE:
            plan, nplan, bands = _scatter_plan("max_unpool", grad_output, sample_map,
                                               interp_weights, in_h, in_w, kernel_size, P, interp)
            if plan is not None and bands:
                _capi.call("sdk_mapped_max_unpool_planned_bands", _ptr(grad_output),
                           _ptr(idx_mask), _ptr(sample_map), _ptr(gin), _ptr(plan), nplan, B, C,
                           int(in_h), int(in_w), OH, OW, int(kernel_size), int(interp),
                           _DTYPES[grad_output.dtype], _stream(grad_output))
                return gin
            if plan is not None:
                _capi.call("sdk_mapped_max_unpool_planned", _ptr(grad_output), _ptr(idx_mask),
                           _ptr(sample_map), _ptr(interp_weights), _ptr(gin), _ptr(plan), nplan,
                           B, C, int(in_h), int(in_w), OH, OW, int(kernel_size), P, int(interp),
                           _DTYPES[grad_output.dtype], _stream(grad_output))
                return gin
        ws, nws = _scatter_workspace(grad_output, in_h, in_w,
                                     "sdk_mapped_max_unpool_workspace_bytes")
        if not _UNPOOL_WORKSPACE:
            ws, nws = None, 0
        _capi.call("sdk_mapped_max_unpool", _ptr(grad_output), _ptr(idx_mask), _ptr(sample_map),
                   _ptr(interp_weights), _ptr(gin), _ptr(ws), nws, B, C, int(in_h), int(in_w),
                   OH, OW,
                   int(kernel_size), P, int(interp), _DTYPES[grad_output.dtype],
                   _stream(grad_output))
    return gin


def mapped_gather_at_index(x, idx_mask, sample_map, interp_weights, kernel_size, interp):
    """The transpose of mapped_max_unpool: x [B,C,H,W] read at the sample every index names."""
    _check(x, x=x, idx_mask=idx_mask, sample_map=sample_map, interp_weights=interp_weights)
    if idx_mask.dtype != torch.int64 or idx_mask.dim() != 4 or \
            tuple(idx_mask.shape[:2]) != tuple(x.shape[:2]):
        raise RuntimeError("idx_mask must be an int64 [B, C, OH, OW] tensor with x's B and C")
    P = _npts(sample_map, interp_weights, 4)
    B, C, H, W = x.shape
    OH, OW = idx_mask.shape[2:]
    if tuple(sample_map.shape[:3]) != (OH, OW, int(kernel_size)):
        raise RuntimeError("sample_map %s does not match idx_mask %s / kernel_size %d"
                           % (tuple(sample_map.shape), tuple(idx_mask.shape), int(kernel_size)))
    out = torch.empty((B, C, OH, OW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _capi.call("sdk_mapped_gather_at_index", _ptr(x), _ptr(idx_mask), _ptr(sample_map),
                   _ptr(interp_weights), _ptr(out), B, C, H, W, OH, OW, int(kernel_size), P,
                   int(interp), _DTYPES[x.dtype], _stream(x))
    return out


def mapped_avg_pool(x, sample_map, interp_weights, kernel_size, interp):
    _check(x, x=x, sample_map=sample_map, interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 4)
    B, C, H, W = x.shape
    OH, OW, K = sample_map.shape[:3]
    if K != int(kernel_size):
        raise RuntimeError("kernel_size %d does not match sample_map %s"
                           % (int(kernel_size), tuple(sample_map.shape)))
    out = torch.empty((B, C, OH, OW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        _capi.call("sdk_mapped_avg_pool", _ptr(x), _ptr(sample_map), _ptr(interp_weights),
                   _ptr(out), B, C, H, W, OH, OW, K, P, int(interp), _DTYPES[x.dtype], _stream(x))
    return out


def mapped_avg_unpool(grad_output, sample_map, interp_weights, in_h, in_w, kernel_size, interp):
    _check(grad_output, grad_output=grad_output, sample_map=sample_map,
           interp_weights=interp_weights)
    P = _npts(sample_map, interp_weights, 4)
    B, C, OH, OW = grad_output.shape
    if tuple(sample_map.shape[:3]) != (OH, OW, int(kernel_size)):
        raise RuntimeError("sample_map %s does not match grad_output %s / kernel_size %d"
                           % (tuple(sample_map.shape), tuple(grad_output.shape), int(kernel_size)))
    gin = torch.empty((B, C, int(in_h), int(in_w)), dtype=grad_output.dtype,
                      device=grad_output.device)
    with torch.cuda.device(grad_output.device):
        plan, nplan, complete = _scatter_plan("avg_unpool", grad_output, sample_map,
                                              interp_weights, in_h, in_w, kernel_size, P, interp)
        if plan is not None:
            _capi.call("sdk_mapped_avg_unpool_planned", _ptr(grad_output), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(gin), _ptr(plan), nplan, complete, B, C,
                       int(in_h), int(in_w), OH, OW, int(kernel_size), P, int(interp),
                       _DTYPES[grad_output.dtype], _stream(grad_output))
            return gin
        ws, nws = _scatter_workspace(grad_output, in_h, in_w)
        _capi.call("sdk_mapped_avg_unpool", _ptr(grad_output), _ptr(sample_map),
                   _ptr(interp_weights), _ptr(gin), _ptr(ws), nws, B, C, int(in_h), int(in_w),
                   OH, OW, int(kernel_size), P, int(interp), _DTYPES[grad_output.dtype],
                   _stream(grad_output))
    return gin


# --------------------------------------------------------------------------- convolution
def _conv_dims(x_shape, weight, sample_map, kernel_size, transposed):
    K = int(kernel_size)
    if sample_map.shape[2] != K or weight.shape[2] != K:
        raise RuntimeError("kernel_size %d does not match sample_map %s / weight %s"
                           % (K, tuple(sample_map.shape), tuple(weight.shape)))
    B, Cin = int(x_shape[0]), int(x_shape[1])
    if weight.shape[0 if transposed else 1] != Cin:
        raise RuntimeError("weight %s does not match %d input channels"
                           % (tuple(weight.shape), Cin))
    Cout = int(weight.shape[1 if transposed else 0])
    return B, Cin, Cout, K


def mapped_conv_forward(x, sample_map, interp_weights, weight, bias, kernel_size, interp):
    _check(x, input=x, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
           bias=bias)
    P = _npts(sample_map, interp_weights, 4)
    B, Cin, Cout, K = _conv_dims(x.shape, weight, sample_map, kernel_size, False)
    H, W = x.shape[2:]
    OH, OW = sample_map.shape[:2]
    out = torch.empty((B, Cout, OH, OW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        ws, nws = _workspace(x, B, Cin, Cout, H, W, OH, OW, K, P, int(interp))
        plan, nplan = _conv_plan(x, sample_map, interp_weights, H, W, K, P, int(interp))
        dims = (B, Cin, H, W, Cout, OH, OW, K, P, int(interp), _DTYPES[x.dtype], _current_mode(),
                _stream(x))
        if plan is None:
            _capi.call("sdk_mapped_conv_forward", _ptr(x), _ptr(sample_map), _ptr(interp_weights),
                       _ptr(weight), _ptr(bias), _ptr(out), _ptr(ws), nws, *dims)
        else:
            _capi.call("sdk_mapped_conv_forward_planned", _ptr(x), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(weight), _ptr(bias), _ptr(out), _ptr(ws), nws,
                       _ptr(plan), nplan, *dims)
    return out


def mapped_conv_backward(grad_output, sample_map, interp_weights, x, weight, bias, kernel_size,
                         interp):
    # The reference checks input, sample_map, weight and bias here, not grad_output
    # (include/layers/mapped_convolution_layer.h:93-96); the kernels need it dense too.
    grad_output = grad_output.contiguous()
    _check(grad_output, grad_output=grad_output, input=x, sample_map=sample_map,
           interp_weights=interp_weights, weight=weight, bias=bias)
    P = _npts(sample_map, interp_weights, 4)
    B, Cin, Cout, K = _conv_dims(x.shape, weight, sample_map, kernel_size, False)
    H, W = x.shape[2:]
    OH, OW = sample_map.shape[:2]
    gi = torch.empty_like(x)
    gw = torch.empty_like(weight)
    gb = torch.empty((Cout,), dtype=x.dtype, device=x.device)
    dt = _DTYPES[x.dtype]
    with torch.cuda.device(x.device):
        ws, nws = _workspace(x, B, Cin, Cout, H, W, OH, OW, K, P, int(interp))
        s = _stream(x)
        dims = (B, Cin, H, W, Cout, OH, OW, K, P, int(interp), dt, _current_mode(), s)
        plan, nplan = _conv_plan(x, sample_map, interp_weights, H, W, K, P, int(interp))
        if plan is None:
            _capi.call("sdk_mapped_conv_backward", _ptr(grad_output), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(x), _ptr(weight), _ptr(gi), _ptr(gw), _ptr(gb),
                       _ptr(ws), nws, *dims)
        else:
            _capi.call("sdk_mapped_conv_backward_planned", _ptr(grad_output), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(x), _ptr(weight), _ptr(gi), _ptr(gw), _ptr(gb),
                       _ptr(ws), nws, _ptr(plan), nplan, *dims)
    return gi, gw, gb


def mapped_transposed_conv_forward(x, sample_map, interp_weights, weight, bias, out_h, out_w,
                                   kernel_size, interp):
    _check(x, input=x, sample_map=sample_map, interp_weights=interp_weights, weight=weight,
           bias=bias)
    P = _npts(sample_map, interp_weights, 4)
    B, Cin, Cout, K = _conv_dims(x.shape, weight, sample_map, kernel_size, True)
    IH, IW = x.shape[2:]
    if tuple(sample_map.shape[:2]) != (IH, IW):
        raise RuntimeError("sample_map grid %s must match the input's %s"
                           % (tuple(sample_map.shape[:2]), (IH, IW)))
    OH, OW = int(out_h), int(out_w)
    out = torch.empty((B, Cout, OH, OW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        ws, nws = _workspace(x, B, Cin, Cout, OH, OW, IH, IW, K, P, int(interp))
        plan, nplan = _conv_plan(x, sample_map, interp_weights, OH, OW, K, P, int(interp))
        dims = (B, Cin, IH, IW, Cout, OH, OW, K, P, int(interp), _DTYPES[x.dtype], _current_mode(),
                _stream(x))
        if plan is None:
            _capi.call("sdk_mapped_transposed_conv_forward", _ptr(x), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(weight), _ptr(bias), _ptr(out), _ptr(ws), nws,
                       *dims)
        else:
            _capi.call("sdk_mapped_transposed_conv_forward_planned", _ptr(x), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(weight), _ptr(bias), _ptr(out), _ptr(ws), nws,
                       _ptr(plan), nplan, *dims)
    return out


def mapped_transposed_conv_backward(grad_output, sample_map, interp_weights, x, weight, bias,
                                    kernel_size, interp):
    grad_output = grad_output.contiguous()
    _check(grad_output, grad_output=grad_output, input=x, sample_map=sample_map,
           interp_weights=interp_weights, weight=weight, bias=bias)
    P = _npts(sample_map, interp_weights, 4)
    B, Cin, Cout, K = _conv_dims(x.shape, weight, sample_map, kernel_size, True)
    IH, IW = x.shape[2:]
    OH, OW = grad_output.shape[2:]
    gi = torch.empty_like(x)
    gw = torch.empty_like(weight)
    gb = torch.empty((Cout,), dtype=x.dtype, device=x.device)
    dt = _DTYPES[x.dtype]
    with torch.cuda.device(x.device):
        ws, nws = _workspace(x, B, Cin, Cout, OH, OW, IH, IW, K, P, int(interp))
        s = _stream(x)
        dims = (B, Cin, IH, IW, Cout, OH, OW, K, P, int(interp), dt, _current_mode(), s)
        plan, nplan = _conv_plan(x, sample_map, interp_weights, OH, OW, K, P, int(interp))
        if plan is None:
            _capi.call("sdk_mapped_transposed_conv_backward", _ptr(grad_output), _ptr(sample_map),
                       _ptr(interp_weights), _ptr(x), _ptr(weight), _ptr(gi), _ptr(gw), _ptr(gb),
                       _ptr(ws), nws, *dims)
        else:
            _capi.call("sdk_mapped_transposed_conv_backward_planned", _ptr(grad_output),
                       _ptr(sample_map), _ptr(interp_weights), _ptr(x), _ptr(weight), _ptr(gi),
                       _ptr(gw), _ptr(gb), _ptr(ws), nws, _ptr(plan), nplan, *dims)
    return gi, gw, gb


# --------------------------------------------------------------------------- UV resample
def _uv_dims(quad_idx, tex_uv):
    if quad_idx.dtype != torch.int64 or quad_idx.dim() != 2:
        raise RuntimeError("quad_idx must be a 2-D int64 tensor, got %s %s"
                           % (quad_idx.dtype, tuple(quad_idx.shape)))
    if tuple(tex_uv.shape) != tuple(quad_idx.shape) + (2,):
        raise RuntimeError("tex_uv %s must be quad_idx %s + (2,)"
                           % (tuple(tex_uv.shape), tuple(quad_idx.shape)))
    return int(quad_idx.shape[0]), int(quad_idx.shape[1])


def resample_from_uv_maps(textures, quad_idx, tex_uv, interp):
    _check(textures, textures=textures, quad_idx=quad_idx, tex_uv=tex_uv)
    if textures.dim() != 5:
        raise RuntimeError("textures must be [B, C, T, TH, TW], got %s" % (tuple(textures.shape),))
    H, W = _uv_dims(quad_idx, tex_uv)
    B, C, NT, TH, TW = textures.shape
    out = torch.empty((B, C, H, W), dtype=textures.dtype, device=textures.device)
    with torch.cuda.device(textures.device):
        _capi.call("sdk_resample_from_uv_maps", _ptr(textures), _ptr(quad_idx), _ptr(tex_uv),
                   _ptr(out), B, C, NT, TH, TW, H, W, int(interp), _DTYPES[textures.dtype],
                   _stream(textures))
    return out


def _uv_plan(ref, quad_idx, NT, TH, TW, H, W, nbytes):
    """The image pixels bucketed by texture (sdk_resample_to_uv_maps_plan_build), kept per
    quad_idx tensor like the other plans; None when the cache is off or cannot key the tensor
    (the call then builds the buckets in its workspace)."""
    if not _plan_cache_enabled:
        return None
    kq = _tensor_key(quad_idx)
    if _uncacheable(kq):
        return None
    dt = _DTYPES[ref.dtype]
    key = ("uv_scatter", ref.device, dt, kq, NT, TH, TW, H, W)
    cur = torch.cuda.current_stream(ref.device)
    ent = _cache_lookup(key, cur)
    if ent is not None:
        return ent.plan
    if torch.cuda.is_current_stream_capturing():
        return None
    plan = torch.empty(nbytes, dtype=torch.uint8, device=ref.device)
    _capi.call("sdk_resample_to_uv_maps_plan_build", _ptr(quad_idx), _ptr(plan), nbytes, NT, TH,
               TW, H, W, dt, _stream(ref))
    _cache_insert(key, _PlanEntry(plan, nbytes, (quad_idx.untyped_storage(),), cur))
    return plan


def resample_to_uv_maps(x, quad_idx, tex_uv, num_textures, tex_h, tex_w, interp):
    _check(x, x=x, quad_idx=quad_idx, tex_uv=tex_uv)
    H, W = _uv_dims(quad_idx, tex_uv)
    if x.dim() != 4 or tuple(x.shape[2:]) != (H, W):
        raise RuntimeError("input %s must be [B, C, %d, %d]" % (tuple(x.shape), H, W))
    B, C = x.shape[:2]
    NT, TH, TW = int(num_textures), int(tex_h), int(tex_w)
    out = torch.empty((B, C, NT, TH, TW), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        nws = _capi.load().sdk_resample_to_uv_maps_workspace_bytes(NT, TH, TW, H, W,
                                                                   _DTYPES[x.dtype])
        plan = _uv_plan(x, quad_idx, NT, TH, TW, H, W, nws) if nws else None
        if plan is not None:
            _capi.call("sdk_resample_to_uv_maps_planned", _ptr(x), _ptr(quad_idx), _ptr(tex_uv),
                       _ptr(out), _ptr(plan), nws, B, C, NT, TH, TW, H, W, int(interp),
                       _DTYPES[x.dtype], _stream(x))
            return out
        ws = torch.empty(nws, dtype=torch.uint8, device=x.device) if nws else None
        _capi.call("sdk_resample_to_uv_maps", _ptr(x), _ptr(quad_idx), _ptr(tex_uv), _ptr(out),
                   _ptr(ws), nws, B, C, NT, TH, TW, H, W, int(interp), _DTYPES[x.dtype],
                   _stream(x))
    return out


# --------------------------------------------------------------------------- voting resample
def voting_resample_to_map(labels, sample_map, out_h, out_w, num_candidates):
    for name, t in (("input", labels), ("sample_map", sample_map)):
        if not t.is_cuda:
            raise RuntimeError("this backend runs on the GPU only: %s must be a CUDA/HIP tensor"
                               % name)
        if t.dtype != torch.int64:
            raise RuntimeError("%s must be int64 (got %s)" % (name, t.dtype))
        if not t.is_contiguous():
            raise RuntimeError("%s must be contiguous" % name)
    if labels.dim() != 4 or tuple(sample_map.shape) != tuple(labels.shape[2:]) + (2,):
        raise RuntimeError("input %s must be [B, C, IH, IW] and sample_map %s [IH, IW, 2]"
                           % (tuple(labels.shape), tuple(sample_map.shape)))
    B, C, IH, IW = labels.shape
    OH, OW, NC = int(out_h), int(out_w), int(num_candidates)
    out = torch.empty((B, C, OH, OW), dtype=torch.int64, device=labels.device)
    with torch.cuda.device(labels.device):
        nws = _capi.load().sdk_voting_resample_workspace_bytes(C, OH, OW, NC)
        # room for several batch elements per pass, within 256 MiB
        nws *= max(1, min(B, (256 << 20) // max(nws, 1)))
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=labels.device)
        _capi.call("sdk_voting_resample_to_map", _ptr(labels), _ptr(sample_map), _ptr(out),
                   _ptr(ws), nws, B, C, IH, IW, OH, OW, NC, _stream(labels))
    return out


# --------------------------------------------------------------------------- map generation
# Factory functions (no tensor argument to dispatch on): plain Python, not registered operators.

def equirect_kernel_map(height, width, kernel_h, kernel_w, stride=1, dilation=1, projection=1,
                        dtype=torch.float32, device="cuda"):
    """[ceil(H/stride), ceil(W/stride), kh*kw, 2] kernel map of an H x W equirectangular image,
    computed on the device.  projection: 0 grid, 1 inverse gnomonic, 2 inverse equirectangular."""
    if dtype not in _DTYPES:
        raise RuntimeError("unsupported dtype %s (float32 and float64 only)" % dtype)
    device = torch.device(device)
    if device.type != "cuda":
        raise RuntimeError("this backend runs on the GPU only: device must be a CUDA/HIP device")
    H, W, s = int(height), int(width), int(stride)
    if H < 2 or W < 1 or s < 1:
        raise RuntimeError("image %d x %d (height at least 2), stride %d" % (H, W, s))
    out = torch.empty((-(-H // s), -(-W // s), int(kernel_h) * int(kernel_w), 2), dtype=dtype,
                      device=device)
    with torch.cuda.device(out.device):
        _capi.call("sdk_equirect_kernel_map", _ptr(out), H, W, int(kernel_h), int(kernel_w), s,
                   int(dilation), int(projection), _DTYPES[dtype], _stream(out))
    return out


def gnomonic_kernel_at(lonlat, kernel_h, kernel_w, res_lat, res_lon, image_h=0, image_w=0):
    """[N, kh*kw, 2] gnomonic kernels about the points lonlat [N, 2] (lon, lat): spherical
    coordinates, or pixel coordinates of an image_h x image_w equirectangular image."""
    _check(lonlat, lonlat=lonlat)
    if lonlat.dim() != 2 or lonlat.shape[1] != 2:
        raise RuntimeError("lonlat must be [N, 2], got %s" % (tuple(lonlat.shape),))
    n = int(lonlat.shape[0])
    out = torch.empty((n, int(kernel_h) * int(kernel_w), 2), dtype=lonlat.dtype,
                      device=lonlat.device)
    with torch.cuda.device(lonlat.device):
        _capi.call("sdk_gnomonic_kernel_at", _ptr(lonlat), _ptr(out), n, int(kernel_h),
                   int(kernel_w), float(res_lat), float(res_lon), int(image_h), int(image_w),
                   _DTYPES[lonlat.dtype], _stream(lonlat))
    return out


def four_nearest_weighted_map(sample_map, height, width, eps=1e-6):
    """sample_map [..., 2] -> (map [..., 4, 2], weights [..., 4]): the four pixel centres around
    every sample (column wrapped, row clamped) with normalised inverse great-circle distance
    weights, the weighted form a bispherical P = 4 convolution takes."""
    _check(sample_map, sample_map=sample_map)
    if sample_map.shape[-1] != 2:
        raise RuntimeError("sample_map must end in 2, got %s" % (tuple(sample_map.shape),))
    lead = tuple(sample_map.shape[:-1])
    n = 1
    for v in lead:
        n *= int(v)
    out_map = torch.empty(lead + (4, 2), dtype=sample_map.dtype, device=sample_map.device)
    out_w = torch.empty(lead + (4,), dtype=sample_map.dtype, device=sample_map.device)
    with torch.cuda.device(sample_map.device):
        _capi.call("sdk_four_nearest_weighted_map", _ptr(sample_map), _ptr(out_map), _ptr(out_w),
                   n, int(height), int(width), float(eps), _DTYPES[sample_map.dtype],
                   _stream(sample_map))
    return out_map, out_w


# --------------------------------------------------------------------------- registration
_SCHEMAS = (
    ("resample_from_map",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, int interp) -> Tensor",
     resample_from_map),
    ("resample_to_map",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, int out_h, int out_w, int interp)"
     " -> Tensor", resample_to_map),
    ("resample_to_map_normalized",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, int out_h, int out_w, int interp,"
     " float eps) -> (Tensor, Tensor)", resample_to_map_normalized),
    ("resample_from_uv_maps",
     "(Tensor textures, Tensor quad_idx, Tensor tex_uv, int interp) -> Tensor",
     resample_from_uv_maps),
    ("resample_to_uv_maps",
     "(Tensor x, Tensor quad_idx, Tensor tex_uv, int num_textures, int tex_h, int tex_w,"
     " int interp) -> Tensor", resample_to_uv_maps),
    ("voting_resample_to_map",
     "(Tensor labels, Tensor sample_map, int out_h, int out_w, int num_candidates) -> Tensor",
     voting_resample_to_map),
    ("mapped_im2col",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, int interp) -> Tensor",
     mapped_im2col),
    ("mapped_col2im",
     "(Tensor col, Tensor sample_map, Tensor? interp_weights, int height, int width, int interp)"
     " -> Tensor", mapped_col2im),
    ("mapped_max_pool",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, int kernel_size, int interp)"
     " -> (Tensor, Tensor)", mapped_max_pool),
    ("mapped_max_unpool",
     "(Tensor grad_output, Tensor idx_mask, Tensor sample_map, Tensor? interp_weights, int in_h,"
     " int in_w, int kernel_size, int interp) -> Tensor", mapped_max_unpool),
    ("mapped_gather_at_index",
     "(Tensor x, Tensor idx_mask, Tensor sample_map, Tensor? interp_weights, int kernel_size,"
     " int interp) -> Tensor", mapped_gather_at_index),
    ("mapped_avg_pool",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, int kernel_size, int interp)"
     " -> Tensor", mapped_avg_pool),
    ("mapped_avg_unpool",
     "(Tensor grad_output, Tensor sample_map, Tensor? interp_weights, int in_h, int in_w,"
     " int kernel_size, int interp) -> Tensor", mapped_avg_unpool),
    ("mapped_conv_forward",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, Tensor weight, Tensor bias,"
     " int kernel_size, int interp) -> Tensor", mapped_conv_forward),
    ("mapped_conv_backward",
     "(Tensor grad_output, Tensor sample_map, Tensor? interp_weights, Tensor x, Tensor weight,"
     " Tensor bias, int kernel_size, int interp) -> (Tensor, Tensor, Tensor)",
     mapped_conv_backward),
    ("mapped_transposed_conv_forward",
     "(Tensor x, Tensor sample_map, Tensor? interp_weights, Tensor weight, Tensor bias,"
     " int out_h, int out_w, int kernel_size, int interp) -> Tensor",
     mapped_transposed_conv_forward),
    ("mapped_transposed_conv_backward",
     "(Tensor grad_output, Tensor sample_map, Tensor? interp_weights, Tensor x, Tensor weight,"
     " Tensor bias, int kernel_size, int interp) -> (Tensor, Tensor, Tensor)",
     mapped_transposed_conv_backward),
)

def _load_native():
    """Loads the compiled operator layer when it is built (its static registration implements
    the operators it names for the CUDA key) and returns (ctypes handle, operator names)."""
    path = os.path.join(os.path.dirname(_capi.LIB_PATH), "libsdk_torch_ops.so")
    if os.environ.get("SDK_TORCH_OPS", "") == "python" or not os.path.exists(path):
        return None, frozenset()
    _capi.load()
    torch.ops.load_library(path)
    lib = ctypes.CDLL(path)
    lib.sdk_torch_native_ops.restype = ctypes.c_char_p
    lib.sdk_torch_set_thread_mode.restype = ctypes.c_int
    lib.sdk_torch_plan_cache_size.restype = ctypes.c_int
    lib.sdk_torch_current_mode.restype = ctypes.c_int
    for name in ("sdk_torch_set_default_mode", "sdk_torch_set_plan_cache",
                 "sdk_torch_set_unpool_workspace"):
        getattr(lib, name).restype = None
    return lib, frozenset(lib.sdk_torch_native_ops().decode().split(","))


_library = torch.library.Library(_NS, "DEF")
for _name, _schema, _fn in _SCHEMAS:
    _library.define(_name + _schema)
_native, _NATIVE_OPS = _load_native()
for _name, _schema, _fn in _SCHEMAS:
    if _name not in _NATIVE_OPS:
        _library.impl(_name, _fn, "CUDA")


# The functions above stay reachable under their own names in PYTHON_IMPL; where the compiled
# layer implements an operator, the module-level name is the registered operator itself, so
# that callers of this module and callers of torch.ops.sdk_mapped_ops run the same code.
ops = getattr(torch.ops, _NS)
PYTHON_IMPL = {_name: _fn for _name, _schema, _fn in _SCHEMAS}
for _name in _NATIVE_OPS:
    globals()[_name] = getattr(ops, _name)
