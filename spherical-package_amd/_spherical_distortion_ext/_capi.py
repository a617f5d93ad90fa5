"""ctypes view of libsdk_mapped_ops.so, the C-ABI library built from csrc/.

The declarations below mirror include/sdk_mapped_ops.h one to one.  Loading
fails loudly when the library has not been built: there is no fallback path.
"""
import ctypes
import os

_PKG_ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_PKG_ROOT, "libsdk_mapped_ops.so")

SDK_F32, SDK_F64 = 0, 1
SDK_COMPUTE_NATIVE, SDK_COMPUTE_BF16, SDK_COMPUTE_UNFUSED, SDK_COMPUTE_SPLIT = 0, 1, 2, 3

_vp, _i64, _i32, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_size_t

# name -> argument types, in header order
_CONV_DIMS = [_i64] * 8 + [_i32] * 4 + [_vp]
SIGNATURES = {
    "sdk_resample_from_map": [_vp] * 4 + [_i64] * 6 + [_i32] * 3 + [_vp],
    "sdk_resample_to_map": [_vp] * 6 + [_sz] + [_i64] * 6 + [_i32] * 3 + [_vp],
    "sdk_resample_to_map_normalized": [_vp] * 6 + [_sz, ctypes.c_double] + [_i64] * 6 + [_i32] * 3
                                      + [_vp],
    "sdk_normalize_by_weight_sum": [_vp, _vp, ctypes.c_double, _i64, _i64, _i32, _vp],
    "sdk_resample_from_uv_maps": [_vp] * 4 + [_i64] * 7 + [_i32] * 2 + [_vp],
    "sdk_resample_to_uv_maps": [_vp] * 5 + [_sz] + [_i64] * 7 + [_i32] * 2 + [_vp],
    "sdk_resample_to_uv_maps_plan_build": [_vp, _vp, _sz] + [_i64] * 5 + [_i32, _vp],
    "sdk_resample_to_uv_maps_planned": [_vp] * 5 + [_sz] + [_i64] * 7 + [_i32] * 2 + [_vp],
    "sdk_equirect_kernel_map": [_vp] + [_i64] * 6 + [_i32] * 2 + [_vp],
    "sdk_gnomonic_kernel_at": [_vp, _vp] + [_i64] * 3 + [ctypes.c_double] * 2 + [_i64] * 2
                              + [_i32, _vp],
    "sdk_voting_resample_to_map": [_vp] * 4 + [_sz] + [_i64] * 7 + [_vp],
    "sdk_four_nearest_weighted_map": [_vp] * 3 + [_i64] * 3 + [ctypes.c_double, _i32, _vp],
    "sdk_mapped_im2col": [_vp] * 4 + [_i64] * 6 + [_i32] * 3 + [_vp],
    "sdk_mapped_col2im": [_vp] * 4 + [_i64] * 6 + [_i32] * 3 + [_vp],
    "sdk_mapped_max_pool": [_vp] * 5 + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_max_unpool": [_vp] * 6 + [_sz] + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_max_unpool_static": [_vp] * 5 + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_gather_at_index": [_vp] * 5 + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_avg_pool": [_vp] * 4 + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_avg_unpool": [_vp] * 5 + [_sz] + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_conv_forward": [_vp] * 7 + [_sz] + _CONV_DIMS,
    "sdk_mapped_conv_backward_input": [_vp] * 6 + [_sz] + _CONV_DIMS,
    "sdk_mapped_conv_backward_weight": [_vp] * 6 + [_sz] + _CONV_DIMS,
    "sdk_bias_grad": [_vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "sdk_mapped_conv_backward": [_vp] * 9 + [_sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_backward": [_vp] * 9 + [_sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_forward": [_vp] * 7 + [_sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_backward_input": [_vp] * 6 + [_sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_backward_weight": [_vp] * 6 + [_sz] + _CONV_DIMS,
    # the same entry points taking a plan (pointer, bytes) after the workspace pair
    "sdk_mapped_conv_forward_planned": [_vp] * 7 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_conv_backward_input_planned": [_vp] * 6 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_conv_backward_weight_planned": [_vp] * 6 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_conv_backward_planned": [_vp] * 9 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_backward_planned": [_vp] * 9 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_forward_planned": [_vp] * 7 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_backward_input_planned": [_vp] * 6 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_transposed_conv_backward_weight_planned": [_vp] * 6 + [_sz, _vp, _sz] + _CONV_DIMS,
    "sdk_mapped_conv_plan_build": [_vp] * 3 + [_sz] + [_i64] * 5 + [_i32] * 3 + [_vp],
    # plans of the scatter direction
    "sdk_resample_to_map_plan_build": [_vp] * 3 + [_sz] + [_i64] * 5 + [_i32] * 3 + [_vp],
    "sdk_resample_plan_complete": [_vp, _sz, _vp, _vp],
    "sdk_resample_to_map_planned": [_vp] * 6 + [_sz, _i32, _i32, ctypes.c_double] + [_i64] * 6
                                   + [_i32] * 3 + [_vp],
    "sdk_mapped_avg_unpool_planned": [_vp] * 5 + [_sz, _i32] + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_max_unpool_plan_build": [_vp, _vp, _sz] + [_i64] * 5 + [_i32] * 3 + [_vp],
    "sdk_mapped_max_unpool_planned": [_vp] * 6 + [_sz] + [_i64] * 7 + [_i32] * 3 + [_vp],
    "sdk_mapped_max_unpool_plan_bands": [_vp, _sz, _i64, _i64, _i32, _vp, _vp],
    "sdk_mapped_max_unpool_planned_bands": [_vp] * 5 + [_sz] + [_i64] * 7 + [_i32] * 2 + [_vp],
}
OTHER_SYMBOLS = ("sdk_last_error", "sdk_version", "sdk_mapped_conv_workspace_bytes",
                 "sdk_resample_to_map_workspace_bytes", "sdk_mapped_max_unpool_workspace_bytes",
                 "sdk_resample_to_uv_maps_workspace_bytes", "sdk_voting_resample_workspace_bytes",
                 "sdk_mapped_conv_plan_bytes")

_lib = None


def load():
    """Returns the loaded library, raising ImportError when it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "%s not found: build the HIP extension first (make -C %s)"
            % (LIB_PATH, os.path.join(_PKG_ROOT, "csrc")))
    lib = ctypes.CDLL(LIB_PATH)
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    lib.sdk_last_error.argtypes = []
    lib.sdk_last_error.restype = ctypes.c_char_p
    lib.sdk_version.argtypes = []
    lib.sdk_version.restype = ctypes.c_int
    lib.sdk_mapped_conv_workspace_bytes.argtypes = [_i64] * 8 + [_i32] * 4
    lib.sdk_mapped_conv_workspace_bytes.restype = _sz
    lib.sdk_resample_to_map_workspace_bytes.argtypes = [_i64, _i64, _i32]
    lib.sdk_resample_to_map_workspace_bytes.restype = _sz
    lib.sdk_mapped_max_unpool_workspace_bytes.argtypes = [_i64, _i64, _i32]
    lib.sdk_mapped_max_unpool_workspace_bytes.restype = _sz
    lib.sdk_resample_to_uv_maps_workspace_bytes.argtypes = [_i64] * 5 + [_i32]
    lib.sdk_resample_to_uv_maps_workspace_bytes.restype = _sz
    lib.sdk_voting_resample_workspace_bytes.argtypes = [_i64] * 4
    lib.sdk_voting_resample_workspace_bytes.restype = _sz
    lib.sdk_mapped_conv_plan_bytes.argtypes = [_i64] * 5 + [_i32] * 3
    lib.sdk_mapped_conv_plan_bytes.restype = _sz
    _lib = lib
    return lib


def call(name, *args):
    """Calls an entry point; a non-zero status becomes a RuntimeError."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        raise RuntimeError("%s failed (status %d): %s"
                           % (name, rc, lib.sdk_last_error().decode()))
