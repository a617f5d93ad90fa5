"""numpy front-end of the CPU oracle (oracle/sdk_oracle.cpp).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg.  The shipped package never imports this module.

All functions take and return C-contiguous numpy arrays of float32 or float64
(the index tensor of the pooling pair is int64).  Argument order follows the
reference's pybind entry points (ext_modules/include/layers/*.h) with
``interp_weights=None`` selecting the unweighted variant.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libsdk_oracle.so")
_lib = None

NEAREST, BILINEAR, BISPHERICAL = 0, 1, 2


def build(force=False):
    """Compile oracle/libsdk_oracle.so with g++ (a few seconds)."""
    src = os.path.join(_HERE, "sdk_oracle.cpp")
    if force or not os.path.exists(_LIB_PATH) or \
            os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "oracle"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
    return _lib


def _dt(a):
    if a.dtype == np.float32:
        return 0
    if a.dtype == np.float64:
        return 1
    raise TypeError("oracle supports float32 / float64, got %s" % a.dtype)


def _c(a, dtype=None):
    if a is None:
        return None
    if hasattr(a, "detach"):  # torch tensor on the CPU
        a = a.detach().cpu().numpy()
    a = np.ascontiguousarray(a)
    if dtype is not None and a.dtype != dtype:
        raise TypeError("dtype mismatch: %s vs %s" % (a.dtype, dtype))
    return a


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _i64(*v):
    return [ctypes.c_int64(int(x)) for x in v]


def _i32(*v):
    return [ctypes.c_int(int(x)) for x in v]


def _check(rc):
    if rc != 0:
        raise RuntimeError("oracle call failed with status %d" % rc)


def _num_pts(sample_map, interp_weights):
    return 0 if interp_weights is None else int(interp_weights.shape[-1])


def resample_from_map(x, sample_map, interp, interp_weights=None):
    """Gather.  x [B,C,H,W], map [MH,MW,(P,)2] -> [B,C,MH,MW]."""
    x = _c(x); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    B, C, H, W = x.shape
    MH, MW = m.shape[:2]
    out = np.empty((B, C, MH, MW), x.dtype)
    _check(lib().sdk_oracle_resample_from_map(
        _p(x), _p(m), _p(w), _p(out), *_i64(B, C, H, W, MH, MW),
        *_i32(_num_pts(m, w), int(interp), _dt(x))))
    return out


def resample_to_map(x, sample_map, out_h, out_w, interp, interp_weights=None):
    """Scatter.  x [B,C,MH,MW], map [MH,MW,(P,)2] -> [B,C,out_h,out_w]."""
    x = _c(x); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    B, C, MH, MW = x.shape
    out = np.empty((B, C, out_h, out_w), x.dtype)
    _check(lib().sdk_oracle_resample_to_map(
        _p(x), _p(m), _p(w), _p(out), *_i64(B, C, MH, MW, out_h, out_w),
        *_i32(_num_pts(m, w), int(interp), _dt(x))))
    return out


def mapped_im2col(im, sample_map, interp, interp_weights=None):
    """im [C,H,W], map [OH,OW,K,(P,)2] -> col [C*K, OH*OW]."""
    im = _c(im); m = _c(sample_map, im.dtype); w = _c(interp_weights, im.dtype)
    C, H, W = im.shape
    OH, OW, K = m.shape[:3]
    col = np.empty((C * K, OH * OW), im.dtype)
    _check(lib().sdk_oracle_mapped_im2col(
        _p(im), _p(m), _p(w), _p(col), *_i64(C, H, W, OH * OW, K),
        *_i32(_num_pts(m, w), int(interp), _dt(im))))
    return col


def mapped_col2im(col, sample_map, height, width, interp, interp_weights=None):
    """col [C*K, OH*OW], map [OH,OW,K,(P,)2] -> im [C,height,width]."""
    col = _c(col); m = _c(sample_map, col.dtype); w = _c(interp_weights, col.dtype)
    OH, OW, K = m.shape[:3]
    C = col.shape[0] // K
    im = np.zeros((C, height, width), col.dtype)
    _check(lib().sdk_oracle_mapped_col2im(
        _p(col), _p(m), _p(w), _p(im), *_i64(C, height, width, OH * OW, K),
        *_i32(_num_pts(m, w), int(interp), _dt(col))))
    return im


def mapped_max_pool(x, sample_map, kernel_size, interp, interp_weights=None,
                    host_init_quirk=False):
    """-> (values [B,C,OH,OW], indices int64).  ``host_init_quirk`` selects the
    reference host branch's initial running maximum (smallest positive normal
    instead of -FLT_MAX)."""
    x = _c(x); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    B, C, H, W = x.shape
    OH, OW, K = m.shape[:3]
    assert K == kernel_size
    out = np.empty((B, C, OH, OW), x.dtype)
    idx = np.empty((B, C, OH, OW), np.int64)
    _check(lib().sdk_oracle_mapped_max_pool(
        _p(x), _p(m), _p(w), _p(out), _p(idx), *_i64(B, C, H, W, OH, OW, K),
        *_i32(_num_pts(m, w), int(interp), _dt(x), 1 if host_init_quirk else 0)))
    return out, idx


def mapped_max_unpool(grad_output, idx_mask, sample_map, in_h, in_w, kernel_size,
                      interp, interp_weights=None):
    g = _c(grad_output); m = _c(sample_map, g.dtype); w = _c(interp_weights, g.dtype)
    idx = _c(idx_mask, np.int64)
    B, C, OH, OW = g.shape
    out = np.empty((B, C, in_h, in_w), g.dtype)
    _check(lib().sdk_oracle_mapped_max_unpool(
        _p(g), _p(idx), _p(m), _p(w), _p(out), *_i64(B, C, in_h, in_w, OH, OW, kernel_size),
        *_i32(_num_pts(m, w), int(interp), _dt(g))))
    return out


def mapped_avg_pool(x, sample_map, kernel_size, interp, interp_weights=None):
    x = _c(x); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    B, C, H, W = x.shape
    OH, OW = m.shape[:2]
    out = np.empty((B, C, OH, OW), x.dtype)
    _check(lib().sdk_oracle_mapped_avg_pool(
        _p(x), _p(m), _p(w), _p(out), *_i64(B, C, H, W, OH, OW, kernel_size),
        *_i32(_num_pts(m, w), int(interp), _dt(x))))
    return out


def mapped_avg_unpool(grad_output, sample_map, in_h, in_w, kernel_size, interp,
                      interp_weights=None):
    g = _c(grad_output); m = _c(sample_map, g.dtype); w = _c(interp_weights, g.dtype)
    B, C, OH, OW = g.shape
    out = np.empty((B, C, in_h, in_w), g.dtype)
    _check(lib().sdk_oracle_mapped_avg_unpool(
        _p(g), _p(m), _p(w), _p(out), *_i64(B, C, in_h, in_w, OH, OW, kernel_size),
        *_i32(_num_pts(m, w), int(interp), _dt(g))))
    return out


def resample_from_uv_maps(textures, quad_idx, tex_uv, interp):
    """textures [B,C,NT,TH,TW], quad_idx [H,W] int64, tex_uv [H,W,2] -> [B,C,H,W]."""
    t = _c(textures); q = _c(quad_idx, np.int64); uv = _c(tex_uv, t.dtype)
    B, C, NT, TH, TW = t.shape
    H, W = q.shape
    out = np.empty((B, C, H, W), t.dtype)
    _check(lib().sdk_oracle_resample_from_uv_maps(
        _p(t), _p(q), _p(uv), _p(out), *_i64(B, C, NT, TH, TW, H, W), *_i32(int(interp), _dt(t))))
    return out


def resample_to_uv_maps(x, quad_idx, tex_uv, num_textures, tex_h, tex_w, interp):
    """x [B,C,H,W] -> [B,C,NT,TH,TW]: the adjoint of resample_from_uv_maps."""
    x = _c(x); q = _c(quad_idx, np.int64); uv = _c(tex_uv, x.dtype)
    B, C, H, W = x.shape
    out = np.empty((B, C, num_textures, tex_h, tex_w), x.dtype)
    _check(lib().sdk_oracle_resample_to_uv_maps(
        _p(x), _p(q), _p(uv), _p(out), *_i64(B, C, num_textures, tex_h, tex_w, H, W),
        *_i32(int(interp), _dt(x))))
    return out


def mapped_conv_forward(x, sample_map, weight, bias, kernel_size, interp,
                        interp_weights=None):
    x = _c(x); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    weight = _c(weight, x.dtype); bias = _c(bias, x.dtype)
    B, Cin, H, W = x.shape
    Cout = weight.shape[0]
    OH, OW = m.shape[:2]
    out = np.empty((B, Cout, OH, OW), x.dtype)
    _check(lib().sdk_oracle_mapped_conv_forward(
        _p(x), _p(m), _p(w), _p(weight), _p(bias), _p(out),
        *_i64(B, Cin, H, W, Cout, OH, OW, kernel_size),
        *_i32(_num_pts(m, w), int(interp), _dt(x))))
    return out


def mapped_conv_backward(grad_output, sample_map, x, weight, bias, kernel_size, interp,
                         interp_weights=None):
    """-> (grad_input, grad_weight, grad_bias)."""
    g = _c(grad_output); m = _c(sample_map, g.dtype); w = _c(interp_weights, g.dtype)
    x = _c(x, g.dtype); weight = _c(weight, g.dtype)
    B, Cin, H, W = x.shape
    Cout = weight.shape[0]
    OH, OW = m.shape[:2]
    gi = np.empty_like(x)
    gw = np.empty_like(weight)
    gb = np.empty((Cout,), g.dtype)
    dims = _i64(B, Cin, H, W, Cout, OH, OW, kernel_size)
    tail = _i32(_num_pts(m, w), int(interp), _dt(g))
    _check(lib().sdk_oracle_mapped_conv_backward_input(
        _p(g), _p(m), _p(w), _p(weight), _p(gi), *dims, *tail))
    _check(lib().sdk_oracle_mapped_conv_backward_weight(
        _p(g), _p(m), _p(w), _p(x), _p(gw), *dims, *tail))
    _check(lib().sdk_oracle_bias_grad(_p(g), _p(gb), *_i64(B, Cout, OH * OW),
                                      *_i32(_dt(g))))
    return gi, gw, gb


def mapped_conv_backward_input(grad_output, sample_map, x_shape, weight, kernel_size, interp,
                               interp_weights=None):
    """grad_input [B,Cin,H,W] alone (x_shape = the input's shape)."""
    g = _c(grad_output); m = _c(sample_map, g.dtype); w = _c(interp_weights, g.dtype)
    weight = _c(weight, g.dtype)
    B, Cin, H, W = (int(v) for v in x_shape)
    Cout = weight.shape[0]
    OH, OW = m.shape[:2]
    gi = np.empty((B, Cin, H, W), g.dtype)
    _check(lib().sdk_oracle_mapped_conv_backward_input(
        _p(g), _p(m), _p(w), _p(weight), _p(gi), *_i64(B, Cin, H, W, Cout, OH, OW, kernel_size),
        *_i32(_num_pts(m, w), int(interp), _dt(g))))
    return gi


def mapped_transposed_conv_forward(x, sample_map, weight, bias, out_h, out_w,
                                   kernel_size, interp, interp_weights=None):
    x = _c(x); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    weight = _c(weight, x.dtype); bias = _c(bias, x.dtype)
    B, Cin, IH, IW = x.shape
    Cout = weight.shape[1]
    out = np.empty((B, Cout, out_h, out_w), x.dtype)
    _check(lib().sdk_oracle_mapped_transposed_conv_forward(
        _p(x), _p(m), _p(w), _p(weight), _p(bias), _p(out),
        *_i64(B, Cin, IH, IW, Cout, out_h, out_w, kernel_size),
        *_i32(_num_pts(m, w), int(interp), _dt(x))))
    return out


def mapped_transposed_conv_backward(grad_output, sample_map, x, weight, bias,
                                    kernel_size, interp, interp_weights=None):
    g = _c(grad_output); m = _c(sample_map, g.dtype); w = _c(interp_weights, g.dtype)
    x = _c(x, g.dtype); weight = _c(weight, g.dtype)
    B, Cin, IH, IW = x.shape
    Cout = weight.shape[1]
    OH, OW = g.shape[2:]
    gi = np.empty_like(x)
    gw = np.empty_like(weight)
    gb = np.empty((Cout,), g.dtype)
    dims = _i64(B, Cin, IH, IW, Cout, OH, OW, kernel_size)
    tail = _i32(_num_pts(m, w), int(interp), _dt(g))
    _check(lib().sdk_oracle_mapped_transposed_conv_backward_input(
        _p(g), _p(m), _p(w), _p(weight), _p(gi), *dims, *tail))
    _check(lib().sdk_oracle_mapped_transposed_conv_backward_weight(
        _p(g), _p(m), _p(w), _p(x), _p(gw), *dims, *tail))
    _check(lib().sdk_oracle_bias_grad(_p(g), _p(gb), *_i64(B, Cout, OH * OW),
                                      *_i32(_dt(g))))
    return gi, gw, gb


def num_threads():
    return int(lib().sdk_oracle_num_threads())


GRID, INVERSE_GNOMONIC, INVERSE_EQUIRECTANGULAR = 0, 1, 2


def equirect_kernel_map(shape, kernel_size, stride=1, dilation=1, projection=INVERSE_GNOMONIC,
                        dtype=np.float32):
    """[ceil(H/stride), ceil(W/stride), kh*kw, 2] kernel map of an H x W equirectangular image
    (layers/util/mapping_functions.py:43-160)."""
    H, W = shape
    kh, kw = kernel_size
    out = np.empty((-(-H // stride), -(-W // stride), kh * kw, 2), dtype)
    _check(lib().sdk_oracle_equirect_kernel_map(
        _p(out), *_i64(H, W, kh, kw, stride, dilation), *_i32(projection, _dt(out))))
    return out


def gnomonic_kernel_at(lonlat, kh, kw, res_lat, res_lon, image_shape=None):
    """[N, kh*kw, 2] gnomonic kernels about the points lonlat [N, 2], in (lon, lat) or, with
    image_shape, in equirectangular pixel coordinates
    (layers/util/icosahedron_functions.py:47-103, layers/util/conversions.py:33-52)."""
    pts = _c(lonlat)
    out = np.empty((pts.shape[0], kh * kw, 2), pts.dtype)
    ih, iw = image_shape if image_shape is not None else (0, 0)
    _check(lib().sdk_oracle_gnomonic_kernel_at(
        _p(pts), _p(out), *_i64(pts.shape[0], kh, kw), ctypes.c_double(res_lat),
        ctypes.c_double(res_lon), *_i64(ih, iw), *_i32(_dt(pts))))
    return out


def voting_resample_to_map(labels, sample_map, out_h, out_w, num_candidates):
    """labels [B,C,IH,IW] int64, sample_map [IH,IW,2] int64 -> [B,C,OH,OW] int64: the label
    with the most votes per output pixel (src/cpp/voting_resample_layer.cpp:8-37)."""
    x = _c(labels, np.int64); m = _c(sample_map, np.int64)
    B, C, IH, IW = x.shape
    out = np.empty((B, C, out_h, out_w), np.int64)
    _check(lib().sdk_oracle_voting_resample(_p(x), _p(m), _p(out),
                                            *_i64(B, C, IH, IW, out_h, out_w, num_candidates)))
    return out


def mapped_gather_at_index(image, idx_mask, sample_map, interp, interp_weights=None):
    """image [B,C,H,W], idx_mask [B,C,OH,OW] int64 -> [B,C,OH,OW]: the image interpolated at the
    sample every index names; the transpose of mapped_max_unpool."""
    x = _c(image); m = _c(sample_map, x.dtype); w = _c(interp_weights, x.dtype)
    idx = _c(idx_mask, np.int64)
    B, C, H, W = x.shape
    OH, OW = idx.shape[2:]
    out = np.empty((B, C, OH, OW), x.dtype)
    _check(lib().sdk_oracle_mapped_gather_at_index(
        _p(x), _p(idx), _p(m), _p(w), _p(out), *_i64(B, C, H, W, OH, OW),
        *_i32(_num_pts(m, w), int(interp), _dt(x))))
    return out
