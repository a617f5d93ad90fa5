"""sdk_mapped_max_unpool_static, the unpool entry point that allocates nothing (its tile-window
scratch is an array inside the library), against sdk_mapped_max_unpool with a caller-owned
workspace: both called through the C ABI on the same inputs, twice in a row, the second call on
a smaller input so that stale contents of the shared array would show.  Tolerance: 1e-4 of the
largest gradient (float32 backward; the two calls add a pixel's few contributions in an order
that may differ), and both against the CPU oracle.
"""
import ctypes

import numpy as np
import pytest
import torch

from conftest import relerr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _unpool_both_ways(oracle, B, C, H, W, seed, weighted=False):
    """weighted: bilinear taps about P = 4 weighted points per sample instead of one nearest
    tap (the entry point forwards interp and num_interp_pts to the same kernels)."""
    import workloads
    from _spherical_distortion_ext import _capi, _ops
    rng = np.random.default_rng(seed)
    K = 9
    m = workloads.gnomonic_kernel_map(H, W, stride=2, dilation=2)
    OH, OW = m.shape[:2]
    iw, P, interp = None, 0, 0
    if weighted:
        P, interp = 4, 1
        m = (m[:, :, :, None, :] + rng.uniform(-0.7, 0.7, (OH, OW, K, P, 2))).astype(np.float32)
        iw = rng.uniform(0.1, 1.0, (OH, OW, K, P)).astype(np.float32)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    tm, tg = _t(m), _t(g)
    tiw = None if iw is None else _t(iw)
    _, idx = _ops.mapped_max_pool(_t(x), tm, tiw, K, interp)
    p, s = _ops._ptr, _ops._stream(tg)
    dims = (B, C, H, W, OH, OW, K, P, interp, _capi.SDK_F32, s)
    # the existing entry point with its workspace
    nws = _capi.load().sdk_mapped_max_unpool_workspace_bytes(H, W, _capi.SDK_F32)
    assert nws > 0
    ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
    want = torch.full((B, C, H, W), float("nan"), device=DEV)
    _capi.call("sdk_mapped_max_unpool", p(tg), p(idx), p(tm), p(tiw), p(want), p(ws), nws, *dims)
    # the entry point under test: no workspace argument, no allocation
    got = torch.full((B, C, H, W), float("nan"), device=DEV)
    _capi.call("sdk_mapped_max_unpool_static", p(tg), p(idx), p(tm), p(tiw), p(got), *dims)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(got).all())
    scale = float(want.abs().max())
    assert float((got - want).abs().max()) <= 1e-4 * scale
    ref = oracle.mapped_max_unpool(g, idx.cpu().numpy(), m, H, W, K, interp, iw)
    assert relerr(got.cpu().numpy(), ref) <= 1e-4


def test_static_unpool_matches_the_workspace_entry_point_twice(oracle):
    _unpool_both_ways(oracle, 2, 12, 128, 256, seed=1)   # 16 tiles
    _unpool_both_ways(oracle, 1, 5, 48, 80, seed=2)      # smaller: 3 tiles of the same array


def test_static_unpool_with_weighted_bilinear_taps(oracle):
    _unpool_both_ways(oracle, 2, 6, 64, 128, seed=3, weighted=True)
    _unpool_both_ways(oracle, 1, 3, 32, 48, seed=4, weighted=True)


def test_static_unpool_rejects_a_plane_beyond_its_scratch():
    from _spherical_distortion_ext import _capi
    lib = _capi.load()
    one = ctypes.c_void_p(256)   # never dereferenced: the size check comes first
    rc = lib.sdk_mapped_max_unpool_static(one, one, one, None, one, 1, 1, 4096, 4224, 8, 8, 9, 0,
                                          0, _capi.SDK_F32, None)
    assert rc != 0
    assert b"built-in scratch" in lib.sdk_last_error()
