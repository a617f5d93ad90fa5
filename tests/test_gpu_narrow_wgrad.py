"""Weight gradient of narrow layers with nearest taps (at most 64 output channels, no
interpolation weights), which has a kernel of its own: every kernel size it is built for, both
widths of the output-channel block, a grid whose right edge cuts a tile, channel counts that
leave the last chunk and the last rows partly empty, taps outside the image, and a launch in
which every workgroup walks several tiles (the requests for a tile are made while the one
before it is multiplied).
"""
import numpy as np
import pytest
import torch

from conftest import relerr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _nearest_case(seed, B, Cin, Cout, H, W, K):
    """A map of the image's own size: sample k of pixel (y, x) lies near (y, x) + offset k,
    jittered by less than half a pixel; some samples of border pixels fall outside."""
    rng = np.random.default_rng(seed)
    ys, xs = np.meshgrid(np.arange(H), np.arange(W), indexing="ij")
    dy = rng.integers(-2, 3, K)
    dx = rng.integers(-2, 3, K)
    cx = xs[..., None] + dx + rng.uniform(-0.4, 0.4, (H, W, K))
    cy = ys[..., None] + dy + rng.uniform(-0.4, 0.4, (H, W, K))
    m = np.ascontiguousarray(np.stack([cx, cy], -1).astype(np.float32))
    x = rng.standard_normal((B, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    g = rng.standard_normal((B, Cout, H, W)).astype(np.float32)
    return m, x, w, b, g


@pytest.mark.parametrize("mode", ["native", "split", "bf16"])
@pytest.mark.parametrize("Cout", [24, 48])
@pytest.mark.parametrize("K", range(1, 11))
def test_every_kernel_size_and_block_width(ops, oracle, K, Cout, mode):
    m, x, w, b, g = _nearest_case(100 * K + Cout, 2, 40, Cout, 20, 37, K)
    ops.set_conv_compute(mode)
    try:
        gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), None, _t(x), _t(w), _t(b), K, 0)
    finally:
        ops.set_conv_compute("native")
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, 0, None)
    tol = 1e-2 if mode == "bf16" else 1e-4
    assert relerr(gw.cpu().numpy(), ww) <= tol
    assert relerr(gi.cpu().numpy(), wi) <= tol
    assert relerr(gb.cpu().numpy(), wb) <= 1e-4


@pytest.mark.parametrize("mode", ["native", "split"])
@pytest.mark.parametrize("Cout,K", [(40, 7), (8, 9), (64, 4)])
def test_workgroups_that_walk_several_tiles(ops, oracle, Cout, K, mode):
    # 8 batch elements x 8 chunks of image channels: eight workgroups per kind share the 24
    # tiles of the 48 x 64 grid, three each
    m, x, w, b, g = _nearest_case(7 + Cout + K, 8, 256, Cout, 48, 64, K)
    tm = _t(m)
    ops.set_conv_compute(mode)
    try:
        for rep in range(2):                   # second call: the plan comes from the cache
            gi, gw, gb = ops.mapped_conv_backward(_t(g), tm, None, _t(x), _t(w), _t(b), K, 0)
    finally:
        ops.set_conv_compute("native")
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, 0, None)
    assert relerr(gw.cpu().numpy(), ww) <= 1e-4
    assert relerr(gi.cpu().numpy(), wi) <= 1e-4


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("M", [1, 3, 5, 642, 1023, 4098, 20007])
def test_bias_gradient_on_planes_of_any_size(M, dtype):
    """Planes whose size is not a multiple of four elements start at any alignment: the sum
    takes the elements up to a 16-byte boundary singly, then 16-byte loads."""
    from _spherical_distortion_ext import _capi
    lib = _capi.load()
    rng = np.random.default_rng(M)
    g = rng.standard_normal((3, 5, M)).astype(dtype)
    tg = torch.from_numpy(g).to(DEV)
    out = torch.empty(5, dtype=tg.dtype, device=DEV)
    code = _capi.SDK_F32 if dtype == np.float32 else _capi.SDK_F64
    rc = lib.sdk_bias_grad(tg.data_ptr(), out.data_ptr(), 3, 5, M, code, None)
    assert rc == 0, lib.sdk_last_error()
    torch.cuda.synchronize()
    want = g.astype(np.float64).sum(axis=(0, 2))
    tol = 1e-5 if dtype == np.float32 else 1e-12
    scale = np.abs(g.astype(np.float64)).sum(axis=(0, 2)).max()
    assert np.abs(out.cpu().numpy() - want).max() <= tol * scale
