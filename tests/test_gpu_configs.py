"""The benchmark's own configurations against the CPU oracle: configuration 1 at its full
size, configurations 2-5 from the same generators (workloads.py) at sizes the oracle finishes
in seconds.  Same seeds and bits on both sides.  Tolerances are the ones the task states:
pooling indices and nearest-neighbour values bit-exact, float32 forward 1e-5, float32 backward
(atomic or tiled accumulation order) 1e-4, relative to the largest magnitude of the result.
"""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import workloads  # noqa: E402
from conftest import relerr  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FWD, BWD = 1e-5, 1e-4


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _n(t):
    return t.detach().cpu().numpy()


def _conv_both_ways(ops, oracle, c):
    K, it = c["kernel_size"], c["interp"]
    iw = c.get("interp_weights")
    x, m, w, b, g = c["x"], c["sample_map"], c["weight"], c["bias"], c["grad_output"]
    y = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(w), _t(b), K, it))
    assert relerr(y, oracle.mapped_conv_forward(x, m, w, b, K, it, iw)) <= FWD
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(w), _t(b), K, it)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, it, iw)
    assert relerr(_n(gi), wi) <= BWD
    assert relerr(_n(gw), ww) <= BWD
    assert relerr(_n(gb), wb) <= BWD


def test_configuration1_full_size(ops, oracle):
    """x [1,3,64,128] -> 16 channels, K = 9 gnomonic map, bilinear, zero bias."""
    _conv_both_ways(ops, oracle, workloads.config1())


def test_configuration2_reduced(ops, oracle):
    """Tangent patches (80 faces, 16 x 16 samples) on a 128 x 256 image: gather, scatter back,
    weight-sum normalisation (epsilon as layers/functional/sphere_ops.py:74-80)."""
    c = workloads.config2(batch=2, H=128, W=256, patch=16)
    x, m, it = c["x"], c["sample_map"], c["interp"]
    H, W = c["out_shape"]
    patches = _n(ops.resample_from_map(_t(x), _t(m), None, it))
    want = oracle.resample_from_map(x, m, it)
    assert relerr(patches, want) <= FWD
    back = _n(ops.resample_to_map(_t(want), _t(m), None, H, W, it))
    want_back = oracle.resample_to_map(want, m, H, W, it)
    assert relerr(back, want_back) <= BWD
    norm, wsum = ops.resample_to_map_normalized(_t(want), _t(m), None, H, W, it, 1e-12)
    want_sum = oracle.resample_to_map(np.ones((1, 1) + want.shape[2:], np.float32), m, H, W, it)[0, 0]
    assert relerr(_n(wsum), want_sum) <= BWD
    # non-negative weights: the quotient's error stays at n * eps * max|value| (scatter bound)
    assert relerr(_n(norm), want_back / (want_sum + np.float32(1e-12))) <= BWD
    # nearest-neighbour gather: bit-exact
    near = _n(ops.resample_from_map(_t(x), _t(m), None, 0))
    assert np.array_equal(near, oracle.resample_from_map(x, m, 0))


def test_configuration3_reduced(ops, oracle):
    """Stride-2 gnomonic 3 x 3 max pool, nearest: values and indices bit-exact, unpool with and
    without its workspace."""
    c = workloads.config3(batch=2, channels=5, H=64, W=128)
    x, m, g = c["x"], c["sample_map"], c["grad_output"]
    K, it = c["kernel_size"], c["interp"]
    val, idx = ops.mapped_max_pool(_t(x), _t(m), None, K, it)
    wval, widx = oracle.mapped_max_pool(x, m, K, it)
    assert np.array_equal(_n(idx), widx)
    assert np.array_equal(_n(val), wval)
    want = oracle.mapped_max_unpool(g, widx, m, x.shape[2], x.shape[3], K, it)
    for with_ws in (True, False):
        ops.set_unpool_workspace(with_ws)
        try:
            got = _n(ops.mapped_max_unpool(_t(g), idx, _t(m), None, x.shape[2], x.shape[3], K, it))
        finally:
            ops.set_unpool_workspace(True)
        assert relerr(got, want) <= BWD


def test_configuration4_reduced(ops, oracle):
    """Weighted (P = 4) bispherical convolution on a 32 x 64 grid, 40 -> 24 channels."""
    _conv_both_ways(ops, oracle, workloads.config4(batch=2, cin=40, cout=24, H=32, W=64))


@pytest.mark.parametrize("order", ["hierarchical", "append"])
def test_configuration5_reduced(ops, oracle, order):
    """Level-3 icosphere (642 vertices): vertex convolution and transposed up-sampling from
    level 2, nearest; with the vertices numbered for locality and in subdivision order."""
    c = workloads.config5(batch=2, channels=16, level=3, order=order)
    _conv_both_ways(ops, oracle, c)
    K, it = c["kernel_size"], c["interp"]
    xc, um, uw, ub = c["x_coarse"], c["up_map"], c["up_weight"], c["up_bias"]
    OH, OW = c["out_hw"]
    yt = _n(ops.mapped_transposed_conv_forward(_t(xc), _t(um), None, _t(uw), _t(ub), OH, OW, K, it))
    want = oracle.mapped_transposed_conv_forward(xc, um, uw, ub, OH, OW, K, it)
    assert relerr(yt, want) <= BWD      # the forward of the transposed layer is the scatter
    gt = np.random.default_rng(55).standard_normal(want.shape).astype(np.float32)
    gi, gw, gb = ops.mapped_transposed_conv_backward(_t(gt), _t(um), None, _t(xc), _t(uw), _t(ub),
                                                     K, it)
    wi, ww, wb = oracle.mapped_transposed_conv_backward(gt, um, xc, uw, ub, K, it)
    assert relerr(_n(gi), wi) <= BWD
    assert relerr(_n(gw), ww) <= BWD
    assert relerr(_n(gb), wb) <= BWD
