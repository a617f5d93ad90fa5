"""Pooling from a kept plan (sdk_mapped_max_pool_planned / sdk_mapped_avg_pool_planned: tiles
inside their window pool from LDS, the others in the per-pixel kernel over their list) against
the plain entry points and the oracle: identical values and indices, on maps whose tiles take
both routes, with samples outside the image, ties, NaN and planes where no sample wins.
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _map(seed, OH, OW, K, H, W, kind):
    rng = np.random.default_rng(seed)
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / K
    cx = xs[..., None] * (W / OW) + 1.3 * np.cos(ang)
    cy = ys[..., None] * (H / OH) + 1.3 * np.sin(ang)
    if kind == "polar":      # rows near the top spread their samples wide, as near a pole
        spread = 1.0 + 40.0 / (1.0 + ys[..., None])
        cx = xs[..., None] * (W / OW) + spread * 1.3 * np.cos(ang)
    if kind == "outside":    # a band of samples beyond the image: they read as 0
        cx = cx - 3.0
        cy = cy - 2.0
    if kind == "integer":    # integer coordinates: bilinear weights of exactly 0 and 1, ties
        cx, cy = np.round(cx), np.round(cy)
    else:
        cx = cx + rng.uniform(-0.3, 0.3, cx.shape)
        cy = cy + rng.uniform(-0.3, 0.3, cy.shape)
    return np.ascontiguousarray(np.stack([cx, cy], -1).astype(np.float32))


# (OH, OW, K, H, W, kind)
CASES = [
    (32, 64, 9, 64, 128, "plain"),
    (40, 48, 9, 80, 96, "polar"),
    (24, 40, 5, 48, 80, "outside"),
    (16, 48, 9, 32, 96, "integer"),
    (19, 23, 4, 37, 45, "plain"),       # ragged tiles
    (1, 300, 7, 1, 600, "plain"),       # one row
]


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("tc", CASES, ids=lambda t: "x".join(map(str, t)))
def test_planned_pooling_is_the_plain_pooling(ops, oracle, tc, interp):
    OH, OW, K, H, W, kind = tc
    m = _map(sum(tc[:5]) + interp, OH, OW, K, H, W, kind)
    rng = np.random.default_rng(3)
    x = rng.standard_normal((2, 37, H, W)).astype(np.float32)
    x[0, 0] = -1.0                          # with samples outside the image (0) winning
    x[0, 1] = np.round(x[0, 1])             # ties
    x[1, 2, ::3, ::5] = np.nan              # NaN never wins
    x[1, 3] = np.nan                        # ... and a plane where no sample wins
    x[1, 4, 1::2] = -np.inf
    tx, tm = _t(x), _t(m)
    ops.set_conv_plan_cache(False)
    try:
        v0, i0 = ops.mapped_max_pool(tx, tm, None, K, interp)
        a0 = ops.mapped_avg_pool(tx, tm, None, K, interp)
    finally:
        ops.set_conv_plan_cache(True)
    v1, i1 = ops.mapped_max_pool(tx, tm, None, K, interp)
    a1 = ops.mapped_avg_pool(tx, tm, None, K, interp)
    assert torch.equal(i0, i1)
    assert torch.equal(torch.nan_to_num(v0, nan=7.0), torch.nan_to_num(v1, nan=7.0))
    assert torch.equal(torch.isnan(a0), torch.isnan(a1))
    assert torch.equal(torch.nan_to_num(a0, nan=7.0), torch.nan_to_num(a1, nan=7.0))
    # against the oracle on the finite batch element (under a zero interpolation weight the
    # reference turns Inf / NaN into NaN, this library skips the tap)
    want_v, want_i = oracle.mapped_max_pool(x[:1], m, K, interp, None)
    assert np.array_equal(i1[:1].cpu().numpy(), want_i)
    assert np.allclose(v1[:1].cpu().numpy(), want_v, rtol=0, atol=0 if interp == 0 else 1e-6)
    want_a = oracle.mapped_avg_pool(x[:1], m, K, interp, None)
    assert np.allclose(a1[:1].cpu().numpy(), want_a, rtol=0, atol=1e-6)


def test_planned_pooling_backward_through_the_layers(ops, oracle):
    """The autograd path (max pool forward from the plan, unpool backward) on a coherent map."""
    from spherical_distortion import nn as sdnn
    OH, OW, K, H, W = 32, 64, 9, 64, 128
    m = _map(11, OH, OW, K, H, W, "plain")
    x = np.random.default_rng(4).standard_normal((2, 8, H, W)).astype(np.float32)
    tx = _t(x).requires_grad_(True)
    y = sdnn.MappedMaxPool(K, 1)(tx, _t(m))
    g = np.random.default_rng(5).standard_normal(y.shape).astype(np.float32)
    y.backward(_t(g))
    _, want_i = oracle.mapped_max_pool(x, m, K, 1, None)
    want = oracle.mapped_max_unpool(g, want_i, m, H, W, K, 1, None)
    got = tx.grad.cpu().numpy()
    assert np.abs(got - want).max() <= 1e-5 * np.abs(want).max()
