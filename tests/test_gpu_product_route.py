"""The inverse direction (transposed forward, backward-input) of maps with single nearest taps
whose image has at least twice the pixels of their grid: a matrix product at the grid's
resolution, then a gather of the products over the inverted map.  Against the oracle at the
float32 backward tolerance (1e-4 of the largest value), on shapes that cut the kernels' tiles
(pixel counts, columns (k, c), channel counts on either side), maps with taps outside the image,
image elements no tap reaches, and elements that collect hundreds of taps; planned against
plain calls and call against call bit for bit (sums in list order, no atomics).
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
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _n(t):
    return t.detach().cpu().numpy()


def _map(rng, OH, OW, K, H, W, kind):
    if kind == "spread":      # anywhere in the image and a little outside it
        xy = rng.uniform(-1.5, [W + 0.5, H + 0.5], size=(OH, OW, K, 2))
    elif kind == "crowded":   # nearly every sample lands in one corner of 3 x 3 elements
        xy = rng.uniform(-0.4, 2.4, size=(OH, OW, K, 2))
        far = rng.uniform(size=(OH, OW, K)) < 0.05
        xy[far] = rng.uniform(0, [W - 1, H - 1], size=(int(far.sum()), 2))
    else:                     # an up-sampling grid: sample k of pixel (y, x) near (2 y, 2 x)
        ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
        dx = rng.integers(-1, 2, size=(OH, OW, K))
        dy = rng.integers(-1, 2, size=(OH, OW, K))
        xy = np.stack([xs[..., None] * (W / OW) + dx, ys[..., None] * (H / OH) + dy], -1)
        xy = xy + rng.uniform(-0.3, 0.3, size=xy.shape)
    return np.ascontiguousarray(xy.astype(np.float32))


# (image channels, grid channels, H, W, OH, OW, K, B, map)
CASES = [
    (24, 40, 20, 36, 10, 18, 7, 3, "grid"),      # every tile cut: 180 pixels, 168 columns, 40 rows
    (64, 64, 32, 64, 16, 32, 9, 2, "grid"),      # 4 pixel tiles, 4.5 column tiles
    (72, 16, 24, 24, 12, 12, 4, 1, "spread"),    # two channel chunks in the gather, one row chunk
    (5, 64, 9, 33, 4, 16, 3, 2, "spread"),       # the fewest image channels the route takes
    (33, 48, 16, 40, 8, 40, 9, 2, "crowded"),    # hundreds of taps on a few elements
    (128, 32, 40, 20, 20, 10, 1, 2, "grid"),     # one sample per pixel
]


@pytest.mark.parametrize("tc", CASES, ids=lambda t: "x".join(map(str, t)))
def test_products_then_gather_match_the_oracle(ops, oracle, tc):
    Cg, Cp, H, W, OH, OW, K, B, kind = tc
    rng = np.random.default_rng(sum(tc[:8]))
    m = _map(rng, OH, OW, K, H, W, kind)
    tm = _t(m)
    # transposed layer: input on the grid (Cp channels), output the image (Cg channels)
    x = rng.standard_normal((B, Cp, OH, OW)).astype(np.float32)
    w = (rng.standard_normal((Cp, Cg, K)) / np.sqrt(Cp * K)).astype(np.float32)
    b = rng.standard_normal(Cg).astype(np.float32)
    want = oracle.mapped_transposed_conv_forward(x, m, w, b, H, W, K, 0, None)
    got = {}
    for cached in (False, True):
        ops.set_conv_plan_cache(cached)
        try:
            for rep in range(2):
                got[(cached, rep)] = _n(ops.mapped_transposed_conv_forward(
                    _t(x), tm, None, _t(w), _t(b), H, W, K, 0))
        finally:
            ops.set_conv_plan_cache(True)
    assert relerr(got[(True, 1)], want) <= 1e-4
    for key, val in got.items():
        assert np.array_equal(val, got[(True, 1)]), key
    # convolution over the same map (image Cg channels -> grid Cp channels): backward-input
    xi = rng.standard_normal((B, Cg, H, W)).astype(np.float32)
    wc = (rng.standard_normal((Cp, Cg, K)) / np.sqrt(Cg * K)).astype(np.float32)
    bc = rng.standard_normal(Cp).astype(np.float32)
    g = rng.standard_normal((B, Cp, OH, OW)).astype(np.float32)
    gi, gw, gb = ops.mapped_conv_backward(_t(g), tm, None, _t(xi), _t(wc), _t(bc), K, 0)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, xi, wc, bc, K, 0, None)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4 and relerr(_n(gb), wb) <= 1e-4
    gi2, _, _ = ops.mapped_conv_backward(_t(g), tm, None, _t(xi), _t(wc), _t(bc), K, 0)
    assert np.array_equal(_n(gi2), _n(gi))
