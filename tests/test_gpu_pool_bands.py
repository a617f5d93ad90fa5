"""The row-band pooling kernels (float32, single nearest taps, K = 4 or 9, at least 16 planes,
image width a multiple of 4) against the oracle: values and indices bit for bit, on shapes
chosen so that every route of the kernel runs.  A workgroup owns R rows of the pooled grid
(R = the largest of 8, 4, 2, 1 with at most 1024 pooled pixels whose expected input rows,
R * s + 2 * s + 1 for a row stride s, fit 52 KB of LDS), finds the input rows its taps touch
and stages them for two planes per pass when they fit twice, for one plane when they fit
once, and reads its taps from global memory otherwise.
"""
import numpy as np
import pytest
import torch

import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _grid_map(OH, OW, sx, sy, K, spread_y, rng, jitter=0.3):
    """Kernel of K samples around (sx * ox, sy * oy) whose rows spread over +- spread_y."""
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / K
    cx = xs[..., None] * sx + 2.0 * np.cos(ang)
    cy = ys[..., None] * sy + spread_y * np.sin(ang)
    m = np.stack([cx, cy], -1) + rng.uniform(-jitter, jitter, (OH, OW, K, 2))
    return np.ascontiguousarray(m.astype(np.float32))


def _check(ops, oracle, x, m, K):
    val, idx = ops.mapped_max_pool(_t(x), _t(m), None, K, 0)
    avg = ops.mapped_avg_pool(_t(x), _t(m), None, K, 0)
    torch.cuda.synchronize()
    wval, widx = oracle.mapped_max_pool(x, m, K, 0)
    assert np.array_equal(idx.cpu().numpy(), widx)
    assert np.array_equal(val.cpu().numpy(), wval, equal_nan=True)
    assert np.array_equal(avg.cpu().numpy(), oracle.mapped_avg_pool(x, m, K, 0), equal_nan=True)
    return val, idx


# (B, C, H, W, OH, OW, sx, sy, K, spread_y, what)
CASES = [
    (2, 9, 32, 64, 16, 32, 2, 2, 9, 2.0, "R = 8, two pooled pixels per thread, two planes per pass"),
    (1, 17, 64, 128, 32, 64, 2, 2, 9, 2.0, "R = 8, odd plane count split over eight chunks"),
    (2, 8, 48, 96, 48, 96, 1, 1, 9, 1.0, "stride 1: R = 8 (IPT = 3 -> 4), last band of 48 rows full"),
    (2, 10, 50, 100, 25, 50, 2, 2, 9, 2.0, "OH = 25: the last band has one row; 200 pixels per band row group"),
    (3, 7, 128, 512, 32, 64, 8, 4, 9, 4.0, "R = 4, 21 rows of 512: one plane per pass"),
    (2, 9, 96, 512, 24, 64, 8, 4, 9, 40.0, "bands of about 90 rows: taps from global memory"),
    (2, 9, 96, 512, 24, 64, 8, 4, 4, 3.0, "K = 4"),
    (2, 9, 40, 1024, 10, 1024, 1, 4, 9, 2.0, "OW = 1024: R = 1, four pooled pixels per thread"),
    (4, 64, 64, 128, 32, 64, 2, 2, 9, 2.0, "256 planes: several passes per workgroup"),
]


@pytest.mark.parametrize("tc", CASES, ids=lambda t: t[-1].split(":")[0].replace(" ", "_"))
def test_band_pooling_matches_the_oracle_bit_for_bit(ops, oracle, tc):
    B, C, H, W, OH, OW, sx, sy, K, spread, _ = tc
    rng = np.random.default_rng(B * 1000 + C * 10 + K)
    m = _grid_map(OH, OW, sx, sy, K, spread, rng)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    _check(ops, oracle, x, m, K)


def test_band_pooling_on_the_gnomonic_stride_two_map(ops, oracle):
    """The benchmark's map at a reduced size: polar rows and the wrap seam spread a kernel over
    the whole image width, which a row band holds by construction."""
    H, W = 64, 128
    m = workloads.gnomonic_kernel_map(H, W, stride=2, dilation=2)
    x = np.random.default_rng(3).standard_normal((2, 16, H, W)).astype(np.float32)
    _check(ops, oracle, x, m, 9)


def test_band_pooling_ties_nan_and_taps_outside_the_image(ops, oracle):
    rng = np.random.default_rng(5)
    B, C, H, W, OH, OW, K = 2, 9, 32, 64, 16, 32, 9
    m = _grid_map(OH, OW, 2, 2, K, 2.0, rng)
    m[0:3] -= 40.0                      # a whole band outside the image: no rows to stage
    m[5, :, 2:5, 0] = W + 7.5           # some taps outside in x
    m[9, 3:9, :, 1] = -3.0              # and some pixels wholly outside in y
    x = rng.integers(-2, 3, (B, C, H, W)).astype(np.float32)      # many ties
    x[0, 1, ::3, ::2] = np.nan
    x[1, 2] = -np.inf
    x[1, 3] = np.nan                    # a plane without any winner: index -1
    val, idx = _check(ops, oracle, x, m, K)
    assert int((idx[1, 3] == -1).sum()) > 0
    assert float(val[0, 0, 0].abs().max()) == 0.0   # outside taps read as zero


def test_band_pooling_leaves_other_shapes_to_the_per_pixel_kernel(ops, oracle):
    """Width not a multiple of 4, fewer than 16 planes, K = 5, bilinear taps: same results."""
    rng = np.random.default_rng(6)
    for (B, C, H, W, OH, OW, K) in [(2, 9, 30, 62, 15, 31, 9), (1, 3, 32, 64, 16, 32, 9),
                                    (2, 9, 32, 64, 16, 32, 5)]:
        m = _grid_map(OH, OW, 2, 2, K, 2.0, rng)
        x = rng.standard_normal((B, C, H, W)).astype(np.float32)
        _check(ops, oracle, x, m, K)
    m = _grid_map(16, 32, 2, 2, 9, 2.0, rng)
    x = rng.standard_normal((2, 9, 32, 64)).astype(np.float32)
    val, idx = ops.mapped_max_pool(_t(x), _t(m), None, 9, 1)
    wval, widx = oracle.mapped_max_pool(x, m, 9, 1)
    assert np.array_equal(idx.cpu().numpy(), widx)
    assert np.abs(val.cpu().numpy() - wval).max() <= 1e-5 * np.abs(wval).max()
