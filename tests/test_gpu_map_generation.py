"""GPU parity of the on-device sample-map generators against the CPU oracle.

A map holds coordinates computed with sin / cos / atan / asin / atan2; the device's and the
host's float32 versions of these differ in the last bits, and two spots amplify that: the
longitude of a point next to a pole, and the arcsine that yields a latitude within a degree of
a pole (error ~ 1e-7 / cos(lat)).  Maps are therefore compared as points on the sphere:
float64 to 1e-11 rad, float32 to 2e-6 rad away from the poles and 5e-4 rad next to them; the
grid projection, which has no transcendental function, bit for bit; NaN (the zero-offset
sample of even kernels, as in the reference) in the same places.
"""
import math

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TORCH = {np.float32: torch.float32, np.float64: torch.float64}


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _sphere(xy, H, W):
    lon = -math.pi + 2 * math.pi * xy[..., 0] / W
    lat = -math.pi / 2 + math.pi * xy[..., 1] / (H - 1)
    return lon, lat


def _distance(a, b, H, W):
    la, pa = _sphere(a.astype(np.float64), H, W)
    lb, pb = _sphere(b.astype(np.float64), H, W)
    va = np.stack([np.cos(pa) * np.cos(la), np.cos(pa) * np.sin(la), np.sin(pa)], -1)
    vb = np.stack([np.cos(pb) * np.cos(lb), np.cos(pb) * np.sin(lb), np.sin(pb)], -1)
    return np.linalg.norm(va - vb, axis=-1)


def _same_map(got, want, H, W, dt):
    assert got.shape == want.shape and got.dtype == want.dtype
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    ok = ~nan.any(-1)
    d = _distance(got[ok], want[ok], H, W)
    if dt == np.float64:
        assert d.max() < 1e-11
    else:
        away = np.abs(_sphere(want[ok].astype(np.float64), H, W)[1]) < 1.4
        assert d[away].max() < 2e-6
        assert d.max() < 5e-4


CASES = [((16, 32), (3, 3), 1, 1), ((33, 47), (3, 5), 1, 2), ((24, 40), (2, 2), 2, 1),
         ((20, 64), (5, 3), 3, 1), ((64, 128), (1, 1), 1, 1), ((37, 90), (4, 3), 2, 3)]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("proj", [0, 1, 2])
@pytest.mark.parametrize("shape,ks,stride,dilation", CASES)
def test_equirect_kernel_maps(ops, oracle, shape, ks, stride, dilation, proj, dt):
    got = ops.equirect_kernel_map(shape[0], shape[1], ks[0], ks[1], stride, dilation, proj,
                                  TORCH[dt], DEV).cpu().numpy()
    want = oracle.equirect_kernel_map(shape, ks, stride, dilation, proj, dt)
    if proj == 0:
        assert np.array_equal(got, want)
    _same_map(got, want, shape[0], shape[1], dt)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("kh,kw", [(3, 3), (4, 4), (2, 5), (16, 16)])
def test_gnomonic_kernels_about_points(ops, oracle, kh, kw, dt):
    rng = np.random.default_rng(11)
    n = 333
    pts = np.stack([rng.uniform(-math.pi, math.pi, n), rng.uniform(-1.5, 1.5, n)], -1).astype(dt)
    pts[:3] = [[0.0, 0.0], [-math.pi, 0.3], [1.0, -1.2]]
    rl, ro = 0.013, 0.017
    H, W = 80, 170
    want = oracle.gnomonic_kernel_at(pts, kh, kw, rl, ro, (H, W))
    got = ops.gnomonic_kernel_at(torch.from_numpy(pts).to(DEV), kh, kw, rl, ro, H, W).cpu().numpy()
    _same_map(got, want, H, W, dt)
    # spherical output: the same points before the change of units
    sph = ops.gnomonic_kernel_at(torch.from_numpy(pts).to(DEV), kh, kw, rl, ro).cpu().numpy()
    want_sph = oracle.gnomonic_kernel_at(pts, kh, kw, rl, ro)
    tol = 1e-11 if dt == np.float64 else 5e-4
    dl = np.abs(sph[..., 0] - want_sph[..., 0])
    assert (np.minimum(dl, 2 * math.pi - dl) * np.cos(want_sph[..., 1])).max() < tol
    assert np.abs(sph[..., 1] - want_sph[..., 1]).max() < tol


def test_generated_map_drives_the_mapped_convolution(ops, oracle):
    """End to end in float64: a convolution over the device-generated inverse-gnomonic map
    equals the oracle's convolution over the oracle's map."""
    H, W, K = 24, 48, 9
    rng = np.random.default_rng(5)
    x = rng.standard_normal((2, 5, H, W))
    w = rng.standard_normal((7, 5, K)) / 7
    b = rng.standard_normal(7)
    m = ops.equirect_kernel_map(H, W, 3, 3, 1, 1, 1, torch.float64, DEV)
    y = ops.mapped_conv_forward(torch.from_numpy(x).to(DEV), m, None, torch.from_numpy(w).to(DEV),
                                torch.from_numpy(b).to(DEV), K, 2).cpu().numpy()
    want = oracle.mapped_conv_forward(x, oracle.equirect_kernel_map((H, W), (3, 3), 1, 1, 1,
                                                                    np.float64), w, b, K, 2)
    assert np.abs(y - want).max() <= 1e-9 * np.abs(want).max()


def test_python_builders_and_errors(ops):
    """The builders carry the reference's names and layouts (layers/util/mapping_functions.py)."""
    import spherical_distortion.util as util
    m = util.inverse_gnomonic_projection_map((32, 64), (3, 3), stride=2)
    assert m.shape == (16, 32, 9, 2) and m.dtype == torch.float32 and m.is_cuda
    assert torch.equal(m, util.inverse_gnomonic_projection_map((32, 64), (3, 3))[::2, ::2])
    g = util.grid_projection_map((32, 64), (3, 3), dilation=2)
    assert torch.allclose(g[5, 7, 4], torch.tensor([7.0, 5.0], device=DEV), atol=1e-5)
    # (x - 2, y + 2): rows of the kernel run against latitude
    assert torch.allclose(g[5, 7, 0], torch.tensor([5.0, 7.0], device=DEV), atol=1e-5)
    e = util.inverse_equirectangular_projection_map((32, 64), (1, 3))
    assert e.shape == (32, 64, 3, 2)
    pts = torch.tensor([[0.1, 0.2], [1.0, -0.5]], device=DEV)
    k = util.gnomonic_kernel(pts, 3, 3, 0.01, 0.02)
    assert k.shape == (1, 2, 9, 2)
    assert torch.allclose(k[0, :, 4], pts)
    p = util.gnomonic_kernel_pixels(pts, 3, 3, 0.01, 0.02, (32, 64))
    assert p.shape == (2, 9, 2)
    with pytest.raises(RuntimeError, match="height"):
        ops.equirect_kernel_map(1, 64, 3, 3)
    with pytest.raises(RuntimeError, match="GPU only"):
        ops.equirect_kernel_map(32, 64, 3, 3, device="cpu")
    with pytest.raises(RuntimeError, match="projection"):
        ops.equirect_kernel_map(32, 64, 3, 3, projection=5)
    with pytest.raises(RuntimeError, match="lonlat"):
        ops.gnomonic_kernel_at(torch.zeros(4, 3, device=DEV), 3, 3, 0.1, 0.1)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_four_nearest_weighted_map_against_its_definition(ops, dtype):
    """The weighted (P = 4) form of a map: integer neighbours bit for bit, weights against the
    float64 arccosine form of the same definition.  A sample that coincides with a pixel centre
    has distance 0 there, where arccos(1 - 1e-16) = 1.5e-8 against eps = 1e-6 moves the other
    three weights (~1e-4 each) in the sixth digit: hence 5e-6 for float64; float32 coordinates
    carry ~1e-7 rad of their own, 5e-5."""
    import workloads as wl
    H, W = 24, 48
    base = wl.gnomonic_kernel_map(H, W, dtype=np.float64)
    rng = np.random.default_rng(5)
    extra = np.stack([rng.uniform(-3, W + 3, (H, W, 9)), rng.uniform(-2, H + 1, (H, W, 9))], -1)
    for m in (base, extra):
        m = m.astype(dtype)
        want_m, want_w = wl.four_nearest_weighted(m, H, W, dtype=np.float64)
        got_m, got_w = ops.four_nearest_weighted_map(torch.from_numpy(m).to(DEV), H, W)
        assert got_m.shape == m.shape[:-1] + (4, 2) and got_w.shape == m.shape[:-1] + (4,)
        assert np.array_equal(got_m.cpu().numpy().astype(np.float64), want_m)
        tol = 5e-6 if dtype == np.float64 else 5e-5
        assert np.abs(got_w.cpu().numpy() - want_w).max() < tol
        assert np.abs(got_w.sum(-1).cpu().numpy() - 1).max() < 1e-6
    empty = torch.empty(0, 2, device=DEV, dtype=TORCH[dtype])
    assert ops.four_nearest_weighted_map(empty, H, W)[1].shape == (0, 4)


def test_four_nearest_weighted_map_feeds_the_weighted_convolution(ops):
    """The util front-end end to end: map built on the device, then the weighted convolution on
    it equals the one on the host-built map."""
    import workloads as wl
    from spherical_distortion.util import four_nearest_weighted
    H, W, C = 16, 32, 4
    base = wl.gnomonic_kernel_map(H, W, dtype=np.float32)
    hm, hw = wl.four_nearest_weighted(base, H, W)
    dm, dw = four_nearest_weighted(torch.from_numpy(base).to(DEV), (H, W))
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, C, H, W, generator=g).to(DEV)
    wt = torch.randn(C, C, 9, generator=g).to(DEV)
    b = torch.zeros(C, device=DEV)
    a = ops.mapped_conv_forward(x, dm, dw, wt, b, 9, 2)
    r = ops.mapped_conv_forward(x, torch.from_numpy(hm).to(DEV), torch.from_numpy(hw).to(DEV),
                                wt, b, 9, 2)
    assert (a - r).abs().max().item() < 1e-3 * r.abs().max().item()
