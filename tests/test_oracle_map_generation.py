"""Pins the oracle's sample-map generators by what the geometry fixes, independently of the
formulas they restate: closed forms in pixel units, the forward gnomonic projection (textbook
formula, the inverse of the one the generator uses) giving back every sample's tangent-plane
offset, the centre sample, stride as sub-sampling, and float32 against float64.
"""
import math

import numpy as np
import pytest

SHAPES = [((16, 32), (3, 3), 1, 1), ((33, 47), (3, 5), 1, 2), ((24, 40), (2, 2), 2, 1),
          ((20, 64), (5, 3), 3, 1)]


def _sphere(xy, H, W):
    """Pixel coordinates -> unit vectors (lon = -pi + 2 pi x / W, lat = -pi/2 + pi y / (H-1))."""
    lon = -math.pi + 2 * math.pi * xy[..., 0] / W
    lat = -math.pi / 2 + math.pi * xy[..., 1] / (H - 1)
    return lon, lat


def _offsets(kh, kw, dilation):
    i, j = np.meshgrid(np.arange(kh) - kh // 2, np.arange(kw) - kw // 2, indexing="ij")
    return i.reshape(-1) * dilation, j.reshape(-1) * dilation


@pytest.mark.parametrize("shape,ks,stride,dilation", SHAPES)
def test_grid_map_is_the_pixel_plus_integer_offsets(oracle, shape, ks, stride, dilation):
    H, W = shape
    m = oracle.equirect_kernel_map(shape, ks, stride, dilation, oracle.GRID, np.float64)
    oi, oj = _offsets(ks[0], ks[1], dilation)
    ys, xs = np.arange(0, H, stride), np.arange(0, W, stride)
    want_x = xs[None, :, None] + oj[None, None, :]
    want_y = ys[:, None, None] - oi[None, None, :]     # rows of the kernel run against latitude
    assert m.shape == (len(ys), len(xs), ks[0] * ks[1], 2)
    assert np.abs(m[..., 0] - want_x).max() < 1e-9
    assert np.abs(m[..., 1] - want_y).max() < 1e-9


@pytest.mark.parametrize("shape,ks,stride,dilation", SHAPES)
def test_inverse_equirectangular_widens_the_longitude_step(oracle, shape, ks, stride, dilation):
    H, W = shape
    m = oracle.equirect_kernel_map(shape, ks, stride, dilation, oracle.INVERSE_EQUIRECTANGULAR,
                                   np.float64)
    oi, oj = _offsets(ks[0], ks[1], dilation)
    ys, xs = np.arange(0, H, stride), np.arange(0, W, stride)
    want_y = ys[:, None, None] - oi[None, None, :] + 0 * xs[None, :, None]
    lat = -math.pi / 2 + math.pi * want_y / (H - 1)
    want_x = np.mod(xs[None, :, None] + oj[None, None, :] / np.cos(lat), W)
    assert np.abs(m[..., 1] - want_y).max() < 1e-9
    d = np.abs(m[..., 0] - want_x)
    ok = np.abs(np.cos(lat)) > 1e-6                    # at the poles the step is unbounded
    assert np.minimum(d, W - d)[ok].max() < 1e-6


@pytest.mark.parametrize("shape,ks,stride,dilation", SHAPES)
def test_forward_gnomonic_projection_returns_the_kernel_offsets(oracle, shape, ks, stride,
                                                                dilation):
    """x = cos(lat) sin(dlon) / c, y = (cos(lat0) sin(lat) - sin(lat0) cos(lat) cos(dlon)) / c,
    c = sin(lat0) sin(lat) + cos(lat0) cos(lat) cos(dlon): applied to every sample of the
    inverse-gnomonic map it must give the kernel's tangent-plane grid."""
    H, W = shape
    m = oracle.equirect_kernel_map(shape, ks, stride, dilation, oracle.INVERSE_GNOMONIC,
                                   np.float64)
    lon, lat = _sphere(m, H, W)
    ys, xs = np.arange(0, H, stride), np.arange(0, W, stride)
    lon0 = (-math.pi + 2 * math.pi * xs / W)[None, :, None]
    lat0 = (-math.pi / 2 + math.pi * ys / (H - 1))[:, None, None]
    c = np.sin(lat0) * np.sin(lat) + np.cos(lat0) * np.cos(lat) * np.cos(lon - lon0)
    px = np.cos(lat) * np.sin(lon - lon0) / c
    py = (np.cos(lat0) * np.sin(lat) - np.sin(lat0) * np.cos(lat) * np.cos(lon - lon0)) / c
    oi, oj = _offsets(ks[0], ks[1], dilation)
    want_x = oj * (2 * math.pi / W) + 0 * px
    want_y = -oi * (math.pi / (H - 1)) + 0 * py
    K = ks[0] * ks[1]
    # the sample at index K // 2 is set to the pixel itself whatever its offset; that is the
    # zero-offset sample only for odd x odd kernels, otherwise the zero-offset sample keeps the
    # 0 / 0 of its projection in y (the reference's behaviour, mapping_functions.py:99-108)
    want_x[..., K // 2] = 0
    want_y[..., K // 2] = 0
    zero = (ks[0] // 2) * ks[1] + ks[1] // 2
    if zero != K // 2:
        assert np.isnan(m[..., zero, 1]).all()      # asin(0 / 0); atan2(0, 0) = 0 keeps x
        px[..., zero] = py[..., zero] = want_x[..., zero] = want_y[..., zero] = 0
        m = np.delete(m, zero, axis=2)
    assert not np.isnan(m).any()
    assert np.abs(px - want_x).max() < 1e-9
    assert np.abs(py - want_y).max() < 1e-9
    m = oracle.equirect_kernel_map(shape, ks, stride, dilation, oracle.INVERSE_GNOMONIC,
                                   np.float64)
    centre = m[..., K // 2, :]
    assert np.abs(centre[..., 0] - xs[None, :]).max() < 1e-9
    assert np.abs(centre[..., 1] - ys[:, None]).max() < 1e-9
    ok = ~np.isnan(m[..., 0])
    assert (m[..., 0][ok] >= 0).all() and (m[..., 0][ok] <= W).all()


@pytest.mark.parametrize("proj", [0, 1, 2])
def test_stride_is_subsampling_and_float32_follows_float64(oracle, proj):
    shape, ks = (30, 52), (3, 3)
    full = oracle.equirect_kernel_map(shape, ks, 1, 1, proj, np.float64)
    sub = oracle.equirect_kernel_map(shape, ks, 4, 1, proj, np.float64)
    assert np.array_equal(sub, full[::4, ::4])
    f32 = oracle.equirect_kernel_map(shape, ks, 1, 1, proj, np.float32)
    # compared as points on the sphere: near the poles a longitude is ill-conditioned, and so is
    # the arcsine that gives a latitude within a degree of a pole (error ~ 1e-7 / cos(lat))
    d = _sphere_distance(f32.astype(np.float64), full, *shape)
    away = np.abs(_sphere(full, *shape)[1]) < 1.4
    assert d[away].max() < 2e-6
    assert d.max() < 5e-4


def _sphere_distance(a, b, H, W):
    la, pa = _sphere(a, H, W)
    lb, pb = _sphere(b, H, W)
    va = np.stack([np.cos(pa) * np.cos(la), np.cos(pa) * np.sin(la), np.sin(pa)], -1)
    vb = np.stack([np.cos(pb) * np.cos(lb), np.cos(pb) * np.sin(lb), np.sin(pb)], -1)
    return np.linalg.norm(va - vb, axis=-1)


@pytest.mark.parametrize("kh,kw", [(3, 3), (4, 4), (2, 5)])
def test_gnomonic_kernel_about_points(oracle, kh, kw):
    """Forward projection of every sample about its own centre gives the kernel grid (even
    kernels are centred between samples); the pixel form is the spherical form rescaled."""
    rng = np.random.default_rng(3)
    n = 50
    pts = np.stack([rng.uniform(-math.pi, math.pi, n), rng.uniform(-1.4, 1.4, n)], -1)
    rl, ro = 0.03, 0.04
    out = oracle.gnomonic_kernel_at(pts, kh, kw, rl, ro)
    lon, lat = out[..., 0], out[..., 1]
    lon0, lat0 = pts[:, None, 0], pts[:, None, 1]
    c = np.sin(lat0) * np.sin(lat) + np.cos(lat0) * np.cos(lat) * np.cos(lon - lon0)
    px = np.cos(lat) * np.sin(lon - lon0) / c
    py = (np.cos(lat0) * np.sin(lat) - np.sin(lat0) * np.cos(lat) * np.cos(lon - lon0)) / c
    i, j = np.meshgrid(np.arange(kh) - kh // 2, np.arange(kw) - kw // 2, indexing="ij")
    want_x = j.reshape(-1) * ro + (ro / 2 if kw % 2 == 0 else 0)
    want_y = i.reshape(-1) * rl + (rl / 2 if kh % 2 == 0 else 0)
    assert np.abs(px - want_x[None]).max() < 1e-9
    assert np.abs(py - want_y[None]).max() < 1e-9
    assert (lon >= -math.pi).all() and (lon < math.pi + 1e-12).all()
    H, W = 40, 90
    pix = oracle.gnomonic_kernel_at(pts, kh, kw, rl, ro, (H, W))
    assert np.abs(pix[..., 0] - W * (lon + math.pi) / (2 * math.pi)).max() < 1e-9
    assert np.abs(pix[..., 1] - (H - 1) * (lat + math.pi / 2) / math.pi).max() < 1e-9


@pytest.mark.parametrize("shape,ks,stride,dilation", SHAPES)
def test_float32_grid_map_matches_the_tensor_library_to_the_last_bits(oracle, shape, ks, stride,
                                                                      dilation):
    """The float32 map is built from tensor operations whose rounding the oracle imitates with
    scalars (evenly spaced values computed from the nearer end, Python scalars rounded to
    float32 before they meet a tensor).  The grid projection has no transcendental function in
    it, so the tensor library itself must agree to rounding: its evenly spaced values are
    computed in vector chunks whose width depends on the host CPU, so the last bit of a longitude
    is not fixed by the reference either; two units in the last place of the image size
    cover it."""
    import torch
    H, W = shape
    kh, kw = ks
    lon = torch.linspace(-math.pi, math.pi, steps=W + 1)[:-1].view(1, W, 1)
    lat = torch.linspace(-math.pi / 2, math.pi / 2, steps=H).view(H, 1, 1)
    oi, oj = _offsets(kh, kw, dilation)
    dlon = torch.tensor([float(j) * (2 * math.pi / W) for j in oj], dtype=torch.float32)
    dlat = torch.tensor([float(i) * -(math.pi / (H - 1)) for i in oi], dtype=torch.float32)
    x = W * ((lon + dlon.view(1, 1, -1)) - (-math.pi)) / (math.pi - (-math.pi))
    y = (H - 1) * ((lat + dlat.view(1, 1, -1)) - (-math.pi / 2)) / (math.pi / 2 - (-math.pi / 2))
    x, y = torch.broadcast_tensors(x, y)
    want = torch.stack([x, y], -1)[::stride, ::stride].numpy()
    got = oracle.equirect_kernel_map(shape, ks, stride, dilation, oracle.GRID, np.float32)
    assert np.abs(got - want).max() <= 2 * np.spacing(np.float32(max(H, W)))
