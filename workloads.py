"""Synthetic sample maps and tensors for the five benchmark configurations.

Used by bench.py and by the tests; numpy only (float64 internally, cast at the
end), deterministic.  Conventions follow the reference's map builders so the
access patterns are the ones its layers see:

  * equirectangular pixel <-> sphere: lon = -pi + 2*pi*x/W, lat = -pi/2 + pi*y/(H-1)
    (layers/util/conversions.py:33-76, layers/util/grids.py:5-25);
  * 3x3 inverse-gnomonic kernel about every pixel, tangent offsets
    (j*dlon, -i*dlat), centre sample = the pixel itself, longitude wrapped,
    stride by sub-sampling (layers/util/mapping_functions.py:78-120);
  * an icosphere's V vertices are a 1 x V image, sample = (vertex index, 0)
    (layers/util/icosahedron_functions.py:176, :228).
"""
import math

import numpy as np


# ----------------------------------------------------------------------------- equirectangular
def gnomonic_kernel_map(H, W, stride=1, dilation=1, clamp_lat=True, dtype=np.float32):
    """[H/stride, W/stride, 9, 2] (x, y) sample map of a 3x3 tangent-plane kernel."""
    lon = -math.pi + 2.0 * math.pi * np.arange(W, dtype=np.float64) / W
    lat = -math.pi / 2 + math.pi * np.arange(H, dtype=np.float64) / (H - 1)
    lon = lon[None, ::stride, None]
    lat = lat[::stride, None, None]
    res_lon, res_lat = 2.0 * math.pi / W, math.pi / (H - 1)
    ii, jj = np.meshgrid(np.arange(-1, 2), np.arange(-1, 2), indexing="ij")
    dx = (jj.reshape(-1) * dilation * res_lon)[None, None, :]
    dy = (ii.reshape(-1) * dilation * -res_lat)[None, None, :]
    rho = np.sqrt(dx * dx + dy * dy)
    rho_safe = np.where(rho == 0, 1.0, rho)
    nu = np.arctan(rho)
    out_lat = np.arcsin(np.clip(np.cos(nu) * np.sin(lat) + dy * np.sin(nu) * np.cos(lat) / rho_safe,
                                -1.0, 1.0))
    out_lon = lon + np.arctan2(dx * np.sin(nu),
                               rho * np.cos(lat) * np.cos(nu) - dy * np.sin(lat) * np.sin(nu))
    out_lat = np.broadcast_to(out_lat, out_lon.shape).copy()
    centre = 4
    out_lat[..., centre] = np.broadcast_to(lat[..., 0], out_lat[..., centre].shape)
    out_lon[..., centre] = np.broadcast_to(lon[..., 0], out_lon[..., centre].shape)
    out_lon = np.mod(out_lon + math.pi, 2.0 * math.pi) - math.pi
    x = W * (out_lon + math.pi) / (2.0 * math.pi)
    y = (H - 1) * (out_lat + math.pi / 2) / math.pi
    if clamp_lat:
        y = np.clip(y, 0.0, H - 1.0)
    return np.ascontiguousarray(np.stack([x, y], -1).astype(dtype))


def four_nearest_weighted(sample_map, H, W, eps=1e-6, dtype=np.float32):
    """For every (x, y) sample: the 4 surrounding pixel centres (integer
    coordinates, x wrapped, y clamped) and weights proportional to the inverse
    great-circle distance to them, normalised to sum to one.
    -> (map [..., 4, 2], weights [..., 4])."""
    m = sample_map.astype(np.float64)
    x, y = m[..., 0], m[..., 1]
    x1 = np.floor(x)
    y1 = np.clip(np.floor(y), 0, H - 1)
    xs = np.stack([x1, x1 + 1, x1, x1 + 1], -1)
    ys = np.stack([y1, y1, np.clip(y1 + 1, 0, H - 1), np.clip(y1 + 1, 0, H - 1)], -1)
    xs = np.mod(xs, W)

    def to_sphere(px, py):
        return -math.pi + 2.0 * math.pi * px / W, -math.pi / 2 + math.pi * py / (H - 1)

    lon0, lat0 = to_sphere(x[..., None], y[..., None])
    lon1, lat1 = to_sphere(xs, ys)
    cosd = np.sin(lat0) * np.sin(lat1) + np.cos(lat0) * np.cos(lat1) * np.cos(lon0 - lon1)
    d = np.arccos(np.clip(cosd, -1.0, 1.0))
    w = 1.0 / (d + eps)
    w = w / w.sum(-1, keepdims=True)
    return (np.ascontiguousarray(np.stack([xs, ys], -1).astype(dtype)),
            np.ascontiguousarray(w.astype(dtype)))


# ----------------------------------------------------------------------------- icosphere
def _icosahedron():
    t = (1.0 + math.sqrt(5.0)) / 2.0
    v = np.array([[-1, t, 0], [1, t, 0], [-1, -t, 0], [1, -t, 0], [0, -1, t], [0, 1, t],
                  [0, -1, -t], [0, 1, -t], [t, 0, -1], [t, 0, 1], [-t, 0, -1], [-t, 0, 1]],
                 dtype=np.float64)
    v /= np.linalg.norm(v, axis=1, keepdims=True)
    f = np.array([[0, 11, 5], [0, 5, 1], [0, 1, 7], [0, 7, 10], [0, 10, 11], [1, 5, 9],
                  [5, 11, 4], [11, 10, 2], [10, 7, 6], [7, 1, 8], [3, 9, 4], [3, 4, 2],
                  [3, 2, 6], [3, 6, 8], [3, 8, 9], [4, 9, 5], [2, 4, 11], [6, 2, 10],
                  [8, 6, 7], [9, 8, 1]], dtype=np.int64)
    return v, f


def _icosphere_append(level):
    """Midpoint-subdivided, re-normalised icosahedron: (vertices [V,3], faces [F,3]).
    Midpoints are appended level by level, so vertices of level L keep their indices in
    level L+1 (V = 10*4^L + 2).  The four children of a face lie next to each other in the
    face list (corner 0, corner 1, corner 2, centre), so the list is in quadtree order."""
    v, f = _icosahedron()
    for _ in range(level):
        e = np.concatenate([f[:, [0, 1]], f[:, [1, 2]], f[:, [2, 0]]], 0)
        e.sort(axis=1)
        uniq, inv = np.unique(e, axis=0, return_inverse=True)
        inv = inv.reshape(-1)
        mid = v[uniq[:, 0]] + v[uniq[:, 1]]
        mid /= np.linalg.norm(mid, axis=1, keepdims=True)
        base = len(v)
        v = np.concatenate([v, mid], 0)
        nf = len(f)
        a, b, c = base + inv[:nf], base + inv[nf:2 * nf], base + inv[2 * nf:]
        f = np.stack([np.stack([f[:, 0], a, c], 1), np.stack([f[:, 1], b, a], 1),
                      np.stack([f[:, 2], c, b], 1), np.stack([a, b, c], 1)], 1).reshape(-1, 3)
    return v, f


def _hierarchical_order(f, V):
    """Permutation old_of_new [V]: vertices in the order in which the quadtree-ordered face list
    first names them, so that vertices close on the sphere are close in index."""
    flat = f.reshape(-1)
    vals, first = np.unique(flat, return_index=True)
    assert len(vals) == V
    return vals[np.argsort(first, kind="stable")]


def icosphere(level, order="append"):
    """(vertices [V,3], faces [F,3]) of the level-`level` icosphere.

    order="append": the numbering of midpoint subdivision (level-L vertices keep their indices
    at level L+1; neighbours are up to V apart in index: no locality).
    order="hierarchical": the same mesh renumbered along its quadtree face order
    (_hierarchical_order): a run of consecutive indices is a compact patch of the sphere."""
    v, f = _icosphere_append(level)
    if order == "append":
        return v, f
    if order != "hierarchical":
        raise ValueError("order must be 'append' or 'hierarchical'")
    old_of_new = _hierarchical_order(f, len(v))
    new_of_old = np.empty_like(old_of_new)
    new_of_old[old_of_new] = np.arange(len(v))
    return v[old_of_new], new_of_old[f]


def coarse_to_fine(level, order="append"):
    """[Vc] index, at level `level`, of every vertex of level `level` - 1 (in that level's own
    numbering of the same order): the parent -> child map of an up-sampling layer."""
    Vc = 10 * 4 ** (level - 1) + 2
    if order == "append":
        return np.arange(Vc)
    vf, ff = _icosphere_append(level)
    vc, fc = _icosphere_append(level - 1)
    fine_old_of_new = _hierarchical_order(ff, len(vf))
    fine_new_of_old = np.empty_like(fine_old_of_new)
    fine_new_of_old[fine_old_of_new] = np.arange(len(vf))
    coarse_old_of_new = _hierarchical_order(fc, len(vc))
    # append numbering: coarse vertex i is fine vertex i
    return fine_new_of_old[coarse_old_of_new]


def vertex_ring_map(level, num_vertices=None, dtype=np.float32, order="append"):
    """[1, V, 7, 2]: every vertex followed by its 1-ring neighbours as (index, 0)
    samples; the 12 five-neighbour vertices repeat their last neighbour."""
    v, f = icosphere(level, order)
    V = len(v)
    e = np.concatenate([f[:, [0, 1]], f[:, [1, 2]], f[:, [2, 0]], f[:, [1, 0]], f[:, [2, 1]],
                        f[:, [0, 2]]], 0)
    e = np.unique(e, axis=0)  # sorted by source vertex, then neighbour
    counts = np.bincount(e[:, 0], minlength=V)
    starts = np.concatenate([[0], np.cumsum(counts)[:-1]])
    ring = np.empty((V, 7), dtype=np.int64)
    ring[:, 0] = np.arange(V)
    for j in range(6):
        ring[:, 1 + j] = e[starts + np.minimum(j, counts - 1), 1]
    if num_vertices is not None:
        ring = ring[:num_vertices]
    out = np.zeros((1, ring.shape[0], 7, 2), dtype=dtype)
    out[0, :, :, 0] = ring
    return out


# ----------------------------------------------------------------------------- tangent images
def tangent_patch_map(H, W, level=1, patch=64, dtype=np.float32):
    """[F, patch*patch, 2] map of F = 20*4^level square tangent patches, one per
    icosphere face, each a patch x patch grid on the plane tangent at the face
    centre and wide enough to cover the face, projected back to the sphere
    (inverse gnomonic) and expressed in equirectangular pixel coordinates."""
    v, f = icosphere(level)
    centres = v[f].mean(1)
    centres /= np.linalg.norm(centres, axis=1, keepdims=True)
    # angular radius of a face: centre -> corner
    ang = np.arccos(np.clip((centres * v[f[:, 0]]).sum(1), -1, 1)).max()
    half = math.tan(ang)
    lin = np.linspace(-half, half, patch)
    u, w_ = np.meshgrid(lin, lin, indexing="xy")  # u -> east, w_ -> down
    # this repository's axis convention: lon = atan2(z, x), lat = atan2(-y, hypot(x, z))
    lon0 = np.arctan2(centres[:, 2], centres[:, 0])[:, None, None]
    lat0 = np.arctan2(-centres[:, 1], np.hypot(centres[:, 0], centres[:, 2]))[:, None, None]
    dx, dy = u[None], -w_[None]
    rho = np.sqrt(dx * dx + dy * dy)
    rho_safe = np.where(rho == 0, 1.0, rho)
    nu = np.arctan(rho)
    lat = np.arcsin(np.clip(np.cos(nu) * np.sin(lat0) + dy * np.sin(nu) * np.cos(lat0) / rho_safe,
                            -1, 1))
    lon = lon0 + np.arctan2(dx * np.sin(nu),
                            rho * np.cos(lat0) * np.cos(nu) - dy * np.sin(lat0) * np.sin(nu))
    lon = np.mod(lon + math.pi, 2 * math.pi) - math.pi
    x = W * (lon + math.pi) / (2 * math.pi)
    y = (H - 1) * (lat + math.pi / 2) / math.pi
    m = np.stack([x, y], -1).reshape(len(f), patch * patch, 2)
    return np.ascontiguousarray(m.astype(dtype))


def tangent_uv_map(H, W, level=1, patch=64, dtype=np.float32):
    """The way back from tangent_patch_map's patches: for every pixel of the H x W
    equirectangular image the face whose centre is nearest on the sphere (quad [H, W] int64) and
    the pixel's gnomonic projection onto that face's tangent plane in patch pixel coordinates
    (uv [H, W, 2], x first; 0 .. patch-1 spans the patch)."""
    v, f = icosphere(level)
    centres = v[f].mean(1)
    centres /= np.linalg.norm(centres, axis=1, keepdims=True)
    ang = np.arccos(np.clip((centres * v[f[:, 0]]).sum(1), -1, 1)).max()
    half = math.tan(ang)
    lon = (np.arange(W) * (2 * math.pi / W) - math.pi)[None, :]
    lat = (np.arange(H) * (math.pi / (H - 1)) - math.pi / 2)[:, None]
    # inverse of: lon = atan2(z, x), lat = atan2(-y, hypot(x, z))
    d = np.stack(np.broadcast_arrays(np.cos(lat) * np.cos(lon), -np.sin(lat),
                                     np.cos(lat) * np.sin(lon)), -1)
    quad = np.argmax(d.reshape(-1, 3) @ centres.T, axis=1).reshape(H, W)
    lon0 = np.arctan2(centres[:, 2], centres[:, 0])[quad]
    lat0 = np.arctan2(-centres[:, 1], np.hypot(centres[:, 0], centres[:, 2]))[quad]
    dl = lon - lon0
    cosc = np.sin(lat0) * np.sin(lat) + np.cos(lat0) * np.cos(lat) * np.cos(dl)
    dx = np.cos(lat) * np.sin(dl) / cosc
    dy = (np.cos(lat0) * np.sin(lat) - np.sin(lat0) * np.cos(lat) * np.cos(dl)) / cosc
    u = (dx + half) / (2 * half) * (patch - 1)
    w_ = (-dy + half) / (2 * half) * (patch - 1)
    uv = np.stack([u, w_], -1).astype(dtype)
    return np.ascontiguousarray(quad.astype(np.int64)), np.ascontiguousarray(uv)


# ----------------------------------------------------------------------------- configurations
def _rng(cfg):
    return np.random.default_rng(1234 + cfg)


def _conv_weights(rng, cout, cin, K, dtype, zero_bias=False):
    bound = 1.0 / math.sqrt(cin * K)
    w = rng.uniform(-bound, bound, (cout, cin, K)).astype(dtype)
    b = np.zeros(cout, dtype) if zero_bias else rng.uniform(-bound, bound, cout).astype(dtype)
    return w, b


def config1(dtype=np.float32):
    """Small mapped convolution, bilinear: x [1,3,64,128] -> [1,16,64,128], K = 9."""
    rng = _rng(1)
    x = rng.uniform(-1, 1, (1, 3, 64, 128)).astype(dtype)
    w, b = _conv_weights(rng, 16, 3, 9, dtype, zero_bias=True)
    return dict(x=x, sample_map=gnomonic_kernel_map(64, 128, dtype=dtype), weight=w, bias=b,
                grad_output=rng.standard_normal((1, 16, 64, 128)).astype(dtype),
                kernel_size=9, interp=1)


def config2(batch=4, H=512, W=1024, patch=64, dtype=np.float32):
    """Tangent-image resampling: gather [B,3,H,W] onto 80 patches, scatter back; and the UV
    way back: every image pixel reads its nearest face's patch at (u, v)."""
    rng = _rng(2)
    quad, uv = tangent_uv_map(H, W, 1, patch, dtype)
    return dict(x=rng.uniform(0, 1, (batch, 3, H, W)).astype(dtype),
                sample_map=tangent_patch_map(H, W, 1, patch, dtype), out_shape=(H, W), interp=1,
                quad_idx=quad, tex_uv=uv, patch=patch)


def config3(batch=8, channels=64, H=256, W=512, dtype=np.float32):
    """Mapped max pool, stride 2, nearest: [B,C,H,W] -> [B,C,H/2,W/2]."""
    rng = _rng(3)
    x = rng.standard_normal((batch, channels, H, W)).astype(dtype)
    x += (1e-4 * rng.uniform(0, 1, x.shape)).astype(dtype)
    return dict(x=x, sample_map=gnomonic_kernel_map(H, W, stride=2, dilation=2, dtype=dtype),
                grad_output=rng.standard_normal((batch, channels, H // 2, W // 2)).astype(dtype),
                kernel_size=9, interp=0)


def config4(batch=8, cin=128, cout=128, H=256, W=512, dtype=np.float32):
    """Large weighted (P = 4) bispherical mapped convolution."""
    rng = _rng(4)
    base = gnomonic_kernel_map(H, W, dtype=np.float64)
    m, iw = four_nearest_weighted(base, H, W, dtype=dtype)
    w, b = _conv_weights(rng, cout, cin, 9, dtype)
    return dict(x=rng.standard_normal((batch, cin, H, W)).astype(dtype), sample_map=m,
                interp_weights=iw, weight=w, bias=b,
                grad_output=rng.standard_normal((batch, cout, H, W)).astype(dtype),
                kernel_size=9, interp=2)


def config5(batch=4, channels=64, level=7, dtype=np.float32, order="hierarchical"):
    """Icosphere vertex convolution (level L) and transposed up-sampling (L-1 -> L).

    order: numbering of the vertices (icosphere()).  The layers only see index lists, so the
    numbering is the data layout of the workload; "hierarchical" keeps neighbours close in
    memory, "append" (what plain midpoint subdivision yields) is the incoherent case.  The
    up-sampling map lists, for every coarse vertex, its own fine index and its fine 1-ring."""
    rng = _rng(5)
    V = 10 * 4 ** level + 2
    Vc = 10 * 4 ** (level - 1) + 2
    ring = vertex_ring_map(level, dtype=dtype, order=order)
    w, b = _conv_weights(rng, channels, channels, 7, dtype)
    wt, bt = _conv_weights(rng, channels, channels, 7, dtype)
    up_map = np.ascontiguousarray(ring[:, coarse_to_fine(level, order)])
    return dict(x=rng.standard_normal((batch, channels, 1, V)).astype(dtype), sample_map=ring,
                weight=w, bias=b,
                grad_output=rng.standard_normal((batch, channels, 1, V)).astype(dtype),
                x_coarse=rng.standard_normal((batch, channels, 1, Vc)).astype(dtype),
                up_map=up_map, up_weight=wt.transpose(1, 0, 2).copy(),
                up_bias=bt, out_hw=(1, V), kernel_size=7, interp=0)
