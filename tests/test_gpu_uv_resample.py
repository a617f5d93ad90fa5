"""GPU parity of UV resampling (tangent images back to one image) and of average pooling against
the fixtures the reference's compiled CPU code produced, plus UV resampling against the CPU
oracle on larger seeded cases, through every path of the adjoint: texture by texture in on-chip
memory (one or several workgroups per texture), and atomic adds in memory for calls without
workspace or with textures too large for that.

Tolerances (max|a-b| / max|b|): nearest gather bit-exact, float32 forward 1e-5, float32 backward
(accumulation order) 1e-4, float64 1e-12.
"""
import os

import numpy as np
import pytest
import torch

from conftest import GOLDEN_DIR, relerr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FWD_TOL = {np.float32: 1e-5, np.float64: 1e-12}
BWD_TOL = {np.float32: 1e-4, np.float64: 1e-12}


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _n(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("d", ["f64", "f32"])
@pytest.mark.parametrize("interp", [0, 1, 2])
def test_against_reference_fixtures(ops, d, interp):
    fx = np.load(os.path.join(GOLDEN_DIR, "ref_fixtures_avg_uv.npz"))
    dt = np.float64 if d == "f64" else np.float32
    g = lambda n: _t(fx["%s/in/%s" % (d, n)])  # noqa: E731
    pre = "%s/i%d/" % (d, interp)
    H, W, K = 6, 7, 3
    for wtag, m, iw in (("", g("m_u"), None), ("w", g("m_w"), g("iw"))):
        got = _n(ops.mapped_avg_pool(g("x"), m, iw, K, interp))
        assert relerr(got, fx[pre + wtag + "avg_pool"]) <= FWD_TOL[dt]
        got = _n(ops.mapped_avg_unpool(g("g"), m, iw, H, W, K, interp))
        assert relerr(got, fx[pre + wtag + "avg_unpool"]) <= BWD_TOL[dt]
    nt, th, tw = fx["%s/in/tex" % d].shape[2:]
    got = _n(ops.resample_from_uv_maps(g("tex"), g("quad"), g("uv"), interp))
    if interp == 0:
        assert np.array_equal(got, fx[pre + "from_uv"])
    assert np.array_equal(got, fx[pre + "from_uv"]) or \
        relerr(got, fx[pre + "from_uv"]) <= FWD_TOL[dt]
    got = _n(ops.resample_to_uv_maps(g("x"), g("quad"), g("uv"), nt, th, tw, interp))
    assert relerr(got, fx[pre + "to_uv"]) <= BWD_TOL[dt]


def _uv_case(rng, dt, B, C, NT, TH, TW, H, W, crowd=0.0):
    tex = rng.standard_normal((B, C, NT, TH, TW)).astype(dt)
    quad = rng.integers(0, NT, (H, W)).astype(np.int64)
    uv = np.stack([rng.uniform(-1.5, TW + 0.5, (H, W)), rng.uniform(-1.5, TH + 0.5, (H, W))], -1)
    snap = rng.uniform(size=(H, W)) < 0.25
    uv[snap] = np.round(uv[snap])
    half = rng.uniform(size=(H, W)) < 0.1
    uv[half] = np.floor(uv[half]) + 0.5
    if crowd:
        sel = rng.uniform(size=(H, W)) < crowd
        quad[sel] = NT - 1
        uv[sel] = [1.3, 2.6]
    y = rng.standard_normal((B, C, H, W)).astype(dt)
    return tex, quad, np.ascontiguousarray(uv.astype(dt)), y


def _to_uv_capi(ops, y, quad, uv, NT, TH, TW, interp, with_workspace):
    """sdk_resample_to_uv_maps through the C ABI, with the workspace its query asks for or with
    none; the output starts from garbage, which the call must overwrite everywhere."""
    from _spherical_distortion_ext import _capi
    B, C, H, W = y.shape
    ty, tq, tu = _t(y), _t(quad), _t(uv)
    dtype = 0 if y.dtype == np.float32 else 1
    out = torch.full((B, C, NT, TH, TW), 7.0, dtype=ty.dtype, device=DEV)
    ws, nws = None, 0
    if with_workspace:
        nws = _capi.load().sdk_resample_to_uv_maps_workspace_bytes(NT, TH, TW, H, W, dtype)
        ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=DEV)
    _capi.call("sdk_resample_to_uv_maps", ops._ptr(ty), ops._ptr(tq), ops._ptr(tu), ops._ptr(out),
               ops._ptr(ws), nws, B, C, NT, TH, TW, H, W, interp, dtype, ops._stream(ty))
    return _n(out), nws


# B, C, NT, TH, TW, H, W: ragged sizes; many textures and planes (several planes per workgroup);
# one row of pixels and wide textures; two textures only (several workgroups share a texture);
# textures that do not fit in on-chip memory (the workspace query answers 0); textures that just fit
UV_SHAPES = ((2, 3, 7, 9, 13, 31, 45), (1, 12, 20, 16, 16, 64, 96), (3, 35, 4, 5, 300, 17, 260),
             (2, 40, 300, 6, 5, 40, 70), (1, 3, 2, 12, 10, 50, 130), (1, 2, 3, 130, 140, 33, 47),
             (1, 2, 3, 128, 128, 45, 100))      # float32 textures of exactly 64 KiB
UV_CASES = [(interp, dt, shape) for interp in (0, 1, 2) for dt in (np.float32, np.float64)
            for shape in UV_SHAPES]


@pytest.mark.parametrize("case", UV_CASES,
                         ids=lambda c: "interp%d-%s-%s" % (c[0], np.dtype(c[1]).name,
                                                           "x".join(map(str, c[2]))))
def test_uv_resample_both_directions(ops, oracle, case):
    interp, dt, (B, C, NT, TH, TW, H, W) = case
    rng = np.random.default_rng(900 + interp + H)
    tex, quad, uv, y = _uv_case(rng, dt, B, C, NT, TH, TW, H, W)
    got = _n(ops.resample_from_uv_maps(_t(tex), _t(quad), _t(uv), interp))
    want = oracle.resample_from_uv_maps(tex, quad, uv, interp)
    if interp == 0:
        assert np.array_equal(got, want)
    assert np.array_equal(got, want) or relerr(got, want) <= FWD_TOL[dt]
    want = oracle.resample_to_uv_maps(y, quad, uv, NT, TH, TW, interp)
    got = _n(ops.resample_to_uv_maps(_t(y), _t(quad), _t(uv), NT, TH, TW, interp))
    assert relerr(got, want) <= BWD_TOL[dt]
    for with_ws in (True, False):
        got, nws = _to_uv_capi(ops, y, quad, uv, NT, TH, TW, interp, with_ws)
        assert relerr(got, want) <= BWD_TOL[dt]
        if with_ws:
            assert (nws == 0) == (TH * TW * np.dtype(dt).itemsize > 65536)


def test_uv_scatter_plan_matches_the_plain_call(ops, oracle):
    """sdk_resample_to_uv_maps_plan_build / _planned: the buckets kept between calls (two calls
    on one plan, different inputs), through the C ABI and through the operator's cache (on and
    off); too small a plan is refused."""
    from _spherical_distortion_ext import _capi
    B, C, NT, TH, TW, H, W = 2, 5, 9, 12, 10, 40, 66
    rng = np.random.default_rng(77)
    _, quad, uv, y = _uv_case(rng, np.float32, B, C, NT, TH, TW, H, W, crowd=0.1)
    tq, tu = _t(quad), _t(uv)
    n = _capi.load().sdk_resample_to_uv_maps_workspace_bytes(NT, TH, TW, H, W, 0)
    assert n > 0
    plan = torch.empty(n, dtype=torch.uint8, device=DEV)
    _capi.call("sdk_resample_to_uv_maps_plan_build", ops._ptr(tq), ops._ptr(plan), n, NT, TH, TW,
               H, W, 0, ops._stream(tq))
    for scale in (1.0, -0.5):
        ty = _t(y * np.float32(scale))
        out = torch.full((B, C, NT, TH, TW), 7.0, device=DEV)
        _capi.call("sdk_resample_to_uv_maps_planned", ops._ptr(ty), ops._ptr(tq), ops._ptr(tu),
                   ops._ptr(out), ops._ptr(plan), n, B, C, NT, TH, TW, H, W, 1, 0, ops._stream(ty))
        want = oracle.resample_to_uv_maps(y * np.float32(scale), quad, uv, NT, TH, TW, 1)
        assert relerr(_n(out), want) <= 1e-4
        plain, _ = _to_uv_capi(ops, y * np.float32(scale), quad, uv, NT, TH, TW, 1, True)
        assert relerr(_n(out), plain) <= 1e-5
    with pytest.raises(RuntimeError, match="plan of"):
        _capi.call("sdk_resample_to_uv_maps_plan_build", ops._ptr(tq), ops._ptr(plan), n - 1, NT,
                   TH, TW, H, W, 0, ops._stream(tq))
    want = oracle.resample_to_uv_maps(y, quad, uv, NT, TH, TW, 1)
    for cached in (True, True, False):
        ops.set_conv_plan_cache(cached)
        try:
            got = _n(ops.resample_to_uv_maps(_t(y), tq, tu, NT, TH, TW, 1))
        finally:
            ops.set_conv_plan_cache(True)
        assert relerr(got, want) <= 1e-4


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("coherent", [True, False])
def test_uv_scatter_with_crowded_texels(ops, oracle, interp, coherent):
    """Hundreds of pixels per texel, as near the poles of an equirectangular image: rows of
    pixels that creep over a texture (runs of lanes on one texel), or a third of all pixels
    aimed at one spot."""
    dt = np.float32
    rng = np.random.default_rng(950 + interp)
    B, C, NT, TH, TW, H, W = 2, 5, 6, 8, 11, 23, 700
    tex, quad, uv, y = _uv_case(rng, dt, B, C, NT, TH, TW, H, W, crowd=0.0 if coherent else 0.33)
    if coherent:
        quad = np.repeat((np.arange(H) % NT)[:, None], W, 1).astype(np.int64)
        uv[..., 0] = np.linspace(-1.2, TW + 0.2, W)[None, :] * (np.arange(H)[:, None] % 3 + 1) / 3
        uv[..., 1] = (np.arange(H)[:, None] * 0.37) % (TH + 1) - 0.6
        uv = np.ascontiguousarray(uv.astype(dt))
    want = oracle.resample_to_uv_maps(y, quad, uv, NT, TH, TW, interp)
    for with_ws in (True, False):
        got, _ = _to_uv_capi(ops, y, quad, uv, NT, TH, TW, interp, with_ws)
        assert relerr(got, want) <= 1e-4


@pytest.mark.parametrize("interp", [0, 1])
def test_texture_indices_out_of_range_contribute_nothing(ops, oracle, interp):
    dt = np.float32
    rng = np.random.default_rng(970 + interp)
    B, C, NT, TH, TW, H, W = 2, 3, 4, 6, 7, 15, 22
    tex, quad, uv, y = _uv_case(rng, dt, B, C, NT, TH, TW, H, W)
    quad[::2, ::3] = NT
    quad[1::2, ::4] = -1
    quad[0, 0] = 2 ** 40
    got = _n(ops.resample_from_uv_maps(_t(tex), _t(quad), _t(uv), interp))
    assert relerr(got, oracle.resample_from_uv_maps(tex, quad, uv, interp)) <= 1e-5
    assert (got[:, :, ::2, ::3] == 0).all()
    want = oracle.resample_to_uv_maps(y, quad, uv, NT, TH, TW, interp)
    for with_ws in (True, False):
        got, _ = _to_uv_capi(ops, y, quad, uv, NT, TH, TW, interp, with_ws)
        assert relerr(got, want) <= 1e-4
    # no pixel names a texture at all: the call still writes every texel (zeros)
    quad[:] = -3
    got, _ = _to_uv_capi(ops, y, quad, uv, NT, TH, TW, interp, True)
    assert (got == 0).all()


def test_uv_resample_autograd_and_module(ops, oracle):
    """functional.uv_resample: forward is the gather, backward the splat into the texture stack;
    a 4-D input is one batch element (layers/functional/resample.py:192-209)."""
    import spherical_distortion.functional as F
    from spherical_distortion.nn import UVResample
    dt = np.float32
    rng = np.random.default_rng(990)
    B, C, NT, TH, TW, H, W = 2, 3, 5, 6, 9, 14, 19
    tex, quad, uv, y = _uv_case(rng, dt, B, C, NT, TH, TW, H, W)
    t = _t(tex).requires_grad_(True)
    out = F.uv_resample(t, _t(quad), _t(uv), 1)
    assert relerr(_n(out), oracle.resample_from_uv_maps(tex, quad, uv, 1)) <= 1e-5
    out.backward(_t(y))
    assert relerr(_n(t.grad), oracle.resample_to_uv_maps(y, quad, uv, NT, TH, TW, 1)) <= 1e-4
    one = F.uv_resample(_t(tex[0]), _t(quad), _t(uv), 2)
    assert one.shape == (C, H, W)
    assert relerr(_n(one), oracle.resample_from_uv_maps(tex[:1], quad, uv, 2)[0]) <= 1e-5
    layer = UVResample(_t(quad), _t(uv))
    assert torch.equal(layer(_t(tex)), out.detach())


def test_uv_errors(ops):
    tex = torch.zeros(1, 2, 3, 4, 5, device=DEV)
    quad = torch.zeros(6, 7, dtype=torch.int64, device=DEV)
    uv = torch.zeros(6, 7, 2, device=DEV)
    with pytest.raises(RuntimeError, match="int64"):
        ops.resample_from_uv_maps(tex, quad.int(), uv, 1)
    with pytest.raises(RuntimeError, match="tex_uv"):
        ops.resample_from_uv_maps(tex, quad, uv[:5], 1)
    with pytest.raises(RuntimeError, match="textures must be"):
        ops.resample_from_uv_maps(tex[0], quad, uv, 1)
    with pytest.raises(RuntimeError, match="must be \\[B, C"):
        ops.resample_to_uv_maps(torch.zeros(1, 2, 6, 8, device=DEV), quad, uv, 3, 4, 5, 1)
    # empty batch: nothing to do, nothing launched
    out = ops.resample_from_uv_maps(tex[:0], quad, uv, 1)
    assert out.shape == (0, 2, 6, 7)


# ----------------------------------------------------------------------------- voting resample
def test_voting_resample_is_bit_exact(ops, oracle):
    """Integer work: bit-exact against the compiled reference's fixture (three channels, whose
    histograms overlap in the reference; reproduced) and against the oracle on larger seeded
    cases with targets outside the output and labels outside the range."""
    fx = np.load(os.path.join(GOLDEN_DIR, "ref_fixtures_avg_uv.npz"))
    labels, vmap, want = fx["vote/in/labels"], fx["vote/in/map"], fx["vote/out"]
    got = ops.voting_resample_to_map(_t(labels), _t(vmap), want.shape[2], want.shape[3], 5)
    assert got.dtype == torch.int64 and np.array_equal(_n(got), want)
    for seed, (b, c, ih, iw, oh, ow, nc) in enumerate(((3, 1, 64, 96, 20, 30, 13),
                                                       (2, 4, 33, 47, 31, 45, 3),
                                                       (1, 1, 5, 700, 2, 3, 40),
                                                       (2, 2, 17, 19, 40, 50, 1))):
        rng = np.random.default_rng(60 + seed)
        labels = rng.integers(-1, nc + 1, (b, c, ih, iw))
        vmap = np.stack([rng.integers(-1, ow + 1, (ih, iw)),
                         rng.integers(-1, oh + 1, (ih, iw))], -1)
        got = _n(ops.voting_resample_to_map(_t(labels), _t(vmap), oh, ow, nc))
        assert np.array_equal(got, oracle.voting_resample_to_map(labels, vmap, oh, ow, nc))


def test_voting_resample_functional_and_errors(ops, oracle):
    import spherical_distortion.functional as F
    from _spherical_distortion_ext import _capi
    rng = np.random.default_rng(77)
    labels = rng.integers(0, 6, (1, 12, 20))                 # one image without batch axis
    vmap = np.stack([rng.integers(0, 10, (12, 20)), rng.integers(0, 6, (12, 20))], -1)
    got = F.voting_resample(_t(labels.astype(np.float32)), _t(vmap.astype(np.float32)), None,
                            (6, 10), 6)
    assert got.shape == (1, 6, 10)
    assert np.array_equal(_n(got), oracle.voting_resample_to_map(labels[None], vmap, 6, 10, 6)[0])
    with pytest.raises(RuntimeError, match="int64"):
        ops.voting_resample_to_map(_t(labels[None]).int(), _t(vmap), 6, 10, 6)
    with pytest.raises(RuntimeError, match="sample_map"):
        ops.voting_resample_to_map(_t(labels[None]), _t(vmap[:5]), 6, 10, 6)
    # a workspace of one histogram serves a batch in passes: same result as all at once
    lab4 = rng.integers(0, 6, (4, 2, 12, 20))
    t4 = _t(lab4)
    nws = _capi.load().sdk_voting_resample_workspace_bytes(2, 6, 10, 6)
    ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
    out4 = torch.empty((4, 2, 6, 10), dtype=torch.int64, device=DEV)
    _capi.call("sdk_voting_resample_to_map", ops._ptr(t4), ops._ptr(_t(vmap)), ops._ptr(out4),
               ops._ptr(ws), nws, 4, 2, 12, 20, 6, 10, 6, ops._stream(t4))
    assert np.array_equal(_n(out4), oracle.voting_resample_to_map(lab4, vmap, 6, 10, 6))
    assert torch.equal(out4, ops.voting_resample_to_map(t4, _t(vmap), 6, 10, 6))
    # the histogram workspace is required
    tl, tm = _t(labels[None]), _t(vmap)
    out = torch.empty((1, 1, 6, 10), dtype=torch.int64, device=DEV)
    with pytest.raises(RuntimeError, match="workspace"):
        _capi.call("sdk_voting_resample_to_map", ops._ptr(tl), ops._ptr(tm), ops._ptr(out), None,
                   0, 1, 1, 12, 20, 6, 10, 6, ops._stream(tl))
