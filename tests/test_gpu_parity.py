"""GPU parity: every C-ABI entry point against the CPU oracle on identical seeded inputs,
and against the fixtures the reference's compiled CPU code produced.

Tolerances (norm-relative, max|a-b| / max|b|):
  nearest gather and pooling indices      bit-exact
  float32 forward                         1e-5
  float32 backward (atomic reorder)       1e-4
  float64                                 1e-12
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


def _coords(rng, shape, h, w, dtype, margin=2.0):
    xy = rng.uniform(-margin, [w - 1 + margin, h - 1 + margin], size=tuple(shape) + (2,))
    sel = rng.uniform(size=shape) < 0.25
    xy[sel] = np.round(xy[sel])
    sel = rng.uniform(size=shape) < 0.1
    xy[sel] = np.floor(xy[sel]) + 0.5
    return np.ascontiguousarray(xy.astype(dtype))


CASES = [(i, wgt, dt) for i in (0, 1, 2) for wgt in (False, True)
         for dt in (np.float32, np.float64)]


def _ids(c):
    return "interp%d-%s-%s" % (c[0], "weighted" if c[1] else "plain", np.dtype(c[2]).name)


@pytest.mark.parametrize("case", CASES, ids=_ids)
def test_resample_both_directions(ops, oracle, case):
    interp, weighted, dt = case
    rng = np.random.default_rng(100 + interp)
    B, C, H, W, MH, MW, P = 3, 5, 37, 53, 29, 41, 3   # ragged: nothing divides a tile size
    x = rng.standard_normal((B, C, H, W)).astype(dt)
    m = _coords(rng, (MH, MW, P) if weighted else (MH, MW), H, W, dt)
    iw = rng.uniform(0.1, 1, (MH, MW, P)).astype(dt) if weighted else None
    got = _n(ops.resample_from_map(_t(x), _t(m), _t(iw), interp))
    want = oracle.resample_from_map(x, m, interp, iw)
    if interp == 0 and not weighted:
        assert np.array_equal(got, want)          # nearest resampling: bit-exact
    assert np.array_equal(got, want) or relerr(got, want) <= FWD_TOL[dt]
    y = rng.standard_normal((B, C, MH, MW)).astype(dt)
    got = _n(ops.resample_to_map(_t(y), _t(m), _t(iw), H, W, interp))
    want = oracle.resample_to_map(y, m, H, W, interp, iw)
    assert relerr(got, want) <= BWD_TOL[dt]
    # normalised variant == scatter(y) / (scatter(ones) + eps)
    gotn, wsum = ops.resample_to_map_normalized(_t(y), _t(m), _t(iw), H, W, interp, 1e-12)
    ones = oracle.resample_to_map(np.ones((1, 1, MH, MW), dt), m, H, W, interp, iw)[0, 0]
    assert relerr(_n(wsum), ones) <= BWD_TOL[dt]
    assert relerr(_n(gotn), want / (ones + dt(1e-12))) <= 10 * BWD_TOL[dt]


@pytest.mark.parametrize("interp,weighted", [(0, False), (1, False), (2, True)])
def test_resample_to_map_crowded_targets_and_no_workspace(ops, oracle, interp, weighted):
    """The scatter direction runs as a gather over the inverted map while every image pixel has
    at most 16 sources.  A map that sends a third of its pixels to one spot must fall back to
    the atomic scatter on the device, and a call without workspace must take it directly."""
    from _spherical_distortion_ext import _capi
    dt = np.float32
    rng = np.random.default_rng(300 + interp)
    B, C, H, W, MH, MW, P = 2, 3, 21, 33, 19, 27, 2
    m = _coords(rng, (MH, MW, P) if weighted else (MH, MW), H, W, dt)
    sel = rng.uniform(size=m.shape[:-1]) < 0.33
    m[sel] = np.array([11.3, 7.6], dtype=dt)
    iw = rng.uniform(0.1, 1, (MH, MW, P)).astype(dt) if weighted else None
    y = rng.standard_normal((B, C, MH, MW)).astype(dt)
    want = oracle.resample_to_map(y, m, H, W, interp, iw)
    ones = oracle.resample_to_map(np.ones((1, 1, MH, MW), dt), m, H, W, interp, iw)[0, 0]
    gotn, wsum = ops.resample_to_map_normalized(_t(y), _t(m), _t(iw), H, W, interp, 1e-12)
    assert relerr(_n(wsum), ones) <= 1e-4
    # weights are non-negative, so numerator and weight sum each carry n * eps relative to
    # the weight sum and the quotient n * eps * max|y|: the scatter tolerance holds for it
    assert relerr(_n(gotn), want / (ones + dt(1e-12))) <= 1e-4
    assert relerr(_n(ops.resample_to_map(_t(y), _t(m), _t(iw), H, W, interp)), want) <= 1e-4
    # the same call through the C ABI without workspace
    ty, tm, tw = _t(y), _t(m), _t(iw)
    out = torch.empty((B, C, H, W), dtype=torch.float32, device=DEV)
    _capi.call("sdk_resample_to_map", ops._ptr(ty), ops._ptr(tm), ops._ptr(tw), ops._ptr(out),
               None, None, 0, B, C, MH, MW, H, W, P if weighted else 0, interp, 0, ops._stream(ty))
    assert relerr(_n(out), want) <= 1e-4
    # ... and the normalised variant without workspace: scatter, weight-sum scatter, division
    wsum2 = torch.empty((H, W), dtype=torch.float32, device=DEV)
    _capi.call("sdk_resample_to_map_normalized", ops._ptr(ty), ops._ptr(tm), ops._ptr(tw),
               ops._ptr(out), ops._ptr(wsum2), None, 0, 1e-12, B, C, MH, MW, H, W,
               P if weighted else 0, interp, 0, ops._stream(ty))
    assert relerr(_n(wsum2), ones) <= 1e-4
    assert relerr(_n(out), want / (ones + dt(1e-12))) <= 1e-4


@pytest.mark.parametrize("case", CASES, ids=_ids)
def test_im2col_col2im(ops, oracle, case):
    interp, weighted, dt = case
    rng = np.random.default_rng(200 + interp)
    B, C, H, W, OH, OW, K, P = 2, 11, 19, 23, 13, 17, 5, 2
    x = rng.standard_normal((B, C, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if weighted else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if weighted else None
    got = _n(ops.mapped_im2col(_t(x), _t(m), _t(iw), interp))
    want = np.stack([oracle.mapped_im2col(x[b], m, interp, iw) for b in range(B)])
    assert np.array_equal(got, want) or relerr(got, want) <= FWD_TOL[dt]
    if interp == 0 and not weighted:
        assert np.array_equal(got, want)
    col = rng.standard_normal((B, C * K, OH * OW)).astype(dt)
    got = _n(ops.mapped_col2im(_t(col), _t(m), _t(iw), H, W, interp))
    want = np.stack([oracle.mapped_col2im(col[b], m, H, W, interp, iw) for b in range(B)])
    assert relerr(got, want) <= BWD_TOL[dt]


@pytest.mark.parametrize("case", CASES, ids=_ids)
def test_max_pool_and_unpool(ops, oracle, case):
    interp, weighted, dt = case
    rng = np.random.default_rng(300 + interp)
    B, C, H, W, OH, OW, K, P = 2, 9, 21, 27, 10, 13, 9, 2
    x = rng.standard_normal((B, C, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if weighted else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if weighted else None
    val, idx = ops.mapped_max_pool(_t(x), _t(m), _t(iw), K, interp)
    wval, widx = oracle.mapped_max_pool(x, m, K, interp, iw)          # device-branch init
    assert np.array_equal(_n(idx), widx)                              # indices: bit-exact
    assert np.array_equal(_n(val), wval)
    # against the reference host branch: identical wherever it found a winner
    hval, hidx = oracle.mapped_max_pool(x, m, K, interp, iw, host_init_quirk=True)
    ok = hidx >= 0
    assert np.array_equal(_n(idx)[ok], hidx[ok]) and np.array_equal(_n(val)[ok], hval[ok])
    g = rng.standard_normal((B, C, OH, OW)).astype(dt)
    got = _n(ops.mapped_max_unpool(_t(g), idx, _t(m), _t(iw), H, W, K, interp))
    want = oracle.mapped_max_unpool(g, widx, m, H, W, K, interp, iw)
    assert relerr(got, want) <= BWD_TOL[dt]


@pytest.mark.parametrize("case", CASES, ids=_ids)
def test_avg_pool_and_unpool(ops, oracle, case):
    interp, weighted, dt = case
    rng = np.random.default_rng(350 + interp)
    B, C, H, W, OH, OW, K, P = 2, 9, 21, 27, 10, 13, 5, 2
    x = rng.standard_normal((B, C, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if weighted else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if weighted else None
    got = _n(ops.mapped_avg_pool(_t(x), _t(m), _t(iw), K, interp))
    want = oracle.mapped_avg_pool(x, m, K, interp, iw)
    assert np.array_equal(got, want) or relerr(got, want) <= FWD_TOL[dt]
    g = rng.standard_normal((B, C, OH, OW)).astype(dt)
    got = _n(ops.mapped_avg_unpool(_t(g), _t(m), _t(iw), H, W, K, interp))
    want = oracle.mapped_avg_unpool(g, m, H, W, K, interp, iw)
    assert relerr(got, want) <= BWD_TOL[dt]
    # without workspace (float atomics) through the C ABI
    from _spherical_distortion_ext import _capi
    tg, tm, tw = _t(g), _t(m), _t(iw)
    out = torch.empty((B, C, H, W), dtype=tg.dtype, device=DEV)
    _capi.call("sdk_mapped_avg_unpool", ops._ptr(tg), ops._ptr(tm), ops._ptr(tw), ops._ptr(out),
               None, 0, B, C, H, W, OH, OW, K, P if weighted else 0, interp,
               0 if dt == np.float32 else 1, ops._stream(tg))
    assert relerr(_n(out), want) <= BWD_TOL[dt]


def test_pool_ties_nan_and_no_winner(ops, oracle):
    """First maximum wins; NaN never wins; a window below -FLT_MAX has index -1."""
    x = np.zeros((1, 1, 2, 4), np.float32)
    x[0, 0, 0] = [5, 5, np.nan, 1]
    x[0, 0, 1] = [-np.inf, -np.inf, -np.inf, -np.inf]
    m = np.array([[[[0, 0], [1, 0], [2, 0]], [[2, 0], [3, 0], [0, 0]],
                   [[0, 1], [1, 1], [2, 1]], [[9, 9], [9, 9], [9, 9]]]], np.float32)
    val, idx = ops.mapped_max_pool(_t(x), _t(m), None, 3, 0)
    wval, widx = oracle.mapped_max_pool(x, m, 3, 0)
    assert np.array_equal(_n(idx), widx) and np.array_equal(_n(val), wval)
    assert _n(idx).reshape(-1).tolist() == [0, 6 + 4, -1, 18]
    g = np.ones((1, 1, 1, 4), np.float32)
    got = _n(ops.mapped_max_unpool(_t(g), idx, _t(m), None, 2, 4, 3, 0))
    assert got.reshape(-1).tolist() == [2, 0, 0, 0, 0, 0, 0, 0]  # -1 and out-of-image drop out


def _unpool_capi(ops, g, idx, m, iw, H, W, K, P, interp, with_workspace):
    """mapped_max_unpool through the C ABI; returns (grad_input, gate) where gate is the
    workspace's first word after the call: 0 = the gather ran, > 0 = the call fell back to the
    atomic scatter, None = no workspace was passed."""
    from _spherical_distortion_ext import _capi
    tg, tm, tw = _t(g), _t(m), _t(iw)
    B, C, OH, OW = g.shape
    dtype = 0 if g.dtype == np.float32 else 1
    out = torch.full((B, C, H, W), 7.0, dtype=tg.dtype, device=DEV)   # must be overwritten
    ws, nws = None, 0
    if with_workspace:
        nws = _capi.load().sdk_mapped_max_unpool_workspace_bytes(H, W, dtype)
        assert nws > 0
        ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
    _capi.call("sdk_mapped_max_unpool", ops._ptr(tg), ops._ptr(idx), ops._ptr(tm), ops._ptr(tw),
               ops._ptr(out), ops._ptr(ws), nws, B, C, H, W, OH, OW, K, P, interp, dtype,
               ops._stream(tg))
    gate = int(ws[:4].view(torch.int32)[0]) if with_workspace else None
    return _n(out), gate


UNPOOL_CASES = [
    # (H, W, OH, OW, K, P, interp, dtype, scale)
    (40, 150, 20, 75, 9, 0, 0, np.float32, 1.0),    # strided nearest map over 3 x 3 image tiles
    (40, 150, 20, 75, 9, 0, 1, np.float32, 1.0),    # bilinear: four candidates per sample
    (33, 70, 16, 35, 5, 2, 2, np.float32, 1.0),     # weighted, columns wrap at the seam
    (1, 3000, 1, 1500, 7, 0, 0, np.float32, 1.0),   # one-row vertex list, flat tiles
    (40, 150, 20, 75, 9, 0, 0, np.float64, 1.0),
    (50, 20, 25, 10, 3, 2, 1, np.float64, 1.0),     # narrow image, tall tiles
]


@pytest.mark.parametrize("tc", UNPOOL_CASES, ids=lambda c: "H%dW%d_K%dP%d_i%d_%s" % (
    c[0], c[1], c[4], c[5], c[6], np.dtype(c[7]).name))
def test_unpool_by_image_tile(ops, oracle, tc):
    """Coherent maps: the call with workspace runs tile by tile (gate stays 0) and agrees with
    the oracle and with the atomic scatter of the call without workspace."""
    H, W, OH, OW, K, P, interp, dt, scale = tc
    rng = np.random.default_rng(900 + H + K + interp)
    B, C = 2, 5
    m = _coherent_map(rng, OH, OW, K, P, H, W, dt, scale)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if P else None
    x = rng.standard_normal((B, C, H, W)).astype(dt)
    _, idx = ops.mapped_max_pool(_t(x), _t(m), _t(iw), K, interp)
    g = rng.standard_normal((B, C, OH, OW)).astype(dt)
    want = oracle.mapped_max_unpool(g, _n(idx), m, H, W, K, interp, iw)
    got, gate = _unpool_capi(ops, g, idx, m, iw, H, W, K, P, interp, True)
    assert gate == 0
    assert relerr(got, want) <= BWD_TOL[dt]
    plain, _ = _unpool_capi(ops, g, idx, m, iw, H, W, K, P, interp, False)
    assert relerr(plain, want) <= BWD_TOL[dt]


def test_unpool_falls_back_to_the_scatter(ops, oracle):
    """Indices the pooling never writes and scattered maps raise the gate on the device; the
    result is the oracle's either way."""
    rng = np.random.default_rng(77)
    B, C, H, W, OH, OW, K = 2, 3, 24, 40, 12, 20, 9
    m = _coherent_map(rng, OH, OW, K, 0, H, W, np.float32)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    _, idx = ops.mapped_max_pool(_t(x), _t(m), None, K, 0)
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    # (a) an index that names a sample of another pooled pixel, a negative one, one past the end
    # of the map (the reference would read outside the map there; here it contributes nothing,
    # like a negative one, which is how the oracle is asked)
    idx_np = _n(idx).copy()
    idx_np[0, 0, 3, 4] = idx_np[0, 0, 7, 9]
    idx_np[1, 2, 0, 0] = -1
    idx_dev = idx_np.copy()
    idx_np[1, 1, 5, 5] = -1
    idx_dev[1, 1, 5, 5] = OH * OW * K * 2 + 10
    want = oracle.mapped_max_unpool(g, idx_np, m, H, W, K, 0)
    got, gate = _unpool_capi(ops, g, _t(idx_dev), m, None, H, W, K, 0, 0, True)
    assert gate > 0
    assert relerr(got, want) <= 1e-4
    # the same without the foreign index: negative / out-of-range ones alone do not fall back
    idx_np[0, 0, 3, 4] = idx_dev[0, 0, 3, 4] = _n(idx)[0, 0, 3, 4]
    want = oracle.mapped_max_unpool(g, idx_np, m, H, W, K, 0)
    got, gate = _unpool_capi(ops, g, _t(idx_dev), m, None, H, W, K, 0, 0, True)
    assert gate == 0
    assert relerr(got, want) <= 1e-4
    plain, _ = _unpool_capi(ops, g, _t(idx_dev), m, None, H, W, K, 0, 0, False)
    assert relerr(plain, want) <= 1e-4
    # (b) every sample of every pixel hits one of two image pixels: heavy collisions inside
    # one tile, still no fallback
    mc = np.zeros((OH, OW, K, 2), np.float32)
    mc[..., 0] = rng.integers(5, 7, (OH, OW, K))
    mc[..., 1] = 3
    _, idx_c = ops.mapped_max_pool(_t(x), _t(mc), None, K, 0)
    want = oracle.mapped_max_unpool(g, _n(idx_c), mc, H, W, K, 0)
    got, gate = _unpool_capi(ops, g, idx_c, mc, None, H, W, K, 0, 0, True)
    assert gate == 0
    assert relerr(got, want) <= 1e-4
    # (c) a scattered map: every tile would have to look at the whole pooled grid, which is
    # larger than a tile's window may be
    OH2, OW2 = 100, 120
    ms = _coords(rng, (OH2, OW2, 3), H, W, np.float32)
    _, idx_s = ops.mapped_max_pool(_t(x), _t(ms), None, 3, 0)
    g2 = rng.standard_normal((B, C, OH2, OW2)).astype(np.float32)
    want = oracle.mapped_max_unpool(g2, _n(idx_s), ms, H, W, 3, 0)
    got, gate = _unpool_capi(ops, g2, idx_s, ms, None, H, W, 3, 0, 0, True)
    assert gate > 0
    assert relerr(got, want) <= 1e-4


CONV_CASES = [(i, wgt, dt) for i in (0, 1, 2) for wgt in (False, True)
              for dt in (np.float32, np.float64)]


@pytest.mark.parametrize("case", CONV_CASES, ids=_ids)
def test_mapped_convolution(ops, oracle, case):
    interp, weighted, dt = case
    rng = np.random.default_rng(400 + interp)
    B, Cin, Cout, H, W, OH, OW, K, P = 2, 7, 5, 17, 19, 11, 13, 4, 3
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if weighted else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if weighted else None
    wt = rng.standard_normal((Cout, Cin, K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    got = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(wt), _t(b), K, interp))
    assert relerr(got, oracle.mapped_conv_forward(x, m, wt, b, K, interp, iw)) <= FWD_TOL[dt]
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(wt), _t(b), K, interp)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= BWD_TOL[dt]
    assert relerr(_n(gw), ww) <= BWD_TOL[dt]
    assert relerr(_n(gb), wb) <= BWD_TOL[dt]


@pytest.mark.parametrize("case", CONV_CASES, ids=_ids)
def test_mapped_transposed_convolution(ops, oracle, case):
    interp, weighted, dt = case
    rng = np.random.default_rng(500 + interp)
    B, Cin, Cout, IH, IW, OH, OW, K, P = 2, 6, 4, 9, 11, 15, 18, 3, 2
    x = rng.standard_normal((B, Cin, IH, IW)).astype(dt)
    m = _coords(rng, (IH, IW, K, P) if weighted else (IH, IW, K), OH, OW, dt)
    iw = rng.uniform(0.1, 1, (IH, IW, K, P)).astype(dt) if weighted else None
    wt = rng.standard_normal((Cin, Cout, K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    got = _n(ops.mapped_transposed_conv_forward(_t(x), _t(m), _t(iw), _t(wt), _t(b), OH, OW, K,
                                                interp))
    want = oracle.mapped_transposed_conv_forward(x, m, wt, b, OH, OW, K, interp, iw)
    assert relerr(got, want) <= BWD_TOL[dt]      # the forward is the scatter here
    gi, gw, gb = ops.mapped_transposed_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(wt), _t(b),
                                                     K, interp)
    wi, ww, wb = oracle.mapped_transposed_conv_backward(g, m, x, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= BWD_TOL[dt]
    assert relerr(_n(gw), ww) <= BWD_TOL[dt]
    assert relerr(_n(gb), wb) <= BWD_TOL[dt]


@pytest.fixture
def unfused(ops):
    ops.set_conv_compute("unfused")
    yield
    ops.set_conv_compute("native")


@pytest.mark.parametrize("case", [c for c in CONV_CASES if c[2] is np.float32], ids=_ids)
def test_unfused_float32_path(ops, oracle, unfused, case):
    """float32 normally runs the fused MFMA kernels; the separate im2col/col2im + GEMM
    kernels (the float64 route) must give the same answers in float32."""
    test_mapped_convolution(ops, oracle, case)
    test_mapped_transposed_convolution(ops, oracle, case)


# shapes that straddle the fused kernels' tiles: (Cin, Cout, H, W, OH, OW, K, P, interp)
TILE_CASES = [
    (40, 72, 20, 24, 19, 23, 5, 0, 1),     # wide tiles, ragged pixels, 2 reduction chunks
    (130, 130, 9, 12, 9, 12, 3, 2, 2),     # two channel tiles on both sides, weighted
    (33, 64, 16, 40, 8, 40, 9, 0, 0),      # narrow tiles (<= 64 channels), nearest
    (64, 33, 10, 30, 10, 29, 7, 4, 1),     # 16 tap slots per sample
    (3, 16, 64, 128, 64, 128, 9, 0, 1),    # configuration 1's shape
    # images of at most four channels: the packed kernels
    (1, 8, 12, 20, 12, 20, 9, 0, 1),       # one channel
    (2, 40, 14, 18, 7, 9, 25, 0, 0),       # 25 samples, two blocks of columns and of rows
    (4, 100, 10, 16, 10, 16, 9, 2, 2),     # weighted, four row blocks, two column blocks
    (4, 128, 9, 11, 9, 11, 25, 0, 1),      # weight gradient beyond the packed kernel's registers
]


@pytest.mark.parametrize("tc", TILE_CASES, ids=lambda t: "x".join(map(str, t)))
def test_fused_conv_tile_edges(ops, oracle, tc):
    Cin, Cout, H, W, OH, OW, K, P, interp = tc
    dt = np.float32
    rng = np.random.default_rng(sum(tc))
    B = 3
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if P else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if P else None
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    got = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(wt), _t(b), K, interp))
    assert relerr(got, oracle.mapped_conv_forward(x, m, wt, b, K, interp, iw)) <= 1e-5
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(wt), _t(b), K, interp)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4
    assert relerr(_n(gb), wb) <= 1e-4
    # transposed layer over the same map: input lives on the OH x OW grid, output on H x W
    xt = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    wtt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cout * K)).astype(dt)
    bt = rng.standard_normal(Cin).astype(dt)
    gt = rng.standard_normal((B, Cin, H, W)).astype(dt)
    got = _n(ops.mapped_transposed_conv_forward(_t(xt), _t(m), _t(iw), _t(wtt), _t(bt), H, W, K,
                                                interp))
    assert relerr(got, oracle.mapped_transposed_conv_forward(xt, m, wtt, bt, H, W, K, interp,
                                                             iw)) <= 1e-4
    gi, gw, gb = ops.mapped_transposed_conv_backward(_t(gt), _t(m), _t(iw), _t(xt), _t(wtt),
                                                     _t(bt), K, interp)
    wi, ww, wb = oracle.mapped_transposed_conv_backward(gt, m, xt, wtt, bt, K, interp, iw)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4
    assert relerr(_n(gb), wb) <= 1e-4


def test_weight_gradient_without_partial_sums(ops, oracle):
    """The weight gradient normally leaves per-workgroup sums in the workspace and a second
    kernel adds them up; a call whose sums would need more than 160 MB adds to grad_weight
    directly.  192 -> 256 channels at batch 12 on 8 tiles is such a call: 6 channel chunks x 2
    row-block tiles x 12 batch elements x 8 tile runs = 1152 workgroups of 147 456 bytes."""
    dt = np.float32
    rng = np.random.default_rng(77)
    B, Cin, Cout, H, W, K = 12, 192, 256, 16, 64, 9
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    m = _coherent_map(rng, H, W, K, 0, H, W, dt)
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, H, W)).astype(dt)
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), None, _t(x), _t(wt), _t(b), K, 1)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, 1, None)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4
    assert relerr(_n(gb), wb) <= 1e-4


def _coherent_map(rng, OH, OW, K, P, H, W, dtype, scale=1.0, jitter=0.45):
    """Locally coherent map: pixel (y, x) samples around (x, y) * scale * (W/OW, H/OH) with a
    ring of K offsets, as a convolution-style map does; a few samples fall outside the image."""
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / max(K, 1)
    rad = 1.0 + (np.arange(K) % 3)
    cx = xs[..., None] * (scale * W / OW) + rad * np.cos(ang)
    cy = ys[..., None] * (scale * H / OH) + rad * np.sin(ang)
    if P:
        cx = cx[..., None] + rng.uniform(-1, 1, (OH, OW, K, P))
        cy = cy[..., None] + rng.uniform(-1, 1, (OH, OW, K, P))
    xy = np.stack([cx, cy], -1) + rng.uniform(-jitter, jitter, cx.shape + (2,))
    sel = rng.uniform(size=cx.shape) < 0.2
    xy[sel] = np.round(xy[sel])          # exact pixel centres: zero-weight taps are dropped
    return np.ascontiguousarray(xy.astype(dtype))


# (Cin, Cout, H, W, OH, OW, K, P, interp, scale)
PLAN_CASES = [
    (40, 72, 24, 40, 24, 40, 9, 0, 1, 1.0),     # windows cover the taps; ragged tiles
    (32, 128, 20, 36, 20, 36, 9, 4, 2, 1.0),    # weighted bispherical, wrap at the seam
    (16, 24, 16, 24, 32, 48, 4, 0, 1, 0.5),     # up-sampling map: many pixels share a target
    (24, 16, 32, 48, 16, 24, 11, 0, 0, 1.0),    # two blocks of kernel samples (K > 9), nearest
    (8, 8, 12, 20, 12, 18, 25, 0, 1, 1.0),      # three blocks of kernel samples, OW % 4 != 0
    (64, 64, 1, 700, 1, 700, 7, 0, 0, 1.0),     # one-row vertex list
    (20, 20, 40, 3, 40, 3, 5, 0, 1, 1.0),       # narrow grid
    (12, 140, 9, 50, 3, 50, 3, 2, 1, 1.0),      # few rows; more than 128 pixel-side channels
    (8, 8, 10, 10, 10, 10, 2, 10, 1, 1.0),      # 40 tap slots per sample: generic path
    (8, 8, 10, 10, 10, 10, 2, 10, 0, 1.0),      # 10 slots, nearest weighted
    (4, 6, 6, 7, 6, 7, 260, 0, 1, 1.0),         # more kernel samples than a plan holds
]


@pytest.mark.parametrize("tc", PLAN_CASES, ids=lambda t: "x".join(map(str, t)))
def test_fused_conv_coherent_maps(ops, oracle, tc):
    """Maps with the locality the LDS-window kernels are built for, at shapes that hit their
    tiling, blocking and fallback branches; conv and transposed conv, forward and backward."""
    Cin, Cout, H, W, OH, OW, K, P, interp, scale = tc
    dt = np.float32
    rng = np.random.default_rng(11 + int(sum(tc)))
    B = 2
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    m = _coherent_map(rng, OH, OW, K, P, H, W, dt, scale)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if P else None
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    got = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(wt), _t(b), K, interp))
    assert relerr(got, oracle.mapped_conv_forward(x, m, wt, b, K, interp, iw)) <= 1e-5
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(wt), _t(b), K, interp)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4
    xt = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    wtt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cout * K)).astype(dt)
    bt = rng.standard_normal(Cin).astype(dt)
    gt = rng.standard_normal((B, Cin, H, W)).astype(dt)
    got = _n(ops.mapped_transposed_conv_forward(_t(xt), _t(m), _t(iw), _t(wtt), _t(bt), H, W, K,
                                                interp))
    assert relerr(got, oracle.mapped_transposed_conv_forward(xt, m, wtt, bt, H, W, K, interp,
                                                             iw)) <= 1e-4
    gi, gw, gb = ops.mapped_transposed_conv_backward(_t(gt), _t(m), _t(iw), _t(xt), _t(wtt),
                                                     _t(bt), K, interp)
    wi, ww, wb = oracle.mapped_transposed_conv_backward(gt, m, xt, wtt, bt, K, interp, iw)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4


@pytest.mark.parametrize("crowded", [False, True], ids=["injective", "crowded"])
def test_nearest_scatter_inverse_map_and_its_fallback(ops, oracle, crowded):
    """Nearest unweighted maps run the scatter contractions as a gather over the inverse map
    when every (target, sample) pair has at most 8 sources; a crowded map (a quarter of the
    pixels sample one spot) must take the atomic scatter kernel instead.  Same results."""
    dt = np.float32
    rng = np.random.default_rng(99 + crowded)
    B, Cin, Cout, H, W, OH, OW, K = 2, 24, 40, 14, 30, 14, 30, 5
    m = _coherent_map(rng, OH, OW, K, 0, H, W, dt)
    if crowded:
        sel = rng.uniform(size=(OH, OW, K)) < 0.25
        m[sel] = np.array([7.2, 3.9], dtype=dt)
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), None, _t(x), _t(wt), _t(b), K, 0)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, 0, None)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4
    xt = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    wtt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cout * K)).astype(dt)
    bt = rng.standard_normal(Cin).astype(dt)
    got = _n(ops.mapped_transposed_conv_forward(_t(xt), _t(m), None, _t(wtt), _t(bt), H, W, K, 0))
    assert relerr(got, oracle.mapped_transposed_conv_forward(xt, m, wtt, bt, H, W, K, 0,
                                                             None)) <= 1e-4


@pytest.fixture
def bf16_compute(ops):
    ops.set_conv_compute("bf16")
    yield
    ops.set_conv_compute("native")


@pytest.mark.parametrize("tc", TILE_CASES[:4], ids=lambda t: "x".join(map(str, t)))
def test_bf16_compute_within_1e_2(ops, oracle, bf16_compute, tc):
    """bf16 operands with fp32 accumulation in the MFMA contraction: every output within
    1e-2 (norm-relative) of the float32 CPU result."""
    Cin, Cout, H, W, OH, OW, K, P, interp = tc
    dt = np.float32
    rng = np.random.default_rng(7 + sum(tc))
    B = 2
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if P else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if P else None
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    got = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(wt), _t(b), K, interp))
    want = oracle.mapped_conv_forward(x, m, wt, b, K, interp, iw)
    assert 1e-6 < relerr(got, want) <= 1e-2      # really bf16, and inside the tolerance
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(wt), _t(b), K, interp)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= 1e-2
    assert relerr(_n(gw), ww) <= 1e-2
    assert relerr(_n(gb), wb) <= 1e-4
    xt = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    wtt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cout * K)).astype(dt)
    bt = rng.standard_normal(Cin).astype(dt)
    got = _n(ops.mapped_transposed_conv_forward(_t(xt), _t(m), _t(iw), _t(wtt), _t(bt), H, W, K,
                                                interp))
    assert relerr(got, oracle.mapped_transposed_conv_forward(xt, m, wtt, bt, H, W, K, interp,
                                                             iw)) <= 1e-2


@pytest.fixture
def split_compute(ops):
    ops.set_conv_compute("split")
    yield
    ops.set_conv_compute("native")


@pytest.mark.parametrize("tc", TILE_CASES + PLAN_CASES, ids=lambda t: "x".join(map(str, t)))
def test_split_compute_keeps_float32_accuracy(ops, oracle, split_compute, tc):
    """float32 operands split into three bf16 pieces each (six piece products, fp32
    accumulation): the float32 tolerances of the native mode, 1e-5 forward and 1e-4 backward,
    on random maps (tile edges) and on coherent maps (plan-driven kernels)."""
    Cin, Cout, H, W, OH, OW, K, P, interp = tc[:9]
    dt = np.float32
    rng = np.random.default_rng(17 + sum(tc[:9]))
    B = 2
    x = rng.standard_normal((B, Cin, H, W)).astype(dt)
    if len(tc) > 9:
        m = _coherent_map(rng, OH, OW, K, P, H, W, dt, tc[9])
    else:
        m = _coords(rng, (OH, OW, K, P) if P else (OH, OW, K), H, W, dt)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if P else None
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    got = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(wt), _t(b), K, interp))
    assert relerr(got, oracle.mapped_conv_forward(x, m, wt, b, K, interp, iw)) <= 1e-5
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(wt), _t(b), K, interp)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= 1e-4
    assert relerr(_n(gw), ww) <= 1e-4
    assert relerr(_n(gb), wb) <= 1e-4
    xt = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
    wtt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cout * K)).astype(dt)
    bt = rng.standard_normal(Cin).astype(dt)
    got = _n(ops.mapped_transposed_conv_forward(_t(xt), _t(m), _t(iw), _t(wtt), _t(bt), H, W, K,
                                                interp))
    want = oracle.mapped_transposed_conv_forward(xt, m, wtt, bt, H, W, K, interp, iw)
    assert relerr(got, want) <= 1e-4


def test_split_compute_on_values_that_stress_the_pieces(ops, oracle, split_compute):
    """Operands whose low mantissa bits matter: large offsets plus small signals, powers of two,
    denormal-range and huge magnitudes; and float64 tensors, which run as in the native mode."""
    dt = np.float32
    rng = np.random.default_rng(4242)
    B, Cin, Cout, H, W, K = 2, 32, 32, 16, 32, 9
    m = _coords(rng, (H, W, K), H, W, dt)
    x = (1000.0 + rng.standard_normal((B, Cin, H, W)) * 1e-3).astype(dt)
    x[0, 0] = 2.0 ** rng.integers(-20, 20, (H, W))
    x[0, 1] *= 1e30
    x[0, 2] *= 1e-30
    wt = (1.0 + rng.standard_normal((Cout, Cin, K)) * 1e-4).astype(dt)
    wt[0] = 2.0 ** -10
    b = np.zeros(Cout, dt)
    got = _n(ops.mapped_conv_forward(_t(x), _t(m), None, _t(wt), _t(b), K, 1))
    want = oracle.mapped_conv_forward(x.astype(np.float64), m.astype(np.float64),
                                      wt.astype(np.float64), b.astype(np.float64), K, 1)
    ops.set_conv_compute("native")
    native = _n(ops.mapped_conv_forward(_t(x), _t(m), None, _t(wt), _t(b), K, 1))
    ops.set_conv_compute("split")
    # no worse than twice the native mode's distance from the float64 result
    assert relerr(got, want) <= max(2 * relerr(native, want), 1e-6)
    x64 = rng.standard_normal((1, 3, 8, 9))
    m64 = _coords(rng, (5, 6, 4), 8, 9, np.float64)
    w64, b64 = rng.standard_normal((2, 3, 4)), rng.standard_normal(2)
    got = _n(ops.mapped_conv_forward(_t(x64), _t(m64), None, _t(w64), _t(b64), 4, 1))
    assert relerr(got, oracle.mapped_conv_forward(x64, m64, w64, b64, 4, 1)) <= 1e-12


# ------------------------------------------------------------------------------------------
# Against the compiled reference's fixtures directly (no oracle in between).
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("d", ["f64", "f32"])
@pytest.mark.parametrize("interp", [0, 1, 2])
def test_against_reference_fixtures(ops, d, interp):
    fx = np.load(os.path.join(GOLDEN_DIR, "ref_fixtures.npz"))
    dt = np.float64 if d == "f64" else np.float32
    ftol, btol = (1e-12, 1e-12) if d == "f64" else (1e-5, 1e-4)
    g = lambda n: _t(fx["%s/in/%s" % (d, n)])  # noqa: E731
    pre = "%s/i%d/" % (d, interp)
    H, W, K = 6, 7, 3
    assert np.array_equal(_n(ops.resample_from_map(g("x"), g("r_u"), None, interp)),
                          fx[pre + "from"])
    got = _n(ops.resample_from_map(g("x"), g("r_w"), g("riw"), interp))
    assert np.array_equal(got, fx[pre + "wfrom"]) or relerr(got, fx[pre + "wfrom"]) <= ftol
    assert relerr(_n(ops.resample_to_map(g("rin"), g("r_u"), None, H, W, interp)),
                  fx[pre + "to"]) <= btol
    assert relerr(_n(ops.resample_to_map(g("rin"), g("r_w"), g("riw"), H, W, interp)),
                  fx[pre + "wto"]) <= btol
    for wtag, m, iw in (("", g("m_u"), None), ("w", g("m_w"), g("iw"))):
        out = ops.mapped_conv_forward(g("x"), m, iw, g("weight"), g("bias"), K, interp)
        assert relerr(_n(out), fx[pre + wtag + "conv_fwd"]) <= ftol
        gi, gw, gb = ops.mapped_conv_backward(g("gout"), m, iw, g("x"), g("weight"), g("bias"),
                                              K, interp)
        assert relerr(_n(gi), fx[pre + wtag + "conv_gi"]) <= btol
        assert relerr(_n(gw), fx[pre + wtag + "conv_gw"]) <= btol
        assert relerr(_n(gb), fx[pre + wtag + "conv_gb"]) <= btol
        oh, ow = fx["%s/in/tgout" % d].shape[2:]
        out = ops.mapped_transposed_conv_forward(g("tx"), m, iw, g("tweight"), g("bias"), oh, ow,
                                                 K, interp)
        assert relerr(_n(out), fx[pre + wtag + "tconv_fwd"]) <= btol
        gi, gw, gb = ops.mapped_transposed_conv_backward(g("tgout"), m, iw, g("tx"), g("tweight"),
                                                         g("bias"), K, interp)
        assert relerr(_n(gi), fx[pre + wtag + "tconv_gi"]) <= btol
        assert relerr(_n(gw), fx[pre + wtag + "tconv_gw"]) <= btol
        assert relerr(_n(gb), fx[pre + wtag + "tconv_gb"]) <= btol
        # pooling: the GPU follows the reference's device branch; it equals the host-branch
        # fixture wherever that found a winner (index >= 0)
        val, idx = ops.mapped_max_pool(g("x"), m, iw, K, interp)
        ok = fx[pre + wtag + "pool_idx"] >= 0
        assert np.array_equal(_n(idx)[ok], fx[pre + wtag + "pool_idx"][ok])
        assert np.array_equal(_n(val)[ok], fx[pre + wtag + "pool_val"][ok])
    for wtag, m, iw in (("", g("m_ui"), None), ("w", g("m_wi"), g("iw"))):
        val, idx = ops.mapped_max_pool(g("xpos"), m, iw, K, interp)
        assert np.array_equal(_n(idx), fx[pre + wtag + "pospool_idx"])
        assert np.array_equal(_n(val), fx[pre + wtag + "pospool_val"])
        got = _n(ops.mapped_max_unpool(g("gpool"), idx, m, iw, H, W, K, interp))
        assert relerr(got, fx[pre + wtag + "unpool"]) <= btol
    assert dt is not None


def test_errors_are_raised_not_fatal(ops):
    x = torch.zeros(1, 2, 4, 5, device=DEV)
    m = torch.zeros(3, 3, 2, device=DEV)
    with pytest.raises(RuntimeError, match="contiguous"):
        ops.resample_from_map(x.transpose(2, 3), m, None, 1)
    with pytest.raises(RuntimeError, match="dtype"):
        ops.resample_from_map(x, m.double(), None, 1)
    with pytest.raises(RuntimeError, match="CUDA"):
        ops.resample_from_map(x, m.cpu(), None, 1)
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        ops.resample_from_map(x.half(), m.half(), None, 1)
    # unknown interpolation values fall back to nearest like the reference's switch default
    a = ops.resample_from_map(x + 1, m, None, 7)
    assert torch.equal(a, ops.resample_from_map(x + 1, m, None, 0))


# ------------------------------------------------------------------------------------------
# Unpooling as a layer: forward = the unpool entry point, backward = the gather at the index.
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("case", CASES, ids=_ids)
def test_gather_at_index_and_unpool_layer(ops, oracle, case):
    import spherical_distortion.functional as F
    from spherical_distortion.nn import MappedMaxUnpool
    interp, weighted, dt = case
    rng = np.random.default_rng(800 + interp)
    B, C, H, W, OH, OW, K, P = 2, 5, 23, 31, 11, 13, 5, 2
    x = rng.standard_normal((B, C, H, W)).astype(dt)
    m = _coords(rng, (OH, OW, K, P) if weighted else (OH, OW, K), H, W, dt, margin=0.0)
    iw = rng.uniform(0.1, 1, (OH, OW, K, P)).astype(dt) if weighted else None
    val, idx = ops.mapped_max_pool(_t(x), _t(m), _t(iw), K, interp)
    # the pooled value is the image read at the winning sample (same arithmetic: bit-exact)
    got = ops.mapped_gather_at_index(_t(x), idx, _t(m), _t(iw), K, interp)
    ok = _n(idx) >= 0
    assert np.array_equal(_n(got)[ok], _n(val)[ok])
    assert (_n(got)[~ok] == 0).all()
    # arbitrary indices, some of them outside the map, against the oracle
    q = P if weighted else 1
    any_idx = (rng.integers(0, K, (B, C, OH, OW)) + np.arange(OH * OW).reshape(OH, OW) * K) * q * 2
    any_idx[0, 0, 0, :3] = -1
    got = _n(ops.mapped_gather_at_index(_t(x), _t(any_idx), _t(m), _t(iw), K, interp))
    want = oracle.mapped_gather_at_index(x, any_idx, m, interp, iw)
    assert np.array_equal(got, want) or relerr(got, want) <= FWD_TOL[dt]
    # the layer: forward is the unpool, backward the gather
    pooled = torch.from_numpy(rng.standard_normal((B, C, OH, OW)).astype(dt)).to(DEV)
    pooled.requires_grad_(True)
    safe = np.where(any_idx < 0, 0, any_idx)
    layer = MappedMaxUnpool(K, interp)
    up = layer(pooled, _t(safe), _t(m), (H, W), _t(iw))
    want_up = oracle.mapped_max_unpool(_n(pooled), safe, m, H, W, K, interp, iw)
    assert relerr(_n(up), want_up) <= BWD_TOL[dt]
    up.backward(_t(x))
    want_grad = oracle.mapped_gather_at_index(x, safe, m, interp, iw)
    assert relerr(_n(pooled.grad), want_grad) <= FWD_TOL[dt]
    if dt == np.float64 and interp == 1 and not weighted:
        probe = torch.from_numpy(rng.standard_normal((1, 2, OH, OW))).to(DEV).requires_grad_(True)
        assert torch.autograd.gradcheck(
            lambda t: F.mapped_max_unpool(t, _t(safe[:1, :2]), _t(m), (H, W), K, interp), (probe,),
            eps=1e-6, atol=1e-7, nondet_tol=1e-9)


@pytest.mark.parametrize("mode", ["native", "bf16", "split"])
@pytest.mark.parametrize("shape", [(9, 12), (16, 20), (8, 28), (20, 36)],
                         ids=lambda s: "%dx%d" % s)
def test_weight_gradient_reads_nothing_behind_its_rows(ops, oracle, mode, shape):
    """Grids whose width is a multiple of 4 but not of 8: the weight gradient loads runs of 4
    (float32) or 8 (bf16, split) pixels per lane.  The pixel-side tensor is the tail of a buffer
    whose remaining bytes are NaN, so a run that leaves its row, or the tensor, poisons
    grad_weight."""
    OH, OW = shape
    dt = np.float32
    rng = np.random.default_rng(5 + OH * OW)
    B, Cin, Cout, K = 2, 16, 32, 9
    x = rng.standard_normal((B, Cin, OH, OW)).astype(dt)
    m = _coherent_map(rng, OH, OW, K, 0, OH, OW, dt)
    wt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(dt)
    b = rng.standard_normal(Cout).astype(dt)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(dt)

    def guarded(a):
        """a on the device, followed directly by 64 NaNs of the same allocation."""
        buf = torch.full((a.size + 64,), float("nan"), dtype=torch.float32, device=DEV)
        buf[:a.size] = _t(a).reshape(-1)
        return buf[:a.size].view(*a.shape), buf

    tol = 1e-2 if mode == "bf16" else 1e-4
    ops.set_conv_compute(mode)
    try:
        gg, keep_g = guarded(g)
        _, gw, _ = ops.mapped_conv_backward(gg, _t(m), None, _t(x), _t(wt), _t(b), K, 1)
        ww = oracle.mapped_conv_backward(g, m, x, wt, b, K, 1, None)[1]
        assert bool(torch.isfinite(gw).all())
        assert relerr(_n(gw), ww) <= tol
        # transposed layer: its input is the pixel-side tensor of the weight gradient
        xt = rng.standard_normal((B, Cout, OH, OW)).astype(dt)
        wtt = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cout * K)).astype(dt)
        bt = rng.standard_normal(Cin).astype(dt)
        gt = rng.standard_normal((B, Cin, OH, OW)).astype(dt)
        xg, keep_x = guarded(xt)
        _, gw, _ = ops.mapped_transposed_conv_backward(_t(gt), _t(m), None, xg, _t(wtt), _t(bt),
                                                       K, 1)
        ww = oracle.mapped_transposed_conv_backward(gt, m, xt, wtt, bt, K, 1, None)[1]
        assert bool(torch.isfinite(gw).all())
        assert relerr(_n(gw), ww) <= tol
    finally:
        ops.set_conv_compute("native")
