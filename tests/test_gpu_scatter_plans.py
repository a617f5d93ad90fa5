"""Plans of the scatter direction (sdk_resample_to_map_plan_build, sdk_mapped_max_unpool_plan_build
and the *_planned entry points) against the plain entry points, which rebuild the same scratch
inside every call, and against the oracle: resampling to a map (plain and normalised, with and
without point weights), average unpooling and max unpooling; a map whose targets collect more
sources than a list holds (the plan reports itself incomplete and the planned call falls back);
the operator-level cache with an in-place change of the map; refused plan sizes.
"""
import ctypes

import numpy as np
import pytest
import torch

from conftest import relerr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F32 = 0


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


@pytest.fixture(scope="module")
def capi():
    from _spherical_distortion_ext import _capi
    return _capi


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _n(t):
    return t.detach().cpu().numpy()


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _resample_case(seed, MH, MW, H, W, P, crowded=False):
    rng = np.random.default_rng(seed)
    shape = (MH, MW, P) if P else (MH, MW)
    m = np.stack([rng.uniform(-0.5, W - 0.5, shape), rng.uniform(-0.5, H - 0.5, shape)], -1)
    if crowded:   # a third of the samples land near one pixel: more than 16 sources there
        sel = rng.uniform(size=shape) < 0.33
        m[..., 0] = np.where(sel, 3.2, m[..., 0])
        m[..., 1] = np.where(sel, 2.7, m[..., 1])
    m = m.astype(np.float32)
    iw = rng.uniform(0.1, 1, shape).astype(np.float32) if P else None
    x = rng.standard_normal((2, 5, MH, MW)).astype(np.float32)
    return m, iw, x


def _build_resample_plan(capi, m, iw, H, W, K, P, interp):
    n = capi.load().sdk_resample_to_map_workspace_bytes(H, W, F32)
    plan = torch.empty(n, dtype=torch.uint8, device=DEV)
    capi.call("sdk_resample_to_map_plan_build", _p(m), _p(iw), _p(plan), n, m.shape[0], m.shape[1],
              H, W, K, P, interp, F32, _stream())
    flag = ctypes.c_int32(-1)
    capi.call("sdk_resample_plan_complete", _p(plan), n, _stream(),
              ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
    return plan, n, int(flag.value)


@pytest.mark.parametrize("P,interp,crowded", [(0, 1, False), (0, 0, False), (3, 2, False),
                                              (0, 1, True)])
def test_resample_to_map_planned(capi, oracle, P, interp, crowded):
    MH, MW, H, W = 40, 56, 48, 80    # about 2.3 taps per target (x P): lists of 16 suffice
    if P:
        MH, MW = 20, 28
    m, iw, x = _resample_case(7 + P + interp, MH, MW, H, W, P, crowded)
    tm, tiw, tx = _t(m), _t(iw), _t(x)
    B, C = x.shape[:2]
    plan, n, complete = _build_resample_plan(capi, tm, tiw, H, W, 1, P, interp)
    assert complete == (0 if crowded else 1)
    want = oracle.resample_to_map(x, m, H, W, interp, iw)
    ws = torch.empty(n, dtype=torch.uint8, device=DEV)
    plain = torch.empty(B, C, H, W, device=DEV)
    capi.call("sdk_resample_to_map", _p(tx), _p(tm), _p(tiw), _p(plain), None, _p(ws), n, B, C, MH,
              MW, H, W, P, interp, F32, _stream())
    assert relerr(_n(plain), want) <= 1e-5
    # plan_complete as reported, and 0 (fallback launches kept) in any case
    for flag in sorted({complete, 0}):
        out = torch.full((B, C, H, W), float("nan"), device=DEV)
        capi.call("sdk_resample_to_map_planned", _p(tx), _p(tm), _p(tiw), _p(out), None, _p(plan),
                  n, flag, 0, 0.0, B, C, MH, MW, H, W, P, interp, F32, _stream())
        assert relerr(_n(out), want) <= 1e-5
        # (the fallback adds hundreds of terms to the crowded pixel with float atomics)
        assert relerr(_n(out), _n(plain)) <= (1e-5 if crowded else 1e-6)
    if complete:   # a complete plan needs neither the map nor the weights
        out = torch.full((B, C, H, W), float("nan"), device=DEV)
        capi.call("sdk_resample_to_map_planned", _p(tx), None, None, _p(out), None, _p(plan), n, 1,
                  0, 0.0, B, C, MH, MW, H, W, P, interp, F32, _stream())
        assert relerr(_n(out), want) <= 1e-5
    # normalised, with the weight sum
    out = torch.full((B, C, H, W), float("nan"), device=DEV)
    wsum = torch.full((H, W), float("nan"), device=DEV)
    capi.call("sdk_resample_to_map_planned", _p(tx), _p(tm), _p(tiw), _p(out), _p(wsum), _p(plan),
              n, complete, 1, 1e-12, B, C, MH, MW, H, W, P, interp, F32, _stream())
    ones = oracle.resample_to_map(np.ones((1, 1, MH, MW), np.float32), m, H, W, interp, iw)[0, 0]
    assert relerr(_n(wsum), ones) <= 1e-5
    assert relerr(_n(out), want / (ones + 1e-12)) <= 1e-5


def _pool_map(rng, OH, OW, K, H, W, P):
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / K
    cx = xs[..., None] * (W / OW) + 1.2 * np.cos(ang) + rng.uniform(-0.3, 0.3, (OH, OW, K))
    cy = ys[..., None] * (H / OH) + 1.2 * np.sin(ang) + rng.uniform(-0.3, 0.3, (OH, OW, K))
    if P:
        cx = cx[..., None] + rng.uniform(-0.5, 0.5, (OH, OW, K, P))
        cy = cy[..., None] + rng.uniform(-0.5, 0.5, (OH, OW, K, P))
    m = np.stack([cx, cy], -1).astype(np.float32)
    iw = rng.uniform(0.1, 1, m.shape[:-1]).astype(np.float32) if P else None
    return np.ascontiguousarray(m), iw


@pytest.mark.parametrize("P,interp", [(0, 0), (0, 1), (2, 2)])
def test_avg_unpool_planned(capi, oracle, P, interp):
    rng = np.random.default_rng(21 + P)
    OH, OW, K, H, W = 20, 28, 5, 40, 56
    m, iw = _pool_map(rng, OH, OW, K, H, W, P)
    g = rng.standard_normal((2, 6, OH, OW)).astype(np.float32)
    tm, tiw, tg = _t(m), _t(iw), _t(g)
    B, C = g.shape[:2]
    n = capi.load().sdk_resample_to_map_workspace_bytes(H, W, F32)
    plan = torch.empty(n, dtype=torch.uint8, device=DEV)
    capi.call("sdk_resample_to_map_plan_build", _p(tm), _p(tiw), _p(plan), n, OH, OW, H, W, K, P,
              interp, F32, _stream())
    flag = ctypes.c_int32(-1)
    capi.call("sdk_resample_plan_complete", _p(plan), n, _stream(),
              ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
    # every tile's window of the pooled grid is small here, so the call runs tiled over the
    # image and the lists (which K * P * 4 = 40 taps per pooled pixel would overfill in the
    # weighted case) are not needed
    assert flag.value == 3          # no fallback needed (1), the tiled kernel runs (2)
    want = oracle.mapped_avg_unpool(g, m, H, W, K, interp, iw)
    for complete in sorted({int(flag.value), 0}):
        out = torch.full((B, C, H, W), float("nan"), device=DEV)
        capi.call("sdk_mapped_avg_unpool_planned", _p(tg), _p(tm), _p(tiw), _p(out), _p(plan), n,
                  complete, B, C, H, W, OH, OW, K, P, interp, F32, _stream())
        assert relerr(_n(out), want) <= 1e-5


@pytest.mark.parametrize("K,want_flag", [(2, 1), (8, 0)])
def test_avg_unpool_of_a_scattered_map(capi, oracle, K, want_flag):
    """Samples anywhere in the image: every image tile is reached from all over the pooled grid
    (96 x 96 > 8192 pooled pixels per window), so the tiled kernel stands back and the call
    gathers through the lists (K = 2, nearest taps: about 4.5 sources per image pixel) or, where those
    overflow (K = 8: about 18), falls back to the atomic scatter; planned with either
    plan_complete value, and unplanned with the call's own workspace and without one."""
    rng = np.random.default_rng(5 + K)
    OH, OW, H, W = 96, 96, 64, 64
    m = np.stack([rng.uniform(-0.4, W - 0.6, (OH, OW, K)),
                  rng.uniform(-0.4, H - 0.6, (OH, OW, K))], -1).astype(np.float32)
    g = rng.standard_normal((2, 3, OH, OW)).astype(np.float32)
    tm, tg = _t(m), _t(g)
    B, C = g.shape[:2]
    n = capi.load().sdk_resample_to_map_workspace_bytes(H, W, F32)
    plan = torch.empty(n, dtype=torch.uint8, device=DEV)
    capi.call("sdk_resample_to_map_plan_build", _p(tm), None, _p(plan), n, OH, OW, H, W, K, 0,
              0, F32, _stream())
    flag = ctypes.c_int32(-1)
    capi.call("sdk_resample_plan_complete", _p(plan), n, _stream(),
              ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
    assert flag.value == want_flag
    want = oracle.mapped_avg_unpool(g, m, H, W, K, 0, None)
    for complete in sorted({int(flag.value), 0}):
        out = torch.full((B, C, H, W), float("nan"), device=DEV)
        capi.call("sdk_mapped_avg_unpool_planned", _p(tg), _p(tm), None, _p(out), _p(plan), n,
                  complete, B, C, H, W, OH, OW, K, 0, 0, F32, _stream())
        assert relerr(_n(out), want) <= 1e-5
    for ws, nws in ((torch.empty(n, dtype=torch.uint8, device=DEV), n), (None, 0)):
        out = torch.full((B, C, H, W), float("nan"), device=DEV)
        capi.call("sdk_mapped_avg_unpool", _p(tg), _p(tm), None, _p(out), _p(ws), nws, B, C, H, W,
                  OH, OW, K, 0, 0, F32, _stream())
        assert relerr(_n(out), want) <= 1e-5


@pytest.mark.parametrize("P,interp", [(0, 0), (0, 1), (2, 1)])
def test_max_unpool_planned(capi, ops, oracle, P, interp):
    rng = np.random.default_rng(33 + P)
    OH, OW, K, H, W = 24, 40, 9, 48, 80
    m, iw = _pool_map(rng, OH, OW, K, H, W, P)
    x = rng.standard_normal((2, 6, H, W)).astype(np.float32)
    g = rng.standard_normal((2, 6, OH, OW)).astype(np.float32)
    tm, tiw, tg = _t(m), _t(iw), _t(g)
    _, idx = ops.mapped_max_pool(_t(x), tm, tiw, K, interp)
    B, C = g.shape[:2]
    n = capi.load().sdk_mapped_max_unpool_workspace_bytes(H, W, F32)
    plan = torch.empty(n, dtype=torch.uint8, device=DEV)
    capi.call("sdk_mapped_max_unpool_plan_build", _p(tm), _p(plan), n, H, W, OH, OW, K, P, interp,
              F32, _stream())
    want = oracle.mapped_max_unpool(g, _n(idx), m, H, W, K, interp, iw)
    ws = torch.empty(n, dtype=torch.uint8, device=DEV)
    plain = torch.empty(B, C, H, W, device=DEV)
    capi.call("sdk_mapped_max_unpool", _p(tg), _p(idx), _p(tm), _p(tiw), _p(plain), _p(ws), n, B, C,
              H, W, OH, OW, K, P, interp, F32, _stream())
    for _ in range(2):   # the plan survives its use (only its flag word is rewritten)
        out = torch.full((B, C, H, W), float("nan"), device=DEV)
        capi.call("sdk_mapped_max_unpool_planned", _p(tg), _p(idx), _p(tm), _p(tiw), _p(out),
                  _p(plan), n, B, C, H, W, OH, OW, K, P, interp, F32, _stream())
        assert relerr(_n(out), want) <= 1e-5
        assert relerr(_n(out), _n(plain)) <= 1e-6
    # indices that name samples of other pooled pixels: the tile kernel raises the flag and
    # the call falls back, with the same plan
    bad = torch.roll(idx, shifts=(3, 5), dims=(2, 3)).contiguous()
    want_bad = oracle.mapped_max_unpool(g, _n(bad), m, H, W, K, interp, iw)
    out = torch.full((B, C, H, W), float("nan"), device=DEV)
    capi.call("sdk_mapped_max_unpool_planned", _p(tg), _p(bad), _p(tm), _p(tiw), _p(out), _p(plan),
              n, B, C, H, W, OH, OW, K, P, interp, F32, _stream())
    assert relerr(_n(out), want_bad) <= 1e-5


def test_operator_cache_follows_the_map(ops, oracle):
    MH, MW, H, W = 32, 48, 40, 64    # about 2.4 taps per target: the plan is complete
    m, _, x = _resample_case(90, MH, MW, H, W, 0)
    tm, tx = _t(m), _t(x)
    ops.set_conv_plan_cache(True)
    a = ops.resample_to_map(tx, tm, None, H, W, 1)
    b = ops.resample_to_map(tx, tm, None, H, W, 1)     # from the kept plan
    assert relerr(_n(a), oracle.resample_to_map(x, m, H, W, 1, None)) <= 1e-5
    assert torch.equal(a, b)
    tm.add_(1.25)                                      # in place: the version counter moves on
    c = ops.resample_to_map(tx, tm, None, H, W, 1)
    assert relerr(_n(c), oracle.resample_to_map(x, m + 1.25, H, W, 1, None)) <= 1e-5
    out, wsum = ops.resample_to_map_normalized(tx, tm, None, H, W, 1, 1e-12)
    ones = oracle.resample_to_map(np.ones((1, 1, MH, MW), np.float32), m + 1.25, H, W, 1, None)[0, 0]
    assert relerr(_n(wsum), ones) <= 1e-5
    ops.set_conv_plan_cache(False)
    try:
        d = ops.resample_to_map(tx, tm, None, H, W, 1)
    finally:
        ops.set_conv_plan_cache(True)
    assert relerr(_n(d), _n(c)) <= 1e-6


def test_plans_that_are_too_small_are_refused(capi):
    H, W = 16, 24
    m = torch.zeros(8, 8, 2, device=DEV)
    x = torch.zeros(1, 1, 8, 8, device=DEV)
    out = torch.zeros(1, 1, H, W, device=DEV)
    small = torch.empty(256, dtype=torch.uint8, device=DEV)
    with pytest.raises(RuntimeError):
        capi.call("sdk_resample_to_map_plan_build", _p(m), None, _p(small), 256, 8, 8, H, W, 1, 0,
                  1, F32, _stream())
    with pytest.raises(RuntimeError):
        capi.call("sdk_resample_to_map_planned", _p(x), _p(m), None, _p(out), None, _p(small), 256,
                  0, 0, 0.0, 1, 1, 8, 8, H, W, 0, 1, F32, _stream())
    with pytest.raises(RuntimeError):
        capi.call("sdk_mapped_max_unpool_plan_build", _p(m), _p(small), 64, H, W, 8, 8, 1, 0, 0,
                  F32, _stream())
