"""The row-band unpooling kernels (float32, single nearest taps, K = 4 or 9, image width a
multiple of 4) through the C ABI against the oracle (1e-4 of the largest gradient: float32
backward, sums in an order that depends on scheduling) and against the zero fill + atomic
scatter of the call without workspace.  A workgroup owns RB whole image rows (two planes of
RB rows in 32 KB: 16 rows of 256 pixels, 8 of 512, 4 of 1024) and at most 2048 pooled pixels
that can reach them; maps that ask for more, indices that name another pixel's sample and the
other interpolations take the routes they took before, with the same results.
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


def _p(t, offset=0):
    return ctypes.c_void_p(0 if t is None else t.data_ptr() + offset)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _grid_map(OH, OW, H, W, K, rng, spread=1.0, jitter=0.3):
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / K
    cx = xs[..., None] * (W / OW) + 2.0 * spread * np.cos(ang)
    cy = ys[..., None] * (H / OH) + 2.0 * spread * np.sin(ang)
    m = np.stack([cx, cy], -1) + rng.uniform(-jitter, jitter, (OH, OW, K, 2))
    return np.ascontiguousarray(m.astype(np.float32))


def _max_unpool(capi, g, idx, m, H, W, K, how, misalign=0):
    """how: "workspace" (plain call), "none" (no workspace: atomic scatter), "planned",
    "static".  misalign: byte offset of grad_input from a 16-byte boundary."""
    B, C, OH, OW = g.shape
    lib = capi.load()
    n = lib.sdk_mapped_max_unpool_workspace_bytes(H, W, F32)
    buf = torch.full((B * C * H * W + 8,), float("nan"), device=DEV)
    dims = (B, C, H, W, OH, OW, K, 0, 0, F32, _stream())
    ws = torch.empty(max(n, 16), dtype=torch.uint8, device=DEV)
    if how == "workspace":
        capi.call("sdk_mapped_max_unpool", _p(g), _p(idx), _p(m), None, _p(buf, misalign), _p(ws),
                  n, *dims)
    elif how == "none":
        capi.call("sdk_mapped_max_unpool", _p(g), _p(idx), _p(m), None, _p(buf, misalign), None, 0,
                  *dims)
    elif how == "planned":
        capi.call("sdk_mapped_max_unpool_plan_build", _p(m), _p(ws), n, H, W, OH, OW, K, 0, 0, F32,
                  _stream())
        for _ in range(2):     # the plan survives its use
            buf.fill_(float("nan"))
            capi.call("sdk_mapped_max_unpool_planned", _p(g), _p(idx), _p(m), None,
                      _p(buf, misalign), _p(ws), n, *dims)
    else:
        capi.call("sdk_mapped_max_unpool_static", _p(g), _p(idx), _p(m), None, _p(buf, misalign),
                  *dims)
    torch.cuda.synchronize()
    lead = misalign // 4
    out = buf[lead:lead + B * C * H * W].reshape(B, C, H, W)
    assert bool(torch.isnan(buf[lead + B * C * H * W:]).all()) and bool(torch.isnan(buf[:lead]).all())
    return _n(out), int(ws[:4].view(torch.int32)[0]) if how in ("workspace", "planned") else 0


def _avg_unpool(capi, g, m, H, W, K, with_ws=True, misalign=0):
    B, C, OH, OW = g.shape
    n = capi.load().sdk_resample_to_map_workspace_bytes(H, W, F32) if with_ws else 0
    ws = torch.empty(n, dtype=torch.uint8, device=DEV) if with_ws else None
    buf = torch.full((B * C * H * W + 8,), float("nan"), device=DEV)
    capi.call("sdk_mapped_avg_unpool", _p(g), _p(m), None, _p(buf, misalign), _p(ws), n, B, C, H, W,
              OH, OW, K, 0, 0, F32, _stream())
    torch.cuda.synchronize()
    lead = misalign // 4
    return _n(buf[lead:lead + B * C * H * W].reshape(B, C, H, W))


# (B, C, H, W, OH, OW, K, what)
CASES = [
    (2, 9, 64, 512, 32, 256, 9, "stride 2, bands of 8 rows, 18 planes"),
    (1, 5, 60, 512, 30, 256, 9, "H = 60: the last band has 4 rows; odd plane count"),
    (1, 1, 40, 64, 20, 32, 9, "one plane; bands of 16 rows of 64, the last of 8"),
    (2, 3, 24, 1024, 12, 512, 4, "W = 1024: bands of 4 rows; K = 4"),
    (3, 11, 48, 96, 48, 96, 9, "stride 1: about 20 pooled rows of 96 per band"),
    (2, 4, 32, 256, 64, 48, 9, "pooled rows twice as dense as image rows: about 36 x 48 pooled pixels per band"),
]


@pytest.mark.parametrize("tc", CASES, ids=lambda t: t[-1].split(":")[0].replace(" ", "_"))
@pytest.mark.parametrize("how", ["workspace", "planned", "static"])
def test_band_unpooling_matches_the_oracle(ops, capi, oracle, tc, how):
    B, C, H, W, OH, OW, K, _ = tc
    rng = np.random.default_rng(B * 100 + C + K + H)
    m = _grid_map(OH, OW, H, W, K, rng)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    tm, tg = _t(m), _t(g)
    _, idx = ops.mapped_max_pool(_t(x), tm, None, K, 0)
    want = oracle.mapped_max_unpool(g, _n(idx), m, H, W, K, 0)
    got, gate = _max_unpool(capi, tg, idx, tm, H, W, K, how)
    assert gate == 0
    assert relerr(got, want) <= 1e-4
    if how == "workspace":
        plain, _ = _max_unpool(capi, tg, idx, tm, H, W, K, "none")
        assert relerr(got, plain) <= 1e-5
        assert relerr(_avg_unpool(capi, tg, tm, H, W, K), oracle.mapped_avg_unpool(g, m, H, W, K, 0)) <= 1e-4
        assert relerr(_avg_unpool(capi, tg, tm, H, W, K, with_ws=False),
                      oracle.mapped_avg_unpool(g, m, H, W, K, 0)) <= 1e-4


def test_band_unpooling_into_a_tensor_that_is_not_16_byte_aligned(ops, capi, oracle):
    B, C, H, W, OH, OW, K = 2, 5, 32, 128, 16, 64, 9
    rng = np.random.default_rng(8)
    m = _grid_map(OH, OW, H, W, K, rng)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    tm, tg = _t(m), _t(g)
    _, idx = ops.mapped_max_pool(_t(x), tm, None, K, 0)
    got, _ = _max_unpool(capi, tg, idx, tm, H, W, K, "workspace", misalign=4)
    assert relerr(got, oracle.mapped_max_unpool(g, _n(idx), m, H, W, K, 0)) <= 1e-4
    assert relerr(_avg_unpool(capi, tg, tm, H, W, K, misalign=8),
                  oracle.mapped_avg_unpool(g, m, H, W, K, 0)) <= 1e-4


def test_band_unpooling_stands_back_for_what_it_does_not_take(ops, capi, oracle):
    """More than 2048 pooled pixels reach a band (a pooled grid half again as fine as the image:
    about 27 x 192 per band, which the image tiles still take;
    a scattered map, whose tile windows are too large as well: atomic scatter), indices of
    other pixels' samples (the gate is raised by the band kernel itself), taps outside the
    image, whole bands nobody reaches."""
    rng = np.random.default_rng(9)
    B, C, H, W, K = 2, 3, 32, 128, 9
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    for OH, OW, scattered in [(48, 192, False), (100, 120, True)]:
        m = _grid_map(OH, OW, H, W, K, rng)
        if scattered:
            m = np.stack([rng.uniform(-0.4, W - 0.6, (OH, OW, K)),
                          rng.uniform(-0.4, H - 0.6, (OH, OW, K))], -1).astype(np.float32)
        g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
        tm, tg = _t(m), _t(g)
        _, idx = ops.mapped_max_pool(_t(x), tm, None, K, 0)
        got, gate = _max_unpool(capi, tg, idx, tm, H, W, K, "workspace")
        assert (gate > 0) == scattered
        assert relerr(got, oracle.mapped_max_unpool(g, _n(idx), m, H, W, K, 0)) <= 1e-4
        assert relerr(_avg_unpool(capi, tg, tm, H, W, K),
                      oracle.mapped_avg_unpool(g, m, H, W, K, 0)) <= 1e-4
    OH, OW = 16, 64
    m = _grid_map(OH, OW, H, W, K, rng)
    m[:, :5, :, 0] -= 30.0        # taps left of the image
    m[12:] += 100.0               # the last pooled rows reach nothing: the bottom bands stay zero
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    tm, tg = _t(m), _t(g)
    _, idx = ops.mapped_max_pool(_t(x), tm, None, K, 0)
    want = oracle.mapped_max_unpool(g, _n(idx), m, H, W, K, 0)
    got, gate = _max_unpool(capi, tg, idx, tm, H, W, K, "workspace")
    assert gate == 0 and relerr(got, want) <= 1e-4
    assert float(np.abs(got[:, :, 28:]).max()) == 0.0
    assert relerr(_avg_unpool(capi, tg, tm, H, W, K), oracle.mapped_avg_unpool(g, m, H, W, K, 0)) <= 1e-4
    bad = torch.roll(idx, shifts=(2, 7), dims=(2, 3)).contiguous()
    bad[0, 0, 0, 0] = -1
    bad[1, 2, 3, 3] = OH * OW * K * 2 + 6
    ref_idx = _n(bad).copy()
    ref_idx[1, 2, 3, 3] = -1      # past the map: contributes nothing, like a negative index
    for how in ("workspace", "planned", "static"):
        got, gate = _max_unpool(capi, tg, bad, tm, H, W, K, how)
        assert how == "static" or gate > 0
        assert relerr(got, oracle.mapped_max_unpool(g, ref_idx, m, H, W, K, 0)) <= 1e-4


def test_planned_bands_call_matches_the_planned_call(ops, capi, oracle):
    """sdk_mapped_max_unpool_plan_bands says whether one kernel does a plan's calls;
    sdk_mapped_max_unpool_planned_bands then gives the planned call's result with the flag left
    clear for the next call: indices from the pooling, then indices that name other pixels'
    samples (added behind the band kernel), then the first again on the same plan."""
    B, C, H, W, OH, OW, K = 2, 5, 32, 128, 16, 64, 9
    rng = np.random.default_rng(21)
    m = _grid_map(OH, OW, H, W, K, rng)
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    tm, tg = _t(m), _t(g)
    _, idx = ops.mapped_max_pool(_t(x), tm, None, K, 0)
    bad = torch.roll(idx, shifts=(2, 7), dims=(2, 3)).contiguous()
    bad[0, 0, 0, 0] = -1
    bad[1, 2, 3, 3] = OH * OW * K * 2 + 6
    bad[1, 1, 5, 5] = int(bad[1, 1, 5, 5]) | 1        # an odd index: y of one sample, x of the next
    ref_bad = _n(bad).copy()
    ref_bad[1, 2, 3, 3] = -1
    lib = capi.load()
    n = lib.sdk_mapped_max_unpool_workspace_bytes(H, W, F32)
    ws = torch.empty(n, dtype=torch.uint8, device=DEV)
    capi.call("sdk_mapped_max_unpool_plan_build", _p(tm), _p(ws), n, H, W, OH, OW, K, 0, 0, F32,
              _stream())
    flag = ctypes.c_int32(-1)
    capi.call("sdk_mapped_max_unpool_plan_bands", _p(ws), n, H, W, F32, _stream(),
              ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
    assert flag.value == 1
    buf = torch.empty((B, C, H, W), device=DEV)
    for which, ref_idx in ((idx, _n(idx)), (bad, ref_bad), (idx, _n(idx)), (bad, ref_bad)):
        buf.fill_(float("nan"))
        capi.call("sdk_mapped_max_unpool_planned_bands", _p(tg), _p(which), _p(tm), _p(buf), _p(ws),
                  n, B, C, H, W, OH, OW, K, 0, F32, _stream())
        torch.cuda.synchronize()
        assert int(ws[:8].view(torch.int32)[0]) == 0 and int(ws[:8].view(torch.int32)[1]) == 0
        assert relerr(_n(buf), oracle.mapped_max_unpool(g, ref_idx, m, H, W, K, 0)) <= 1e-4
    # a map the bands do not take: the query says so (and the operator layer then makes the
    # ordinary planned call)
    OH2, OW2 = 100, 120
    m2 = np.stack([rng.uniform(-0.4, W - 0.6, (OH2, OW2, K)),
                   rng.uniform(-0.4, H - 0.6, (OH2, OW2, K))], -1).astype(np.float32)
    capi.call("sdk_mapped_max_unpool_plan_build", _p(_t(m2)), _p(ws), n, H, W, OH2, OW2, K, 0, 0,
              F32, _stream())
    capi.call("sdk_mapped_max_unpool_plan_bands", _p(ws), n, H, W, F32, _stream(),
              ctypes.cast(ctypes.byref(flag), ctypes.c_void_p))
    assert flag.value == 0
    g2 = rng.standard_normal((B, C, OH2, OW2)).astype(np.float32)
    _, idx2 = ops.mapped_max_pool(_t(x), _t(m2), None, K, 0)
    got = ops.mapped_max_unpool(_t(g2), idx2, _t(m2), None, H, W, K, 0)
    assert relerr(_n(got), oracle.mapped_max_unpool(g2, _n(idx2), m2, H, W, K, 0)) <= 1e-4
    # and through the operator layer on the first map (the band variant is what it calls)
    for which, ref_idx in ((idx, _n(idx)), (bad, ref_bad), (idx, _n(idx))):
        got = ops.mapped_max_unpool(tg, which, tm, None, H, W, K, 0)
        assert relerr(_n(got), oracle.mapped_max_unpool(g, ref_idx, m, H, W, K, 0)) <= 1e-4
