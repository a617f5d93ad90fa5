"""Plans kept between calls (sdk_mapped_conv_plan_build and the *_planned entry points) against
the plain entry points, which build the same plan inside every call: identical results, for
mapped and mapped transposed convolution, on maps whose tiles take every route (inside their
window, outside it, more than four rows per sample, target lists too long for the inverse
plan).  The operator-level cache must miss when a map is changed in place.
"""
import ctypes

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


def _case(seed, Cin, Cout, H, W, OH, OW, K, P, interp, kind):
    rng = np.random.default_rng(seed)
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / K
    cx = xs[..., None] * (W / OW) + 1.5 * np.cos(ang)
    cy = ys[..., None] * (H / OH) + 1.5 * np.sin(ang)
    if kind == "polar":          # rows near the top spread their samples wide, as near a pole
        spread = 1.0 + 30.0 / (1.0 + ys[..., None])
        cx = xs[..., None] * (W / OW) + spread * 1.5 * np.cos(ang)
    if kind == "crowded":        # a fifth of the samples land on one spot: long target lists
        sel = rng.uniform(size=cx.shape) < 0.2
        cx = np.where(sel, 5.3, cx)
        cy = np.where(sel, 4.1, cy)
    if kind == "listed":
        # One-row image, nearest, K = 3: the taps of a tile of 128 pixels are far apart (no box
        # fits) and touch exactly 288 distinct elements in the first tile (a listed window, full
        # to the last element), 289 in the second (one too many: a big window) and 128 + 128 +
        # 128 = 384 in the third and in every tile from the fifth on; the fourth names sixteen
        # elements eight times each.
        assert OH == 1 and K == 3 and P == 0
        p = np.arange(OW)
        t, q = p // 128, p % 128
        third = np.select([t == 0, t == 1, t == 3], [q % 32, q % 33, q % 16], q)
        cx = np.stack([q + 1000.0 * t, 300.0 + q + 1000.0 * t, 600.0 + third + 1000.0 * t], -1)
        cx = cx.reshape(1, OW, 3) % W
        cy = np.zeros_like(cx)
        m = np.ascontiguousarray(np.stack([cx, cy], -1).astype(np.float32))
        x = rng.standard_normal((2, Cin, H, W)).astype(np.float32)
        w = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(np.float32)
        b = rng.standard_normal(Cout).astype(np.float32)
        g = rng.standard_normal((2, Cout, OH, OW)).astype(np.float32)
        bt = rng.standard_normal(Cin).astype(np.float32)
        return m, None, x, w, b, g, bt
    if P:
        cx = cx[..., None] + rng.uniform(-1, 1, (OH, OW, K, P))
        cy = cy[..., None] + rng.uniform(-1, 1, (OH, OW, K, P))
    m = np.stack([cx, cy], -1) + rng.uniform(-0.4, 0.4, cx.shape + (2,))
    m = np.ascontiguousarray(m.astype(np.float32))
    iw = rng.uniform(0.1, 1, m.shape[:-1]).astype(np.float32) if P else None
    B = 2
    x = rng.standard_normal((B, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(np.float32)
    bt = rng.standard_normal(Cin).astype(np.float32)   # bias of the transposed layer (Cout -> Cin)
    return m, iw, x, w, b, g, bt


# (Cin, Cout, H, W, OH, OW, K, P, interp, kind)
CASES = [
    (72, 80, 40, 64, 40, 64, 9, 0, 1, "plain"),      # every tile inside its window
    (96, 72, 48, 96, 48, 96, 9, 0, 1, "polar"),      # top tile rows outside, the rest inside
    (80, 96, 24, 40, 24, 40, 5, 2, 1, "plain"),      # eight rows per sample: weight gradient's rest list
    (72, 72, 20, 36, 20, 36, 6, 0, 0, "crowded"),    # inverse lists overflow: scatter fallback
    (130, 40, 27, 42, 24, 42, 10, 0, 2, "plain"),    # 12 tiles (not a multiple of 8), K = 10
    (16, 24, 30, 50, 30, 50, 7, 0, 1, "plain"),      # narrow layers: kernels that ignore the plan
    (72, 80, 1, 4500, 1, 512, 3, 0, 0, "listed"),    # listed windows: 288 (fits), 289, 384 elements
    (40, 48, 1, 4500, 1, 512, 3, 0, 0, "listed"),    # ... in the 64-channel kernels
    (72, 80, 1, 33000, 1, 4096, 3, 0, 0, "listed"),  # 30 of 32 tiles with a big window
    (72, 80, 64, 96, 32, 48, 9, 0, 1, "plain"),      # stride 2: every tile's box is 19 x 35, all big
    (72, 136, 48, 64, 24, 32, 9, 2, 2, "plain"),     # ... weighted, more than 128 pixel-side channels
    (72, 48, 64, 96, 32, 48, 9, 0, 1, "plain"),      # ... 48 output channels: big tiles from the window,
    (72, 40, 64, 96, 32, 48, 9, 0, 0, "plain"),      #     the others from the plan; nearest taps
    (72, 13, 64, 96, 32, 48, 9, 0, 1, "plain"),      #     13 output channels
    (72, 80, 64, 96, 32, 48, 9, 0, 0, "plain"),      # stride 2, nearest taps, wide: one row per sample in big windows
    (72, 80, 40, 64, 40, 64, 9, 0, 0, "plain"),      # ... and in ordinary ones
]


@pytest.mark.parametrize("mode", ["native", "split", "bf16"])
@pytest.mark.parametrize("tc", CASES, ids=lambda t: "x".join(map(str, t)))
def test_planned_calls_match_plain_calls_and_the_oracle(ops, oracle, tc, mode):
    Cin, Cout, H, W, OH, OW, K, P, interp, kind = tc
    m, iw, x, w, b, g, bt = _case(7 + sum(tc[:9]), *tc)
    tol_f, tol_b = (1e-2, 1e-2) if mode == "bf16" else (1e-5, 1e-4)
    res = {}
    ops.set_conv_compute(mode)
    try:
        for cached in (False, True):
            ops.set_conv_plan_cache(cached)
            tm, tiw = _t(m), _t(iw)
            for rep in range(2 if cached else 1):       # second pass: the plan comes from the cache
                y = ops.mapped_conv_forward(_t(x), tm, tiw, _t(w), _t(b), K, interp)
                gi, gw, gb = ops.mapped_conv_backward(_t(g), tm, tiw, _t(x), _t(w), _t(b), K, interp)
                # transposed layer over the same map (Cout -> Cin channels, weight [Cout, Cin, K]):
                # its input lives on the map's grid, its output is H x W
                yt = ops.mapped_transposed_conv_forward(_t(g), tm, tiw, _t(w), _t(bt), H, W, K,
                                                        interp)
                # ... and its backward: cotangent on the H x W image, input = g on the grid
                tgi, tgw, tgb = ops.mapped_transposed_conv_backward(_t(x), tm, tiw, _t(g), _t(w),
                                                                    _t(bt), K, interp)
            res[cached] = [t.cpu().numpy() for t in (y, gi, gw, gb, yt, tgi, tgw, tgb)]
    finally:
        ops.set_conv_plan_cache(True)
        ops.set_conv_compute("native")
    y0, gi0, gw0, gb0, yt0, tgi0, tgw0, tgb0 = res[False]
    y1, gi1, gw1, gb1, yt1, tgi1, tgw1, tgb1 = res[True]
    assert np.array_equal(y0, y1)
    assert np.array_equal(tgi0, tgi1)          # a gather in either case: the same bits
    assert relerr(tgw1, tgw0) <= 1e-6 and relerr(tgb1, tgb0) <= 1e-6
    if kind == "crowded" or Cin <= 64:
        # scatter fallback (float atomics) / narrow layers (source lists in the order the
        # atomics were served): the summation order varies from run to run
        # (with bf16 operands a last-bit difference of a column value can flip its rounding)
        loose = 1e-3 if mode == "bf16" else 1e-5
        assert relerr(gi1, gi0) <= loose and relerr(yt1, yt0) <= loose
    else:                        # gathers over sorted lists: the same bits
        assert np.array_equal(gi0, gi1)
        assert np.array_equal(yt0, yt1)
    assert relerr(gw1, gw0) <= 1e-6
    assert relerr(y1, oracle.mapped_conv_forward(x, m, w, b, K, interp, iw)) <= tol_f
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, interp, iw)
    assert relerr(gi1, wi) <= tol_b and relerr(gw1, ww) <= tol_b
    assert relerr(yt1, oracle.mapped_transposed_conv_forward(g, m, w, bt, H, W, K, interp,
                                                             iw)) <= tol_b
    ti, tw, tb = oracle.mapped_transposed_conv_backward(x, m, g, w, bt, K, interp, iw)
    assert relerr(tgi1, ti) <= tol_b and relerr(tgw1, tw) <= tol_b and relerr(tgb1, tb) <= tol_b


def test_cache_misses_after_an_in_place_change_of_the_map(ops, oracle):
    Cin, Cout, H, W, OH, OW, K, P, interp, kind = CASES[0]
    m, iw, x, w, b, g, _ = _case(3, *CASES[0])
    tm = _t(m)
    y0 = ops.mapped_conv_forward(_t(x), tm, None, _t(w), _t(b), K, interp).cpu().numpy()
    m2 = np.ascontiguousarray(m[:, ::-1].copy())
    tm.copy_(_t(m2))                                    # same storage, new contents
    y1 = ops.mapped_conv_forward(_t(x), tm, None, _t(w), _t(b), K, interp).cpu().numpy()
    assert relerr(y0, oracle.mapped_conv_forward(x, m, w, b, K, interp, None)) <= 1e-5
    assert relerr(y1, oracle.mapped_conv_forward(x, m2, w, b, K, interp, None)) <= 1e-5


def test_plan_buffer_of_the_wrong_size_is_refused(ops):
    from _spherical_distortion_ext import _capi
    lib = _capi.load()
    n = lib.sdk_mapped_conv_plan_bytes(40, 64, 40, 64, 9, 0, 1, _capi.SDK_F32)
    assert n > 0
    assert lib.sdk_mapped_conv_plan_bytes(40, 64, 40, 64, 9, 0, 1, _capi.SDK_F64) == 0
    one = ctypes.c_void_p(256)   # never dereferenced: the size check comes first
    rc = lib.sdk_mapped_conv_plan_build(one, None, one, n - 1, 40, 64, 40, 64, 9, 0, 1,
                                        _capi.SDK_F32, None)
    assert rc != 0 and b"needs" in lib.sdk_last_error()


def test_every_planned_entry_point_refuses_a_plan_that_is_too_small(ops):
    """All eight *_planned entry points check plan_bytes against the geometry's plan before
    they launch anything (the combined backward calls before their bias gradient too)."""
    from _spherical_distortion_ext import _capi
    lib = _capi.load()
    B, Cin, Cout, H, W, K = 1, 72, 80, 40, 64, 9
    n = lib.sdk_mapped_conv_plan_bytes(H, W, H, W, K, 0, 1, _capi.SDK_F32)
    nws = lib.sdk_mapped_conv_workspace_bytes(B, Cin, Cout, H, W, H, W, K, 0, 1, _capi.SDK_F32, 0)
    buf = lambda *shape: torch.zeros(shape, dtype=torch.float32, device=DEV)
    m, x, y = buf(H, W, K, 2), buf(B, Cin, H, W), buf(B, Cout, H, W)
    w, wt, b = buf(Cout, Cin, K), buf(Cin, Cout, K), buf(Cout)
    gw, gb = buf(Cout, Cin, K), buf(Cout)
    ws = torch.empty(nws, dtype=torch.uint8, device=DEV)
    plan = torch.empty(n, dtype=torch.uint8, device=DEV)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    dims = (B, Cin, H, W, Cout, H, W, K, 0, 1, _capi.SDK_F32, 0, None)
    tail = (P(ws), nws, P(plan), n - 256)
    calls = {
        "sdk_mapped_conv_forward_planned": (P(x), P(m), None, P(w), P(b), P(y)),
        "sdk_mapped_conv_backward_input_planned": (P(y), P(m), None, P(w), P(x)),
        "sdk_mapped_conv_backward_weight_planned": (P(y), P(m), None, P(x), P(gw)),
        "sdk_mapped_conv_backward_planned": (P(y), P(m), None, P(x), P(w), P(x), P(gw), P(gb)),
        # transposed layer Cin -> Cout over the same map: input on the grid, output H x W
        "sdk_mapped_transposed_conv_forward_planned": (P(x), P(m), None, P(wt), P(b), P(y)),
        "sdk_mapped_transposed_conv_backward_input_planned": (P(y), P(m), None, P(wt), P(x)),
        "sdk_mapped_transposed_conv_backward_weight_planned": (P(y), P(m), None, P(x), P(gw)),
        "sdk_mapped_transposed_conv_backward_planned": (P(y), P(m), None, P(x), P(wt), P(x), P(gw),
                                                        P(gb)),
    }
    for name, args in calls.items():
        rc = getattr(lib, name)(*args, *tail, *dims)
        assert rc == -3, (name, rc, lib.sdk_last_error())
        assert b"plan buffer" in lib.sdk_last_error(), name
    torch.cuda.synchronize()
    assert float(gb.abs().max()) == 0.0       # no bias gradient was launched by a refused call


def test_maps_made_under_inference_mode_go_past_the_cache(ops, oracle):
    """A tensor created under torch.inference_mode() has no version counter; the cached
    operators take the uncached entry points for it instead of failing."""
    Cin, Cout, H, W, OH, OW, K, P, interp, kind = CASES[0]
    m, iw, x, w, b, g, _ = _case(11, *CASES[0])
    before = ops.plan_cache_size()
    with torch.inference_mode():
        tm = _t(m)
        assert tm.is_inference()
        y = ops.mapped_conv_forward(_t(x), tm, None, _t(w), _t(b), K, interp).cpu().numpy()
        pooled, idx = ops.mapped_max_pool(_t(x), tm, None, K, interp)
        back = ops.mapped_max_unpool(pooled, idx, tm, None, H, W, K, interp).cpu().numpy()
        up = ops.resample_to_map(_t(x), _t(m[:, :, 0]), None, H, W, interp).cpu().numpy()
    assert ops.plan_cache_size() == before
    assert relerr(y, oracle.mapped_conv_forward(x, m, w, b, K, interp, None)) <= 1e-5
    pv, pi = oracle.mapped_max_pool(x, m, K, interp)
    assert np.array_equal(idx.cpu().numpy(), pi)
    assert relerr(back, oracle.mapped_max_unpool(pv, pi, m, H, W, K, interp)) <= 1e-4
    assert relerr(up, oracle.resample_to_map(x, m[:, :, 0], H, W, interp)) <= 1e-4


def test_a_plan_is_not_built_under_graph_capture(ops):
    """A key that misses while the stream is being captured takes the uncached entry points:
    nothing is inserted into the cache, and the replayed graph gives the eager result."""
    Cin, Cout, H, W, OH, OW, K, P, interp, kind = CASES[0]
    m, iw, x, w, b, g, _ = _case(13, *CASES[0])
    tx, tw, tb = _t(x), _t(w), _t(b)
    tm = _t(m)
    eager = ops.mapped_conv_forward(tx, _t(m), None, tw, tb, K, interp)   # another map tensor
    before = ops.plan_cache_size()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        out = torch.empty_like(eager)
        with torch.cuda.graph(graph, stream=side):
            out.copy_(ops.mapped_conv_forward(tx, tm, None, tw, tb, K, interp))
    assert ops.plan_cache_size() == before
    for _ in range(3):
        out.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def test_backward_runs_in_the_arithmetic_of_its_forward(ops, oracle):
    """A layer built with compute="bf16" rounds its operands in forward and backward whatever
    the process default says at backward time; a default layer follows the default."""
    from spherical_distortion import nn as sdnn
    m, iw, x, w, b, g, _ = _case(5, 72, 80, 24, 32, 24, 32, 9, 0, 1, "plain")
    tm, tx, tg = _t(m), _t(x), _t(g)

    def run(layer):
        with torch.no_grad():
            layer.weight.copy_(_t(w))
            layer.bias.copy_(_t(b))
        xin = tx.clone().requires_grad_(True)
        y = layer(xin, tm)
        y.backward(tg)
        return y.detach(), xin.grad, layer.weight.grad

    native = run(sdnn.MappedConvolution(72, 80, 9).to(DEV))
    layer = sdnn.MappedConvolution(72, 80, 9, compute="bf16").to(DEV)
    with torch.no_grad():
        layer.weight.copy_(_t(w))
        layer.bias.copy_(_t(b))
    xin = tx.clone().requires_grad_(True)
    y = layer(xin, tm)
    ops.set_conv_compute("unfused")        # must not reach the backward of the bf16 layer
    try:
        y.backward(tg)
    finally:
        ops.set_conv_compute("native")
    ops.set_conv_compute("bf16")
    try:
        want = run(sdnn.MappedConvolution(72, 80, 9).to(DEV))
    finally:
        ops.set_conv_compute("native")
    assert torch.equal(y.detach(), want[0])
    assert torch.equal(xin.grad, want[1])
    assert relerr(layer.weight.grad.cpu().numpy(), want[2].cpu().numpy()) <= 1e-6
    # and bf16 is visibly not the native arithmetic
    assert not torch.equal(y.detach(), native[0])
    assert relerr(y.detach().cpu().numpy(), native[0].cpu().numpy()) <= 1e-2
