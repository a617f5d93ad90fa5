"""Seeded sweep over random small geometries: every entry-point family against the CPU oracle
with shapes, channel counts, kernel sizes, interpolation, point counts and map character
(locally coherent or scattered) drawn per seed.  The fixed cases of test_gpu_parity.py pin known
corners; this sweep looks for the ones nobody thought of (tile remainders, channel paddings,
plan / inverse-map / tiled-unpool paths and their fallbacks meeting odd sizes).
Tolerances as everywhere: nearest gather and pooling bit-exact, float32 forward 1e-5, float32
backward 1e-4, norm-relative.
"""
import numpy as np
import pytest
import torch

from conftest import relerr

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FWD, BWD = 1e-5, 1e-4


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _bias_grad_ok(got, want, g, tol=BWD):
    """grad_bias is a plain sum of thousands of signed values: its float32 rounding error scales
    with the sum of magnitudes, not with the (possibly cancelled) result, so a channel whose sum
    nearly cancels is compared against 1 % of sum |g| rather than against |sum g|."""
    scale = max(np.abs(want).max(), 1e-2 * np.abs(g).sum(axis=(0, 2, 3)).max())
    return np.abs(np.asarray(got, np.float64) - want).max() <= tol * scale


def _n(t):
    return t.detach().cpu().numpy()


def _map(rng, grid, K, P, H, W, coherent):
    """[*grid, K, (P,) 2] float32 map into an H x W image; about one sample in ten lands outside."""
    shape = tuple(grid) + (K,) + ((P,) if P else ())
    if coherent:
        gy, gx = np.meshgrid(np.arange(grid[0]), np.arange(grid[1]), indexing="ij")
        cx = gx * (W / grid[1])
        cy = gy * (H / grid[0])
        ang = 2 * np.pi * np.arange(K) / K
        rad = 0.8 + (np.arange(K) % 3)
        x = cx[..., None] + rad * np.cos(ang)
        y = cy[..., None] + rad * np.sin(ang)
        if P:
            x = x[..., None] + rng.uniform(-1, 1, shape)
            y = y[..., None] + rng.uniform(-1, 1, shape)
        x = x + rng.uniform(-0.4, 0.4, shape)
        y = y + rng.uniform(-0.4, 0.4, shape)
    else:
        x = rng.uniform(-1.5, W + 0.5, shape)
        y = rng.uniform(-1.5, H + 0.5, shape)
    snap = rng.uniform(size=shape) < 0.25          # exact pixel centres: zero-weight taps
    x = np.where(snap, np.round(x), x)
    y = np.where(snap, np.round(y), y)
    return np.ascontiguousarray(np.stack([x, y], -1).astype(np.float32))


def _geometry(seed):
    rng = np.random.default_rng(5000 + seed)
    interp = int(rng.integers(0, 3))
    P = int(rng.choice([0, 0, 1, 2, 4]))
    K = int(rng.choice([1, 2, 3, 5, 7, 9, 10]))
    H, W = int(rng.integers(1, 40)), int(rng.integers(2, 70))
    OH, OW = int(rng.integers(1, 30)), int(rng.integers(1, 50))
    if rng.uniform() < 0.2:                         # vertex lists: one-row images
        H, OH = 1, 1
        W, OW = int(rng.integers(50, 600)), int(rng.integers(50, 600))
    coherent = bool(rng.uniform() < 0.7)
    return rng, interp, P, K, H, W, OH, OW, coherent


def _conv_case(seed):
    rng, interp, P, K, H, W, OH, OW, coherent = _geometry(seed)
    B = int(rng.integers(1, 4))
    Cin, Cout = int(rng.choice([1, 3, 8, 17, 32, 40, 64, 130])), int(rng.choice([1, 4, 16, 33, 64, 96, 136]))
    m = _map(rng, (OH, OW), K, P, H, W, coherent)
    iw = rng.uniform(0.1, 1, m.shape[:-1]).astype(np.float32) if P else None
    x = rng.standard_normal((B, Cin, H, W)).astype(np.float32)
    w = (rng.standard_normal((Cout, Cin, K)) / np.sqrt(Cin * K)).astype(np.float32)
    b = rng.standard_normal(Cout).astype(np.float32)
    g = rng.standard_normal((B, Cout, OH, OW)).astype(np.float32)
    return rng, interp, K, H, W, OH, OW, B, Cin, Cout, m, iw, x, w, b, g


@pytest.mark.parametrize("seed", range(100, 116))
def test_convolution_bf16_operands(ops, oracle, seed):
    """The bf16 compute mode (operands rounded to bf16, fp32 accumulation) on the same sweep:
    1e-2 norm-relative against the float32 oracle."""
    rng, interp, K, H, W, OH, OW, B, Cin, Cout, m, iw, x, w, b, g = _conv_case(seed)
    ops.set_conv_compute("bf16")
    try:
        y = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(w), _t(b), K, interp))
        gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(w), _t(b), K, interp)
        gi, gw, gb = _n(gi), _n(gw), _n(gb)
    finally:
        ops.set_conv_compute("native")
    assert relerr(y, oracle.mapped_conv_forward(x, m, w, b, K, interp, iw)) <= 1e-2
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, interp, iw)
    assert relerr(gi, wi) <= 1e-2 and relerr(gw, ww) <= 1e-2 and _bias_grad_ok(gb, wb, g)


@pytest.mark.parametrize("seed", range(300, 324))
def test_convolution_split_operands(ops, oracle, seed):
    """The split compute mode (float32 operands as three bf16 pieces, fp32 accumulation) on the
    same sweep, at the float32 tolerances."""
    rng, interp, K, H, W, OH, OW, B, Cin, Cout, m, iw, x, w, b, g = _conv_case(seed)
    ops.set_conv_compute("split")
    try:
        y = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(w), _t(b), K, interp))
        gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(w), _t(b), K, interp)
        gi, gw, gb = _n(gi), _n(gw), _n(gb)
    finally:
        ops.set_conv_compute("native")
    assert relerr(y, oracle.mapped_conv_forward(x, m, w, b, K, interp, iw)) <= FWD
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, interp, iw)
    assert relerr(gi, wi) <= BWD and relerr(gw, ww) <= BWD and _bias_grad_ok(gb, wb, g)


@pytest.mark.parametrize("seed", range(40))
def test_convolution_and_transposed(ops, oracle, seed):
    rng, interp, K, H, W, OH, OW, B, Cin, Cout, m, iw, x, w, b, g = _conv_case(seed)
    y = _n(ops.mapped_conv_forward(_t(x), _t(m), _t(iw), _t(w), _t(b), K, interp))
    assert relerr(y, oracle.mapped_conv_forward(x, m, w, b, K, interp, iw)) <= FWD
    gi, gw, gb = ops.mapped_conv_backward(_t(g), _t(m), _t(iw), _t(x), _t(w), _t(b), K, interp)
    wi, ww, wb = oracle.mapped_conv_backward(g, m, x, w, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= BWD and relerr(_n(gw), ww) <= BWD and _bias_grad_ok(_n(gb), wb, g)
    # the transposed layer over the same map: input on the map's grid, output on the image
    xt = rng.standard_normal((B, Cin, OH, OW)).astype(np.float32)
    wt = (rng.standard_normal((Cin, Cout, K)) / np.sqrt(Cin * K)).astype(np.float32)
    yt = _n(ops.mapped_transposed_conv_forward(_t(xt), _t(m), _t(iw), _t(wt), _t(b), H, W, K, interp))
    want = oracle.mapped_transposed_conv_forward(xt, m, wt, b, H, W, K, interp, iw)
    assert relerr(yt, want) <= BWD
    gt = rng.standard_normal(want.shape).astype(np.float32)
    gi, gw, gb = ops.mapped_transposed_conv_backward(_t(gt), _t(m), _t(iw), _t(xt), _t(wt), _t(b),
                                                     K, interp)
    wi, ww, wb = oracle.mapped_transposed_conv_backward(gt, m, xt, wt, b, K, interp, iw)
    assert relerr(_n(gi), wi) <= BWD and relerr(_n(gw), ww) <= BWD and _bias_grad_ok(_n(gb), wb, gt)


@pytest.mark.parametrize("seed", range(40, 76))
def test_pooling_and_resampling(ops, oracle, seed):
    rng, interp, P, K, H, W, OH, OW, coherent = _geometry(seed)
    B, C = int(rng.integers(1, 4)), int(rng.choice([1, 3, 7, 9, 20]))
    x = rng.standard_normal((B, C, H, W)).astype(np.float32)
    # pooling
    m = _map(rng, (OH, OW), K, P, H, W, coherent)
    iw = rng.uniform(0.1, 1, m.shape[:-1]).astype(np.float32) if P else None
    val, idx = ops.mapped_max_pool(_t(x), _t(m), _t(iw), K, interp)
    wval, widx = oracle.mapped_max_pool(x, m, K, interp, iw)
    assert np.array_equal(_n(idx), widx)
    assert np.array_equal(_n(val), wval)
    g = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    want = oracle.mapped_max_unpool(g, widx, m, H, W, K, interp, iw)
    assert relerr(_n(ops.mapped_max_unpool(_t(g), idx, _t(m), _t(iw), H, W, K, interp)), want) <= BWD
    # average pooling over the same map
    got = _n(ops.mapped_avg_pool(_t(x), _t(m), _t(iw), K, interp))
    assert relerr(got, oracle.mapped_avg_pool(x, m, K, interp, iw)) <= FWD
    back = _n(ops.mapped_avg_unpool(_t(g), _t(m), _t(iw), H, W, K, interp))
    assert relerr(back, oracle.mapped_avg_unpool(g, m, H, W, K, interp, iw)) <= BWD
    # resampling over a map without the sample axis
    mr = np.ascontiguousarray(m[:, :, 0])
    iwr = None if iw is None else np.ascontiguousarray(iw[:, :, 0])
    got = _n(ops.resample_from_map(_t(x), _t(mr), _t(iwr), interp))
    wantr = oracle.resample_from_map(x, mr, interp, iwr)
    if interp == 0 and not P:
        assert np.array_equal(got, wantr)
    else:
        assert relerr(got, wantr) <= FWD
    y = rng.standard_normal((B, C, OH, OW)).astype(np.float32)
    back = _n(ops.resample_to_map(_t(y), _t(mr), _t(iwr), H, W, interp))
    assert relerr(back, oracle.resample_to_map(y, mr, H, W, interp, iwr)) <= BWD


@pytest.mark.parametrize("seed", range(200, 224))
def test_uv_resampling_voting_and_generated_maps(ops, oracle, seed):
    """The entry points either side of the mapped operators on random geometries: UV gather
    (nearest bit-exact) and its adjoint, the label vote (bit-exact), and a device-generated
    kernel map used by a pooling call against the oracle's map and pooling."""
    rng = np.random.default_rng(9000 + seed)
    interp = int(rng.integers(0, 3))
    B, C = int(rng.integers(1, 4)), int(rng.choice([1, 3, 8, 17, 40]))
    NT = int(rng.choice([1, 2, 5, 20, 80, 300]))
    TH, TW = int(rng.integers(1, 20)), int(rng.integers(2, 24))
    H, W = int(rng.integers(1, 40)), int(rng.integers(2, 120))
    tex = rng.standard_normal((B, C, NT, TH, TW)).astype(np.float32)
    if rng.uniform() < 0.5:                          # coherent: runs of pixels on one texture
        quad = np.repeat((np.arange(H) * 7 % NT)[:, None], W, 1).astype(np.int64)
        uv = np.stack(np.broadcast_arrays(np.linspace(-1, TW, W)[None, :] * rng.uniform(0.2, 1),
                                          (np.arange(H)[:, None] * 0.61) % (TH + 1) - 0.5), -1)
    else:
        quad = rng.integers(-1, NT + 1, (H, W)).astype(np.int64)
        uv = np.stack([rng.uniform(-1.5, TW + 0.5, (H, W)), rng.uniform(-1.5, TH + 0.5, (H, W))], -1)
    uv = np.ascontiguousarray(uv.astype(np.float32))
    got = _n(ops.resample_from_uv_maps(_t(tex), _t(quad), _t(uv), interp))
    want = oracle.resample_from_uv_maps(tex, quad, uv, interp)
    assert np.array_equal(got, want) if interp == 0 else relerr(got, want) <= FWD
    y = rng.standard_normal((B, C, H, W)).astype(np.float32)
    back = _n(ops.resample_to_uv_maps(_t(y), _t(quad), _t(uv), NT, TH, TW, interp))
    assert relerr(back, oracle.resample_to_uv_maps(y, quad, uv, NT, TH, TW, interp)) <= BWD
    # label vote through a random integer map
    nc = int(rng.integers(1, 9))
    oh, ow = int(rng.integers(1, 20)), int(rng.integers(1, 30))
    labels = rng.integers(-1, nc + 1, (B, 1, H, W))
    vmap = np.stack([rng.integers(-1, ow + 1, (H, W)), rng.integers(-1, oh + 1, (H, W))], -1)
    assert np.array_equal(_n(ops.voting_resample_to_map(_t(labels), _t(vmap), oh, ow, nc)),
                          oracle.voting_resample_to_map(labels, vmap, oh, ow, nc))
    # a generated kernel map feeding average pooling (float64: both maps agree to rounding)
    ih, iw_ = int(rng.integers(4, 30)), int(rng.integers(4, 50))
    kh, kw = int(rng.choice([1, 3])), int(rng.choice([1, 3, 5]))
    stride, proj = int(rng.integers(1, 4)), int(rng.integers(0, 3))
    m = ops.equirect_kernel_map(ih, iw_, kh, kw, stride, 1, proj, torch.float64, DEV)
    mo = oracle.equirect_kernel_map((ih, iw_), (kh, kw), stride, 1, proj, np.float64)
    x = rng.standard_normal((B, 2, ih, iw_))
    got = _n(ops.mapped_avg_pool(_t(x), m, None, kh * kw, 2))
    want = oracle.mapped_avg_pool(x, mo, kh * kw, 2)
    assert relerr(got, want) <= 1e-9


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_fused_kernels_against_the_unfused_path_on_random_layers(ops, seed):
    """Twenty random layers per seed (nearest, bilinear and bispherical taps, 1 to 12 samples,
    3 to 136 output channels, unit stride and stride 2, one-row grids of thousands of pixels,
    batches that make workgroups walk several tiles): the plan-driven and window kernels against
    the im2col + GEMM path of the same library, which shares none of their code.  The oracle
    pins both elsewhere; here the point is breadth at no CPU cost."""
    rng = np.random.default_rng(seed)

    def err(a, b):
        return float((a - b).abs().max() / max(b.abs().max().item(), 1e-30))

    for case in range(20):
        interp = int(rng.choice([0, 0, 1, 2]))
        K = int(rng.integers(1, 13))
        Cin = int(rng.choice([5, 16, 33, 64, 72, 100, 130, 256]))
        Cout = int(rng.choice([3, 8, 13, 32, 33, 48, 64, 65, 96, 128, 136]))
        B = int(rng.choice([1, 2, 3, 8]))
        stride = int(rng.choice([1, 1, 2]))
        OH, OW = int(rng.integers(1, 40)), int(rng.integers(16, 90))
        if rng.uniform() < 0.2:
            OH, OW = 1, int(rng.integers(200, 3000))
        H, W = OH * stride + int(rng.integers(0, 3)), OW * stride + int(rng.integers(0, 3))
        ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
        dy, dx = rng.integers(-2, 3, K), rng.integers(-3, 4, K)
        spread = float(rng.choice([0.4, 0.4, 3.0]))
        cx = stride * xs[..., None] + dx + rng.uniform(-spread, spread, (OH, OW, K))
        cy = stride * ys[..., None] + dy + rng.uniform(-spread, spread, (OH, OW, K))
        if OH == 1:
            cy = np.zeros_like(cy)
        m = _t(np.stack([cx, cy], -1).astype(np.float32))
        x = torch.randn(B, Cin, H, W, device=DEV)
        g = torch.randn(B, Cout, OH, OW, device=DEV)
        w = torch.randn(Cout, Cin, K, device=DEV) / np.sqrt(Cin * K)
        b = torch.randn(Cout, device=DEV)
        bt = torch.randn(Cin, device=DEV)
        res = {}
        try:
            for mode in ("native", "unfused"):
                ops.set_conv_compute(mode)
                y = ops.mapped_conv_forward(x, m, None, w, b, K, interp)
                gi, gw, gb = ops.mapped_conv_backward(g, m, None, x, w, b, K, interp)
                yt = ops.mapped_transposed_conv_forward(g, m, None, w, bt, H, W, K, interp)
                res[mode] = (y, gi, gw, gb, yt)
        finally:
            ops.set_conv_compute("native")
        what = dict(seed=seed, case=case, interp=interp, K=K, Cin=Cin, Cout=Cout, B=B,
                    stride=stride, OH=OH, OW=OW, H=H, W=W, spread=spread)
        for name, a, r in zip(("forward", "grad_input", "grad_weight", "grad_bias", "transposed"),
                              res["native"], res["unfused"]):
            assert err(a, r) <= BWD, (name, what)
