"""Pins the CPU oracle against (a) fixtures produced by the reference's own compiled
CPU code for the variants its tests do not cover, and (b) what the mathematics fixes:
torch closed forms, the adjoint identity and a brute-force dense operator."""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import GOLDEN_DIR, relerr

DT = {"f64": np.float64, "f32": np.float32}
# float32 results of the reference are themselves rounded; allow a few ulps on sums
TOL = {"f64": 1e-12, "f32": 2e-6}
H, W, K = 6, 7, 3


@pytest.fixture(scope="module")
def fx():
    return np.load(os.path.join(GOLDEN_DIR, "ref_fixtures.npz"))


def _in(fx, d, name):
    return fx["%s/in/%s" % (d, name)]


@pytest.mark.parametrize("d", ["f64", "f32"])
@pytest.mark.parametrize("interp", [0, 1, 2])
class TestAgainstCompiledReference:
    def test_gather_is_bit_exact(self, oracle, fx, d, interp):
        pre = "%s/i%d/" % (d, interp)
        x = _in(fx, d, "x")
        out = oracle.resample_from_map(x, _in(fx, d, "r_u"), interp)
        assert np.array_equal(out, fx[pre + "from"])
        out = oracle.resample_from_map(x, _in(fx, d, "r_w"), interp, _in(fx, d, "riw"))
        assert np.array_equal(out, fx[pre + "wfrom"])

    def test_scatter(self, oracle, fx, d, interp):
        pre = "%s/i%d/" % (d, interp)
        rin = _in(fx, d, "rin")
        out = oracle.resample_to_map(rin, _in(fx, d, "r_u"), H, W, interp)
        assert relerr(out, fx[pre + "to"]) <= TOL[d]
        out = oracle.resample_to_map(rin, _in(fx, d, "r_w"), H, W, interp, _in(fx, d, "riw"))
        assert relerr(out, fx[pre + "wto"]) <= TOL[d]

    @pytest.mark.parametrize("weighted", [False, True])
    def test_conv(self, oracle, fx, d, interp, weighted):
        pre = "%s/i%d/%s" % (d, interp, "w" if weighted else "")
        m = _in(fx, d, "m_w" if weighted else "m_u")
        iw = _in(fx, d, "iw") if weighted else None
        x, wt, b, g = (_in(fx, d, n) for n in ("x", "weight", "bias", "gout"))
        out = oracle.mapped_conv_forward(x, m, wt, b, K, interp, iw)
        assert relerr(out, fx[pre + "conv_fwd"]) <= TOL[d]
        gi, gw, gb = oracle.mapped_conv_backward(g, m, x, wt, b, K, interp, iw)
        assert relerr(gi, fx[pre + "conv_gi"]) <= TOL[d]
        assert relerr(gw, fx[pre + "conv_gw"]) <= TOL[d]
        assert relerr(gb, fx[pre + "conv_gb"]) <= TOL[d]

    @pytest.mark.parametrize("weighted", [False, True])
    def test_transposed_conv(self, oracle, fx, d, interp, weighted):
        pre = "%s/i%d/%s" % (d, interp, "w" if weighted else "")
        m = _in(fx, d, "m_w" if weighted else "m_u")
        iw = _in(fx, d, "iw") if weighted else None
        x, wt, b, g = (_in(fx, d, n) for n in ("tx", "tweight", "bias", "tgout"))
        oh, ow = g.shape[2:]
        out = oracle.mapped_transposed_conv_forward(x, m, wt, b, oh, ow, K, interp, iw)
        assert relerr(out, fx[pre + "tconv_fwd"]) <= TOL[d]
        gi, gw, gb = oracle.mapped_transposed_conv_backward(g, m, x, wt, b, K, interp, iw)
        assert relerr(gi, fx[pre + "tconv_gi"]) <= TOL[d]
        assert relerr(gw, fx[pre + "tconv_gw"]) <= TOL[d]
        assert relerr(gb, fx[pre + "tconv_gb"]) <= TOL[d]

    @pytest.mark.parametrize("weighted", [False, True])
    def test_pool_values_and_indices_host_branch(self, oracle, fx, d, interp, weighted):
        """Values, index encoding, first-maximum tie-break and the host branch's
        (min(), -1) result on windows without a positive sample: all bit-exact."""
        pre = "%s/i%d/%s" % (d, interp, "w" if weighted else "")
        for src, tag, mname in (("x", "pool", "m_"), ("xneg", "poolneg", "m_"),
                                ("xpos", "pospool", "m_")):
            inside = tag == "pospool"
            m = _in(fx, d, mname + ("w" if weighted else "u") + ("i" if inside else ""))
            iw = _in(fx, d, "iw") if weighted else None
            val, idx = oracle.mapped_max_pool(_in(fx, d, src), m, K, interp, iw,
                                              host_init_quirk=True)
            assert np.array_equal(idx, fx[pre + tag + "_idx"])
            assert np.array_equal(val, fx[pre + tag + "_val"])

    @pytest.mark.parametrize("weighted", [False, True])
    def test_device_branch_differs_only_without_positive_sample(self, oracle, fx, d, interp,
                                                                weighted):
        """Starting from -FLT_MAX (the reference's device branch) changes the result
        exactly where the host branch reports index -1, and there it must be the true
        arg-max of the K gathered samples."""
        m = _in(fx, d, "m_w" if weighted else "m_u")
        iw = _in(fx, d, "iw") if weighted else None
        for src in ("x", "xneg"):
            x = _in(fx, d, src)
            vh, ih = oracle.mapped_max_pool(x, m, K, interp, iw, host_init_quirk=True)
            vd, idd = oracle.mapped_max_pool(x, m, K, interp, iw, host_init_quirk=False)
            same = ih >= 0
            assert np.array_equal(idd[same], ih[same]) and np.array_equal(vd[same], vh[same])
            col = np.stack([oracle.mapped_im2col(x[b], m, interp, iw) for b in range(x.shape[0])])
            B, C = x.shape[:2]
            col = col.reshape(B, C, K, -1)
            assert np.array_equal(vd.reshape(B, C, -1), col.max(2))
            q = 1 if iw is None else iw.shape[-1]
            kbest = col.argmax(2)  # first maximum
            pix = np.arange(col.shape[-1])
            assert np.array_equal(idd.reshape(B, C, -1), (pix * K + kbest) * q * 2)

    @pytest.mark.parametrize("weighted", [False, True])
    def test_unpool(self, oracle, fx, d, interp, weighted):
        pre = "%s/i%d/%s" % (d, interp, "w" if weighted else "")
        m = _in(fx, d, "m_wi" if weighted else "m_ui")
        iw = _in(fx, d, "iw") if weighted else None
        out = oracle.mapped_max_unpool(_in(fx, d, "gpool"), fx[pre + "pospool_idx"], m, H, W, K,
                                       interp, iw)
        assert relerr(out, fx[pre + "unpool"]) <= TOL[d]


# ------------------------------------------------------------------------------------------
# Closed forms and invariants (no reference involved).
# ------------------------------------------------------------------------------------------
def _rand_map(rng, shape, h, w, margin=1.5):
    xy = rng.uniform(-margin, [w - 1 + margin, h - 1 + margin], size=tuple(shape) + (2,))
    return np.ascontiguousarray(xy)


def test_bilinear_equals_grid_sample_zero_padding(oracle):
    rng = np.random.default_rng(0)
    x = rng.standard_normal((2, 3, 9, 11))
    m = _rand_map(rng, (5, 6), 9, 11)
    out = oracle.resample_from_map(x, m, 1)
    grid = np.stack([2 * m[..., 0] / (11 - 1) - 1, 2 * m[..., 1] / (9 - 1) - 1], -1)
    ref = F.grid_sample(torch.from_numpy(x), torch.from_numpy(grid)[None].expand(2, -1, -1, -1),
                        mode="bilinear", padding_mode="zeros", align_corners=True).numpy()
    np.testing.assert_allclose(out, ref, atol=1e-12)


def test_bispherical_equals_grid_sample_on_circularly_padded_image(oracle):
    rng = np.random.default_rng(1)
    h, w = 7, 10
    x = rng.standard_normal((1, 2, h, w))
    m = _rand_map(rng, (6, 6), h, w, margin=0.0)
    m[..., 0] = rng.uniform(-1.0, w, size=m.shape[:-1])  # x in [-1, w): wraps on both sides
    out = oracle.resample_from_map(x, m, 2)
    xp = np.concatenate([x[..., -1:], x, x[..., :1]], -1)  # one wrapped column each side
    grid = np.stack([2 * (m[..., 0] + 1) / (w + 2 - 1) - 1, 2 * m[..., 1] / (h - 1) - 1], -1)
    ref = F.grid_sample(torch.from_numpy(xp), torch.from_numpy(grid)[None], mode="bilinear",
                        padding_mode="zeros", align_corners=True).numpy()
    np.testing.assert_allclose(out, ref, atol=1e-12)


def test_nearest_rounds_half_away_from_zero_and_does_not_wrap(oracle):
    x = np.arange(12, dtype=np.float64).reshape(1, 1, 3, 4)
    xs = np.array([-0.5, -0.49, 0.5, 1.5, 2.5, 3.49, 3.5, 0.0])
    m = np.stack([xs, np.full_like(xs, 1.0)], -1).reshape(1, -1, 2)
    out = oracle.resample_from_map(x, m, 0).reshape(-1)
    #            -0.5 -> -1 (out)  -0.49 -> 0   0.5 -> 1  1.5 -> 2  2.5 -> 3  3.49 -> 3  3.5 -> 4 (out)
    assert out.tolist() == [0.0, 4.0, 5.0, 6.0, 7.0, 7.0, 0.0, 4.0]


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("weighted", [False, True])
def test_scatter_is_the_transpose_of_gather(oracle, interp, weighted):
    """Brute force: build the dense [map pixels x image pixels] gather operator column by
    column from unit images; scatter must equal its transpose, hence <Gx, y> = <x, G^T y>."""
    rng = np.random.default_rng(2 + interp)
    h, w, mh, mw, P = 4, 5, 3, 4, 3
    m = _rand_map(rng, (mh, mw, P) if weighted else (mh, mw), h, w)
    m[0, 0] = np.round(m[0, 0])
    iw = rng.uniform(0.1, 1.0, (mh, mw, P)) if weighted else None
    eye = np.eye(h * w).reshape(h * w, 1, h, w)
    G = oracle.resample_from_map(eye, m, interp, iw).reshape(h * w, mh * mw).T  # [map, image]
    y = rng.standard_normal((2, 3, mh, mw))
    st = oracle.resample_to_map(y, m, h, w, interp, iw)
    np.testing.assert_allclose(st.reshape(6, h * w), y.reshape(6, mh * mw) @ G, atol=1e-12)
    if interp == 0 and not weighted:  # nearest rows are one-hot or empty
        assert set(np.unique(G)) <= {0.0, 1.0} and (G.sum(1) <= 1).all()


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("weighted", [False, True])
def test_col2im_and_unpool_are_adjoints(oracle, interp, weighted):
    rng = np.random.default_rng(10 + interp)
    c, h, w, oh, ow, k, P = 2, 5, 6, 3, 4, 3, 2
    m = _rand_map(rng, (oh, ow, k, P) if weighted else (oh, ow, k), h, w)
    iw = rng.uniform(0.1, 1.0, (oh, ow, k, P)) if weighted else None
    x = rng.standard_normal((c, h, w))
    col = rng.standard_normal((c * k, oh * ow))
    lhs = (oracle.mapped_im2col(x, m, interp, iw) * col).sum()
    rhs = (x * oracle.mapped_col2im(col, m, h, w, interp, iw)).sum()
    assert abs(lhs - rhs) <= 1e-12 * max(1.0, abs(lhs))
    # unpool = col2im restricted to the winning sample
    xb = np.abs(x[None]) + 0.5
    mi = np.ascontiguousarray(np.clip(m, 0, [w - 1, h - 1]))
    val, idx = oracle.mapped_max_pool(xb, mi, k, interp, iw)
    g = rng.standard_normal(val.shape)
    q = P if weighted else 1
    kbest = (idx // (2 * q)) % k
    onehot = np.zeros((c, k, oh * ow))
    np.put_along_axis(onehot, kbest.reshape(c, 1, -1), g.reshape(c, 1, -1), 1)
    want = oracle.mapped_col2im(onehot.reshape(c * k, -1), mi, h, w, interp, iw)
    got = oracle.mapped_max_unpool(g, idx, mi, h, w, k, interp, iw)[0]
    np.testing.assert_allclose(got, want, atol=1e-12)


def test_regular_grid_map_reduces_to_conv2d(oracle):
    """An integer 3x3 grid map makes mapped convolution a plain zero-padded convolution."""
    rng = np.random.default_rng(5)
    b, cin, cout, h, w = 2, 3, 4, 6, 7
    x = rng.standard_normal((b, cin, h, w))
    wt = rng.standard_normal((cout, cin, 9))
    bias = rng.standard_normal(cout)
    ys, xs = np.meshgrid(np.arange(h), np.arange(w), indexing="ij")
    di, dj = np.meshgrid([-1, 0, 1], [-1, 0, 1], indexing="ij")
    m = np.stack([xs[..., None] + dj.reshape(-1), ys[..., None] + di.reshape(-1)], -1).astype(float)
    g = rng.standard_normal((b, cout, h, w))
    xt = torch.from_numpy(x).requires_grad_()
    wtt = torch.from_numpy(wt.reshape(cout, cin, 3, 3)).requires_grad_()
    bt = torch.from_numpy(bias).requires_grad_()
    ref = F.conv2d(xt, wtt, bt, padding=1)
    ref.backward(torch.from_numpy(g))
    for interp in (0, 1):
        out = oracle.mapped_conv_forward(x, m, wt, bias, 9, interp)
        np.testing.assert_allclose(out, ref.detach().numpy(), atol=1e-12)
        gi, gw, gb = oracle.mapped_conv_backward(g, m, x, wt, bias, 9, interp)
        np.testing.assert_allclose(gi, xt.grad.numpy(), atol=1e-12)
        np.testing.assert_allclose(gw.reshape(cout, cin, 3, 3), wtt.grad.numpy(), atol=1e-11)
        np.testing.assert_allclose(gb, bt.grad.numpy(), atol=1e-11)


def test_transposed_forward_is_conv_backward_input(oracle):
    rng = np.random.default_rng(6)
    b, cin, cout, ih, iw_, oh, ow, k = 2, 3, 2, 3, 4, 5, 6, 4
    m = _rand_map(rng, (ih, iw_, k), oh, ow)
    x = rng.standard_normal((b, cin, ih, iw_))
    wt = rng.standard_normal((cin, cout, k))
    out = oracle.mapped_transposed_conv_forward(x, m, wt, np.zeros(cout), oh, ow, k, 1)
    # conv with weight [Cout'=cin, Cin'=cout, K] whose backward-input maps x -> out
    gi, _, _ = oracle.mapped_conv_backward(x, m, np.zeros((b, cout, oh, ow)), wt, np.zeros(cin),
                                           k, 1)
    np.testing.assert_allclose(out, gi, atol=1e-12)


@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("weighted", [False, True])
def test_avg_pool_is_the_mean_of_im2col_rows_and_unpool_its_adjoint(oracle, interp, weighted):
    """Average pooling is pinned through functions pinned above: its value is the mean over k of
    the im2col rows (summed in ascending k, then divided), and the unpool is its exact adjoint,
    i.e. col2im of grad / K repeated over the K samples."""
    rng = np.random.default_rng(40 + interp)
    b, c, h, w, oh, ow, k, p = 2, 3, 9, 11, 5, 7, 4, 2
    x = rng.standard_normal((b, c, h, w))
    m = np.stack([rng.uniform(-1.5, w + 0.5, (oh, ow, k, p) if weighted else (oh, ow, k)),
                  rng.uniform(-1.5, h + 0.5, (oh, ow, k, p) if weighted else (oh, ow, k))], -1)
    iw = rng.uniform(0.1, 1, (oh, ow, k, p)) if weighted else None
    got = oracle.mapped_avg_pool(x, m, k, interp, iw)
    col = np.stack([oracle.mapped_im2col(x[i], m, interp, iw) for i in range(b)])
    col = col.reshape(b, c, k, oh, ow)
    want = np.zeros((b, c, oh, ow))
    for kk in range(k):
        want = want + col[:, :, kk]
    want = want / k
    assert np.array_equal(got, want)
    g = rng.standard_normal((b, c, oh, ow))
    back = oracle.mapped_avg_unpool(g, m, h, w, k, interp, iw)
    assert abs((got * g).sum() - (x * back).sum()) <= 1e-10 * np.abs(got * g).sum()
    cols = np.repeat((g / k)[:, :, None], k, axis=2).reshape(b, c * k, oh * ow)
    via = np.stack([oracle.mapped_col2im(cols[i], m, h, w, interp, iw) for i in range(b)])
    assert relerr(back, via) <= 1e-13


# ----------------------------------------------------------------------------- average pooling
# and UV resampling against the compiled reference (tests/golden/ref_fixtures_avg_uv.npz)
@pytest.fixture(scope="module")
def fx2():
    return np.load(os.path.join(GOLDEN_DIR, "ref_fixtures_avg_uv.npz"))


@pytest.mark.parametrize("d", ["f64", "f32"])
@pytest.mark.parametrize("interp", [0, 1, 2])
class TestAvgPoolAndUVAgainstCompiledReference:
    @pytest.mark.parametrize("weighted", [False, True])
    def test_avg_pool_and_unpool(self, oracle, fx2, d, interp, weighted):
        pre = "%s/i%d/%s" % (d, interp, "w" if weighted else "")
        m = _in(fx2, d, "m_w" if weighted else "m_u")
        iw = _in(fx2, d, "iw") if weighted else None
        x, g = _in(fx2, d, "x"), _in(fx2, d, "g")
        assert np.array_equal(oracle.mapped_avg_pool(x, m, K, interp, iw), fx2[pre + "avg_pool"])
        back = oracle.mapped_avg_unpool(g, m, x.shape[2], x.shape[3], K, interp, iw)
        assert relerr(back, fx2[pre + "avg_unpool"]) <= TOL[d]

    def test_uv_gather_is_bit_exact_and_its_adjoint(self, oracle, fx2, d, interp):
        pre = "%s/i%d/" % (d, interp)
        tex, quad, uv, x = (_in(fx2, d, n) for n in ("tex", "quad", "uv", "x"))
        assert np.array_equal(oracle.resample_from_uv_maps(tex, quad, uv, interp),
                              fx2[pre + "from_uv"])
        nt, th, tw = tex.shape[2:]
        back = oracle.resample_to_uv_maps(x, quad, uv, nt, th, tw, interp)
        assert relerr(back, fx2[pre + "to_uv"]) <= TOL[d]


@pytest.mark.parametrize("interp", [0, 1, 2])
def test_uv_resampling_is_the_plain_gather_per_texture(oracle, interp):
    """A UV gather reads, for each pixel, what resample_from_map (pinned above) reads from the
    named texture alone; taps never cross into a neighbouring texture.  The other direction is
    its adjoint, and texture indices outside the range contribute nothing."""
    rng = np.random.default_rng(70 + interp)
    b, c, nt, th, tw, h, w = 2, 3, 6, 5, 8, 9, 13
    tex = rng.standard_normal((b, c, nt, th, tw))
    quad = rng.integers(0, nt, (h, w))
    uv = np.stack([rng.uniform(-1.5, tw + 0.5, (h, w)), rng.uniform(-1.5, th + 0.5, (h, w))], -1)
    got = oracle.resample_from_uv_maps(tex, quad, uv, interp)
    want = np.zeros((b, c, h, w))
    for t in range(nt):
        per = oracle.resample_from_map(np.ascontiguousarray(tex[:, :, t]), uv, interp)
        want = np.where(quad == t, per, want)
    assert np.array_equal(got, want)
    y = rng.standard_normal((b, c, h, w))
    back = oracle.resample_to_uv_maps(y, quad, uv, nt, th, tw, interp)
    assert abs((got * y).sum() - (tex * back).sum()) <= 1e-10 * np.abs(got * y).sum()
    bad = quad.copy()
    bad[::2, ::3] = nt
    bad[1::2, ::4] = -1
    masked = np.where((bad >= 0) & (bad < nt), got, 0.0)
    assert np.array_equal(oracle.resample_from_uv_maps(tex, bad, uv, interp), masked)
    ok = ((bad >= 0) & (bad < nt)).astype(np.float64)
    assert relerr(oracle.resample_to_uv_maps(y, bad, uv, nt, th, tw, interp),
                  oracle.resample_to_uv_maps(y * ok, quad, uv, nt, th, tw, interp)) <= 1e-13


# ----------------------------------------------------------------------------- voting resample
def test_voting_resample_against_compiled_reference_and_brute_force(oracle, fx2):
    labels, vmap, want = fx2["vote/in/labels"], fx2["vote/in/map"], fx2["vote/out"]
    oh, ow = want.shape[2:]
    assert np.array_equal(oracle.voting_resample_to_map(labels, vmap, oh, ow, 5), want)
    # brute force with bincount on another seeded case: most frequent label, smallest on a tie,
    # 0 where no source lands; targets outside the output and labels outside the range ignored.
    # One channel: with more the reference's histograms overlap (fixture above: 3 channels).
    rng = np.random.default_rng(8)
    b, c, ih, iw, oh, ow, nc = 4, 1, 13, 17, 5, 6, 4
    labels = rng.integers(-1, nc + 1, (b, c, ih, iw))
    vmap = np.stack([rng.integers(-1, ow + 1, (ih, iw)), rng.integers(-1, oh + 1, (ih, iw))], -1)
    got = oracle.voting_resample_to_map(labels, vmap, oh, ow, nc)
    want = np.zeros((b, c, oh, ow), np.int64)
    for bi in range(b):
        for ci in range(c):
            for y in range(oh):
                for x in range(ow):
                    src = labels[bi, ci][(vmap[..., 0] == x) & (vmap[..., 1] == y)]
                    src = src[(src >= 0) & (src < nc)]
                    if src.size:
                        want[bi, ci, y, x] = np.bincount(src, minlength=nc).argmax()
    assert np.array_equal(got, want)


# ----------------------------------------------------------------------------- gather at index
@pytest.mark.parametrize("interp", [0, 1, 2])
@pytest.mark.parametrize("weighted", [False, True])
def test_gather_at_index_is_the_transpose_of_the_pinned_unpool(oracle, interp, weighted):
    """<unpool(g), x> = <g, gather_at_index(x)> for any index tensor, and the gather at
    pooling's own indices returns pooling's values (bit-exact): the pooled value IS the image
    read at the winning sample."""
    rng = np.random.default_rng(90 + interp)
    b, c, h, w, oh, ow, k, p = 2, 3, 9, 11, 5, 7, 4, 2
    x = rng.standard_normal((b, c, h, w))
    shape = (oh, ow, k, p) if weighted else (oh, ow, k)
    m = np.stack([rng.uniform(0, w - 1, shape), rng.uniform(0, h - 1, shape)], -1)
    iw = rng.uniform(0.1, 1, shape) if weighted else None
    val, idx = oracle.mapped_max_pool(x, m, k, interp, iw)
    assert (idx >= 0).all()
    assert np.array_equal(oracle.mapped_gather_at_index(x, idx, m, interp, iw), val)
    q = p if weighted else 1
    any_idx = (rng.integers(0, k, (b, c, oh, ow)) +
               np.arange(oh * ow).reshape(oh, ow) * k) * q * 2
    any_idx[0, 0, 0, :3] = -1
    g = rng.standard_normal((b, c, oh, ow))
    g_masked = np.where(any_idx < 0, 0.0, g)
    lhs = oracle.mapped_max_unpool(g_masked, np.where(any_idx < 0, 0, any_idx), m, h, w, k,
                                   interp, iw)
    rhs = oracle.mapped_gather_at_index(x, any_idx, m, interp, iw)
    assert (rhs[0, 0, 0, :3] == 0).all()
    assert abs((lhs * x).sum() - (g * rhs).sum()) <= 1e-10 * np.abs(g * rhs).sum()
