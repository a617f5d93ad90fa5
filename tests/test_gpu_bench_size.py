"""Element-wise parity with the CPU oracle at the exact sizes and batches the benchmark times:
configuration 4 at batch 8 (native float32, split and bf16 arithmetic), configuration 3 at
batch 8, configuration 5 at batch 4, configuration 2 at batch 4.

Configurations 2 and 3 and the transposed up-sampling of configuration 5 are compared with the
oracle in full.  The two convolutions are compared on pixel samples (tests/sampled_parity.py:
the oracle evaluates the full image through the map sliced to the sampled pixels, which gives
exactly the full evaluation's values there): both polar row pairs, the seam columns and random
pixels for the forward and for the gradients of a grad_output that is zero elsewhere; and, for
the dense grad_output the benchmark uses, grad_input on sampled image pixels and grad_weight
on channel subsets (the oracle run on the whole map with four input and four output
channels returns the full evaluation's entries for those channels).  Every element of the
dense results of configuration 4 is also compared with the float64 kernels of the unfused
path, an independent implementation that the small-size tests compare with the oracle.

Tolerances (max|a-b| / max|b|): indices and nearest values bit-exact, float32 forward 1e-5,
float32 backward 1e-4, bf16 operands 1e-2.
"""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import sampled_parity as sp  # noqa: E402
import workloads  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FWD = {"native": 1e-5, "split": 1e-5, "bf16": 1e-2}
BWD = {"native": 1e-4, "split": 1e-4, "bf16": 1e-2}


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _n(t):
    return t.detach().cpu().numpy()


def _gpu_conv(ops, t, g, mode):
    """Forward and backward of the configuration's layer for grad_output g in one mode."""
    K, it = t["kernel_size"], t["interp"]
    ops.set_conv_compute(mode)
    try:
        y = ops.mapped_conv_forward(t["x"], t["sample_map"], t.get("interp_weights"), t["weight"],
                                    t["bias"], K, it)
        gi, gw, gb = ops.mapped_conv_backward(g, t["sample_map"], t.get("interp_weights"), t["x"],
                                              t["weight"], t["bias"], K, it)
    finally:
        ops.set_conv_compute("native")
    torch.cuda.synchronize()
    return y, gi, gw, gb


# --------------------------------------------------------------------------- configuration 4
@pytest.fixture(scope="module")
def conv4(oracle):
    cfg = workloads.config4(batch=8)
    chk = sp.ConvOracle(oracle, cfg, n_random=2048, n_targets=768, seed=40, n_weight_channels=4)
    t = {k: (_t(v) if isinstance(v, np.ndarray) else v) for k, v in cfg.items()}
    t["g_sparse"] = _t(chk.g_sparse)
    yield chk, t
    del t
    torch.cuda.empty_cache()


@pytest.mark.parametrize("mode", ["native", "split", "bf16"])
def test_conv4_batch8_against_the_oracle_on_samples(ops, conv4, mode):
    chk, t = conv4
    assert len(chk.pix) >= 4096
    y, gi, gw, gb = _gpu_conv(ops, t, t["g_sparse"], mode)
    assert chk.check_forward(y) <= FWD[mode]
    e_gi, e_gw, e_gb = chk.check_backward_sparse(gi, gw, gb)
    assert e_gi <= BWD[mode] and e_gw <= BWD[mode] and e_gb <= 1e-4, (e_gi, e_gw, e_gb)
    del y, gi, gw, gb
    _, gi, gw, _ = _gpu_conv(ops, t, t["grad_output"], mode)
    assert chk.check_backward_dense(gi) <= BWD[mode]
    assert len(chk.w_out) == 4 and len(chk.w_in) == 4
    assert chk.check_weight_dense(gw) <= BWD[mode]


@pytest.mark.parametrize("mode", ["native", "split", "bf16"])
def test_conv4_batch8_dense_against_float64_kernels(ops, conv4, mode):
    """Every element of the four results for the dense grad_output, against the unfused
    float64 path on the same inputs."""
    _, t = conv4
    K, it = t["kernel_size"], t["interp"]
    d = {k: t[k].double() for k in ("x", "sample_map", "interp_weights", "weight", "bias",
                                    "grad_output")}
    y64 = ops.mapped_conv_forward(d["x"], d["sample_map"], d["interp_weights"], d["weight"],
                                  d["bias"], K, it)
    y, gi, gw, gb = _gpu_conv(ops, t, t["grad_output"], mode)

    def err(a, b):
        return float((a.double() - b).abs().max() / b.abs().max())
    assert err(y, y64) <= FWD[mode]
    del y, y64
    gi64, gw64, gb64 = ops.mapped_conv_backward(d["grad_output"], d["sample_map"],
                                                d["interp_weights"], d["x"], d["weight"],
                                                d["bias"], K, it)
    assert err(gi, gi64) <= BWD[mode]
    assert err(gw, gw64) <= BWD[mode]
    assert err(gb, gb64) <= 1e-4


def test_conv4_batch8_identities_with_a_structured_cotangent(ops, conv4):
    """<y, y> = <x, backward_input(y)> = <W, backward_weight(y)> for the bias-free layer: with
    the output as its own cotangent the inner product is |y|^2, so 1e-4 of it is a real bound
    on the gradients' relative error in that direction."""
    _, t = conv4
    K, it = t["kernel_size"], t["interp"]
    zero_b = torch.zeros_like(t["bias"])
    y = ops.mapped_conv_forward(t["x"], t["sample_map"], t["interp_weights"], t["weight"], zero_b,
                                K, it)
    gi, gw, _ = ops.mapped_conv_backward(y, t["sample_map"], t["interp_weights"], t["x"],
                                         t["weight"], zero_b, K, it)
    yy = float((y.double() ** 2).sum())
    assert abs(float((t["x"].double() * gi.double()).sum()) - yy) <= 1e-4 * yy
    assert abs(float((t["weight"].double() * gw.double()).sum()) - yy) <= 1e-4 * yy


# --------------------------------------------------------------------------- configuration 5
@pytest.fixture(scope="module", params=["hierarchical", "append"])
def conv5(oracle, request):
    cfg = workloads.config5(batch=4, order=request.param)
    # one-row vertex image: no polar rows; the 12 five-neighbour vertices, the vertices of
    # the coarsest levels and the last ones appended, plus random ones
    cols = tuple(range(0, 64)) + tuple(range(-64, 0))
    chk = sp.ConvOracle(oracle, cfg, n_random=8192, n_targets=4096, seed=50, rows=(), cols=cols,
                        n_weight_channels=4)
    t = {k: (_t(v) if isinstance(v, np.ndarray) else v) for k, v in cfg.items()}
    t["g_sparse"] = _t(chk.g_sparse)
    yield chk, cfg, t
    del t
    torch.cuda.empty_cache()


@pytest.mark.parametrize("mode", ["native", "split"])
def test_icosphere5_batch4_against_the_oracle_on_samples(ops, conv5, mode):
    chk, _, t = conv5
    y, gi, gw, gb = _gpu_conv(ops, t, t["g_sparse"], mode)
    assert bool(torch.isfinite(y).all())
    assert chk.check_forward(y) <= FWD[mode]
    e_gi, e_gw, e_gb = chk.check_backward_sparse(gi, gw, gb)
    assert e_gi <= BWD[mode] and e_gw <= BWD[mode] and e_gb <= 1e-4, (e_gi, e_gw, e_gb)
    _, gi, gw, _ = _gpu_conv(ops, t, t["grad_output"], mode)
    assert chk.check_backward_dense(gi) <= BWD[mode]
    assert chk.check_weight_dense(gw) <= BWD[mode]


@pytest.mark.parametrize("mode", ["native", "split"])
def test_transposed5_batch4_against_the_oracle_in_full(ops, oracle, conv5, mode):
    _, c, t = conv5
    K, it = c["kernel_size"], c["interp"]
    OH, OW = c["out_hw"]
    want = oracle.mapped_transposed_conv_forward(c["x_coarse"], c["up_map"], c["up_weight"],
                                                 c["up_bias"], OH, OW, K, it)
    wi, ww, wb = oracle.mapped_transposed_conv_backward(c["grad_output"], c["up_map"],
                                                        c["x_coarse"], c["up_weight"],
                                                        c["up_bias"], K, it)
    ops.set_conv_compute(mode)
    try:
        yt = ops.mapped_transposed_conv_forward(t["x_coarse"], t["up_map"], None, t["up_weight"],
                                                t["up_bias"], OH, OW, K, it)
        gi, gw, gb = ops.mapped_transposed_conv_backward(t["grad_output"], t["up_map"], None,
                                                         t["x_coarse"], t["up_weight"],
                                                         t["up_bias"], K, it)
    finally:
        ops.set_conv_compute("native")
    assert sp.relerr(_n(yt), want) <= 1e-4      # the transposed layer's forward is the scatter
    assert sp.relerr(_n(gi), wi) <= 1e-4
    assert sp.relerr(_n(gw), ww) <= 1e-4
    assert sp.relerr(_n(gb), wb) <= 1e-4


# --------------------------------------------------------------------------- configuration 3
def test_pool3_batch8_against_the_oracle_in_full(ops, oracle):
    c = workloads.config3(batch=8)
    x, m, g = c["x"], c["sample_map"], c["grad_output"]
    K, it = c["kernel_size"], c["interp"]
    H, W = x.shape[2:]
    wval, widx = oracle.mapped_max_pool(x, m, K, it)
    val, idx = ops.mapped_max_pool(_t(x), _t(m), None, K, it)
    assert np.array_equal(_n(idx), widx)            # bit-exact indices
    assert np.array_equal(_n(val), wval)            # bit-exact values
    want = oracle.mapped_max_unpool(g, widx, m, H, W, K, it)
    for with_ws in (True, False):
        ops.set_unpool_workspace(with_ws)
        try:
            got = _n(ops.mapped_max_unpool(_t(g), idx, _t(m), None, H, W, K, it))
        finally:
            ops.set_unpool_workspace(True)
        assert sp.relerr(got, want) <= 1e-4
    # average pooling on the same input (no index tensor)
    assert sp.relerr(_n(ops.mapped_avg_pool(_t(x), _t(m), None, K, it)),
                     oracle.mapped_avg_pool(x, m, K, it)) <= 1e-5
    assert sp.relerr(_n(ops.mapped_avg_unpool(_t(g), _t(m), None, H, W, K, it)),
                     oracle.mapped_avg_unpool(g, m, H, W, K, it)) <= 1e-4


# --------------------------------------------------------------------------- configuration 2
def test_resample2_batch4_against_the_oracle_in_full(ops, oracle):
    c = workloads.config2(batch=4)
    x, m, it = c["x"], c["sample_map"], c["interp"]
    H, W = c["out_shape"]
    want = oracle.resample_from_map(x, m, it)
    got = _n(ops.resample_from_map(_t(x), _t(m), None, it))
    assert sp.relerr(got, want) <= 1e-5
    assert np.array_equal(_n(ops.resample_from_map(_t(x), _t(m), None, 0)),
                          oracle.resample_from_map(x, m, 0))      # nearest: bit-exact
    want_back = oracle.resample_to_map(want, m, H, W, it)
    assert sp.relerr(_n(ops.resample_to_map(_t(want), _t(m), None, H, W, it)), want_back) <= 1e-4
    norm, wsum = ops.resample_to_map_normalized(_t(want), _t(m), None, H, W, it, 1e-12)
    want_sum = oracle.resample_to_map(np.ones((1, 1) + want.shape[2:], np.float32), m, H, W,
                                      it)[0, 0]
    assert sp.relerr(_n(wsum), want_sum) <= 1e-4
    # The quotient keeps the scatter tolerance: bilinear weights are non-negative, so the
    # numerator's rounding error is at most n * eps * max|value| * weight_sum for n sources
    # and dividing by the weight sum (itself good to n * eps) leaves n * eps * max|value|,
    # however small the weight sum of a pixel is.
    assert sp.relerr(_n(norm), want_back / (want_sum + np.float32(1e-12))) <= 1e-4
    # the UV way back and its adjoint
    quad, uv, tp = c["quad_idx"], c["tex_uv"], c["patch"]
    tex = want.reshape(want.shape[0], want.shape[1], m.shape[0], tp, tp)
    assert sp.relerr(_n(ops.resample_from_uv_maps(_t(tex), _t(quad), _t(uv), it)),
                     oracle.resample_from_uv_maps(tex, quad, uv, it)) <= 1e-5
    assert sp.relerr(_n(ops.resample_to_uv_maps(_t(x), _t(quad), _t(uv), m.shape[0], tp, tp, it)),
                     oracle.resample_to_uv_maps(x, quad, uv, m.shape[0], tp, tp, it)) <= 1e-4
