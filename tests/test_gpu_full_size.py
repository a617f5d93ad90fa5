"""Properties at the full sizes of the benchmark configurations, where the CPU oracle would
take minutes: identities the operators must satisfy whatever the data (adjointness of
gather and scatter, linearity, the defining property of the pooling indices, conservation),
checked on the GPU in float64 reductions.  Batches are cut to 1-2 elements where that only
repeats the same work; spatial sizes, channel counts and maps are the configurations' own.

Every adjoint identity is evaluated with a structured cotangent, the operator's own output
(<y, y> = <x, adjoint(y)>), so both sides equal |y|^2 and the tolerance, 1e-4 of that value
(5e-3 with bf16 operands), bounds the relative error of the adjoint in that direction.  The
element-wise comparisons with the oracle at these sizes are in test_gpu_bench_size.py.
"""
import os
import sys

import numpy as np
import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import workloads  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from _spherical_distortion_ext import _ops
    return _ops


def _t(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _dot(a, b):
    return float((a.double() * b.double()).sum())


def _close(lhs, rhs, tol):
    """Both sides of an identity whose common value is a sum of squares."""
    assert lhs > 0 and abs(lhs - rhs) <= tol * lhs, (lhs, rhs)


# --------------------------------------------------------------------------- configuration 4
@pytest.fixture(scope="module")
def cfg4():
    c = workloads.config4(batch=2)
    return {k: (_t(v) if isinstance(v, np.ndarray) else v) for k, v in c.items()}


def test_conv4_adjoint_and_weight_gradient_identities(ops, cfg4):
    """<y, y> = <x, backward_input(y)> = <W, backward_weight(y)> for y = conv(x) - bias, and
    grad_bias = sum of y, on the 256x512, 128 -> 128 channel, K = 9 weighted bispherical map."""
    c = cfg4
    K, it = c["kernel_size"], c["interp"]
    zero_b = torch.zeros_like(c["bias"])
    y = ops.mapped_conv_forward(c["x"], c["sample_map"], c["interp_weights"], c["weight"], zero_b,
                                K, it)
    gi, gw, gb = ops.mapped_conv_backward(y, c["sample_map"], c["interp_weights"],
                                          c["x"], c["weight"], c["bias"], K, it)
    lhs = _dot(y, y)
    _close(lhs, _dot(c["x"], gi), 1e-4)
    _close(lhs, _dot(c["weight"], gw), 1e-4)
    want_gb = y.double().sum(dim=(0, 2, 3))
    assert float((gb.double() - want_gb).abs().max()) <= 1e-4 * float(want_gb.abs().max() + 1)


def test_conv4_linearity_and_bias(ops, cfg4):
    c = cfg4
    K, it = c["kernel_size"], c["interp"]
    x1 = c["x"]
    x2 = torch.roll(c["x"], shifts=(1, 7, 13), dims=(1, 2, 3)).contiguous()
    f = lambda x, b: ops.mapped_conv_forward(x, c["sample_map"], c["interp_weights"], c["weight"],
                                             b, K, it)
    zero_b = torch.zeros_like(c["bias"])
    y12 = f(0.5 * x1 - 2.0 * x2, zero_b)
    y1, y2 = f(x1, zero_b), f(x2, zero_b)
    err = float((y12 - (0.5 * y1 - 2.0 * y2)).abs().max())
    assert err <= 1e-4 * float(y12.abs().max())
    yb = f(x1, c["bias"])
    err = float((yb - y1 - c["bias"].view(1, -1, 1, 1)).abs().max())
    assert err <= 1e-5 * float(yb.abs().max())


def test_conv4_bf16_identities(ops, cfg4):
    """The same adjoint identities with bf16 operands: each side rounds its operands
    separately, so they agree to bf16 accuracy."""
    c = cfg4
    K, it = c["kernel_size"], c["interp"]
    ops.set_conv_compute("bf16")
    try:
        zero_b = torch.zeros_like(c["bias"])
        y = ops.mapped_conv_forward(c["x"], c["sample_map"], c["interp_weights"], c["weight"],
                                    zero_b, K, it)
        gi, gw, _ = ops.mapped_conv_backward(y, c["sample_map"], c["interp_weights"], c["x"],
                                             c["weight"], c["bias"], K, it)
    finally:
        ops.set_conv_compute("native")
    lhs = _dot(y, y)
    _close(lhs, _dot(c["x"], gi), 5e-3)
    _close(lhs, _dot(c["weight"], gw), 5e-3)


# --------------------------------------------------------------------------- configuration 2
def test_resample2_gather_scatter_adjoint_and_weight_sum(ops):
    c = workloads.config2(batch=4)
    x, m = _t(c["x"]), _t(c["sample_map"])
    H, W = c["out_shape"]
    it = c["interp"]
    patches = ops.resample_from_map(x, m, None, it)
    back = ops.resample_to_map(patches, m, None, H, W, it)
    _close(_dot(patches, patches), _dot(x, back), 1e-4)
    # normalised scatter of a gathered constant image gives the constant back wherever weight fell
    ones = torch.ones_like(x)
    p1 = ops.resample_from_map(ones, m, None, it)
    out, wsum = ops.resample_to_map_normalized(p1, m, None, H, W, it, 1e-12)
    hit = wsum > 1e-3
    # p1 < 1 only where a patch sample's taps leave the image
    assert float(p1.max()) <= 1.0 + 1e-6
    inside = (p1 > 1 - 1e-6).float().mean()
    assert float(inside) > 0.9
    assert float(out[:, :, hit].max()) <= 1.0 + 1e-4
    assert float(wsum.sum()) == pytest.approx(float(p1[0, 0].double().sum()), rel=1e-4)


# --------------------------------------------------------------------------- configuration 3
def test_pool3_indices_select_the_maximum_and_unpool_conserves(ops):
    c = workloads.config3(batch=2)
    x, m = _t(c["x"]), _t(c["sample_map"])
    K, it = c["kernel_size"], c["interp"]
    B, C, H, W = x.shape
    OH, OW = m.shape[:2]
    vals, idx = ops.mapped_max_pool(x, m, None, K, it)
    # all K samples of every pixel through the gather entry point: [B, C, OH, OW*K]
    samples = ops.resample_from_map(x, m.reshape(OH, OW * K, 2).contiguous(), None, it)
    samples = samples.view(B, C, OH, OW, K)
    assert torch.equal(vals, samples.max(dim=-1).values)          # bit-exact values
    # the index names the first sample that attains the maximum
    pix = torch.arange(OH * OW, device=DEV).view(1, 1, OH, OW)
    k_win = (idx // 2) - pix * K
    assert int(k_win.min()) >= 0 and int(k_win.max()) < K
    first = (samples == vals.unsqueeze(-1)).float().argmax(dim=-1)
    assert torch.equal(k_win, first)
    # unpool routes every gradient to one input pixel: totals per plane are conserved, except
    # where the winning sample lies outside the image (it reads as 0 and has no target), and
    # it is the adjoint of "take the winning sample"
    g = _t(c["grad_output"][:2])
    gin = ops.mapped_max_unpool(g, idx, m, None, H, W, K, it)
    xy = m.reshape(-1, 2)[(idx // 2).reshape(-1)].view(B, C, OH, OW, 2)
    rnd = torch.where(xy >= 0, torch.floor(xy + 0.5), torch.ceil(xy - 0.5))
    inside = (rnd[..., 0] >= 0) & (rnd[..., 0] <= W - 1) & (rnd[..., 1] >= 0) & (rnd[..., 1] <= H - 1)
    tot_in = gin.double().sum(dim=(2, 3))
    tot_out = (g.double() * inside).sum(dim=(2, 3))
    assert float((tot_in - tot_out).abs().max()) <= 1e-4 * float(g.double().abs().sum(dim=(2, 3)).max())
    _close(_dot(vals, vals), _dot(ops.mapped_max_unpool(vals, idx, m, None, H, W, K, it), x), 1e-4)


# --------------------------------------------------------------------------- configuration 5
def test_icosphere5_adjoints(ops):
    c = workloads.config5(batch=2)
    K, it = c["kernel_size"], c["interp"]
    x, m, w, b, g = (_t(c[k]) for k in ("x", "sample_map", "weight", "bias", "grad_output"))
    zero_b = torch.zeros_like(b)
    y = ops.mapped_conv_forward(x, m, None, w, zero_b, K, it)
    gi, gw, _ = ops.mapped_conv_backward(y, m, None, x, w, b, K, it)
    lhs = _dot(y, y)
    _close(lhs, _dot(x, gi), 1e-4)
    _close(lhs, _dot(w, gw), 1e-4)
    # transposed up-sampling: forward is a scatter, its backward-input a gather
    xc, um, uw, ub = (_t(c[k]) for k in ("x_coarse", "up_map", "up_weight", "up_bias"))
    OH, OW = c["out_hw"]
    yt = ops.mapped_transposed_conv_forward(xc, um, None, uw, torch.zeros_like(ub), OH, OW, K, it)
    gi, gw, gb = ops.mapped_transposed_conv_backward(yt, um, None, xc, uw, ub, K, it)
    lhs = _dot(yt, yt)
    _close(lhs, _dot(xc, gi), 1e-4)
    _close(lhs, _dot(uw, gw), 1e-4)
