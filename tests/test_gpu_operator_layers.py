"""The two implementations of the torch operators over the C ABI: the compiled layer
(libsdk_torch_ops.so, csrc/torch_ops.cpp) and the Python functions of _ops.py that serve when
it is absent.  Same checks, same plan cache rules, same results: every operator the compiled
layer names is run both ways on the same inputs (bit for bit where the kernels are
deterministic, to rounding where sums depend on scheduling), with the cache on and off, and the
argument errors of both are compared.
"""
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


def _same(a, b, exact):
    a = a if isinstance(a, (tuple, list)) else (a,)
    b = b if isinstance(b, (tuple, list)) else (b,)
    assert len(a) == len(b)
    for x, y in zip(a, b):
        assert x.shape == y.shape and x.dtype == y.dtype and x.device == y.device
        if exact:
            assert torch.equal(x, y)
        else:
            assert relerr(x.cpu().numpy(), y.cpu().numpy()) <= 1e-5


def _inputs(weighted, dtype):
    rng = np.random.default_rng(11 + weighted)
    B, Cin, Cout, H, W, OH, OW, K, P = 2, 6, 5, 24, 40, 12, 20, 9, 2
    ys, xs = np.meshgrid(np.arange(OH), np.arange(OW), indexing="ij")
    ang = 2 * np.pi * np.arange(K) / K
    cx, cy = xs[..., None] * 2 + 2 * np.cos(ang), ys[..., None] * 2 + 2 * np.sin(ang)
    if weighted:
        cx = cx[..., None] + rng.uniform(-1, 1, (OH, OW, K, P))
        cy = cy[..., None] + rng.uniform(-1, 1, (OH, OW, K, P))
    m = (np.stack([cx, cy], -1) + rng.uniform(-0.3, 0.3, cx.shape + (2,))).astype(dtype)
    iw = rng.uniform(0.1, 1, m.shape[:-1]).astype(dtype) if weighted else None
    return dict(
        m=_t(m), iw=_t(iw), K=K, H=H, W=W,
        x=_t(rng.standard_normal((B, Cin, H, W)).astype(dtype)),
        g=_t(rng.standard_normal((B, Cout, OH, OW)).astype(dtype)),
        gp=_t(rng.standard_normal((B, Cin, OH, OW)).astype(dtype)),
        w=_t(rng.standard_normal((Cout, Cin, K)).astype(dtype)),
        b=_t(rng.standard_normal(Cout).astype(dtype)), bt=_t(rng.standard_normal(Cin).astype(dtype)),
        rm=_t(m[:, :, 0]), riw=_t(None if iw is None else iw[:, :, 0]),
        rx=_t(rng.standard_normal((B, Cin, OH, OW)).astype(dtype)))


@pytest.mark.parametrize("cache", [True, False])
@pytest.mark.parametrize("weighted,dtype,interp", [(False, np.float32, 1), (True, np.float32, 2),
                                                   (False, np.float64, 0), (False, np.float32, 0)])
def test_compiled_and_python_operators_agree(ops, weighted, dtype, interp, cache):
    if ops._native is None:
        pytest.skip("the compiled operator layer is not built")
    assert len(ops._NATIVE_OPS) == 11
    d = _inputs(weighted, dtype)
    calls = {
        "resample_from_map": ((d["x"], d["rm"], d["riw"], interp), True),
        "resample_to_map": ((d["rx"], d["rm"], d["riw"], d["H"], d["W"], interp), False),
        "resample_to_map_normalized": ((d["rx"], d["rm"], d["riw"], d["H"], d["W"], interp, 1e-9),
                                       False),
        "mapped_max_pool": ((d["x"], d["m"], d["iw"], d["K"], interp), True),
        "mapped_avg_pool": ((d["x"], d["m"], d["iw"], d["K"], interp), True),
        "mapped_avg_unpool": ((d["gp"], d["m"], d["iw"], d["H"], d["W"], d["K"], interp), False),
        "mapped_conv_forward": ((d["x"], d["m"], d["iw"], d["w"], d["b"], d["K"], interp), True),
        "mapped_conv_backward": ((d["g"], d["m"], d["iw"], d["x"], d["w"], d["b"], d["K"], interp),
                                 False),
        # transposed layer over the same map: Cout -> Cin channels, weight [Cout, Cin, K]
        "mapped_transposed_conv_forward": ((d["g"], d["m"], d["iw"], d["w"], d["bt"], d["H"],
                                            d["W"], d["K"], interp), False),
        "mapped_transposed_conv_backward": ((d["x"], d["m"], d["iw"], d["g"], d["w"], d["bt"],
                                             d["K"], interp), False),
    }
    ops.set_conv_plan_cache(cache)
    try:
        for name, (args, exact) in calls.items():
            native = getattr(ops.ops, name)(*args)
            assert getattr(ops, name) is getattr(ops.ops, name)   # the module-level name
            python = ops.PYTHON_IMPL[name](*args)
            _same(native, python, exact)
        _, idx = ops.ops.mapped_max_pool(d["x"], d["m"], d["iw"], d["K"], interp)
        args = (d["gp"], idx, d["m"], d["iw"], d["H"], d["W"], d["K"], interp)
        for with_ws in (True, False):
            ops.set_unpool_workspace(with_ws)
            _same(ops.ops.mapped_max_unpool(*args), ops.PYTHON_IMPL["mapped_max_unpool"](*args),
                  False)
    finally:
        ops.set_unpool_workspace(True)
        ops.set_conv_plan_cache(True)


def test_compiled_layer_follows_the_compute_mode_and_the_cache_switches(ops):
    if ops._native is None:
        pytest.skip("the compiled operator layer is not built")
    d = _inputs(False, np.float32)
    args = (d["x"], d["m"], None, d["w"], d["b"], d["K"], 1)
    native = ops.ops.mapped_conv_forward(*args)
    with ops.conv_compute("bf16"):
        assert ops._native.sdk_torch_current_mode() == 1
        rounded = ops.ops.mapped_conv_forward(*args)
        assert torch.equal(rounded, ops.PYTHON_IMPL["mapped_conv_forward"](*args))
    assert ops._native.sdk_torch_current_mode() == 0
    assert not torch.equal(native, rounded)
    assert relerr(rounded.cpu().numpy(), native.cpu().numpy()) <= 1e-2
    # the cache of the compiled layer: one entry per map, dropped with the switch
    ops.set_conv_plan_cache(False)
    ops.set_conv_plan_cache(True, max_entries=2)
    try:
        assert ops.plan_cache_size() == 0
        maps = [d["m"].clone() for _ in range(3)]
        for m in maps:
            ops.ops.mapped_conv_forward(d["x"], m, None, d["w"], d["b"], d["K"], 1)
        assert ops.plan_cache_size() == 2
        maps[2].add_(0.25)                       # in place: a new version, a new plan
        y = ops.ops.mapped_conv_forward(d["x"], maps[2], None, d["w"], d["b"], d["K"], 1)
        assert not torch.equal(y, native)
        with torch.inference_mode():
            ops.ops.mapped_conv_forward(d["x"], d["m"].clone(), None, d["w"], d["b"], d["K"], 1)
        assert ops.plan_cache_size() == 2
    finally:
        ops.set_conv_plan_cache(True, max_entries=16)


def test_both_layers_refuse_the_same_arguments(ops):
    d = _inputs(False, np.float32)
    bad = [
        ("mapped_conv_forward", (d["x"].transpose(2, 3), d["m"], None, d["w"], d["b"], d["K"], 1),
         "contiguous"),
        ("mapped_conv_forward", (d["x"], d["m"].double(), None, d["w"], d["b"], d["K"], 1), "dtype"),
        ("mapped_conv_forward", (d["x"], d["m"], None, d["w"], d["b"], d["K"] + 1, 1), "kernel_size"),
        ("mapped_conv_forward", (d["x"], d["m"], None, d["w"][:, :3].contiguous(), d["b"], d["K"], 1),
         "input channels"),
        ("mapped_max_pool", (d["x"], d["m"][..., :1].contiguous(), None, d["K"], 0), "ending in 2"),
        ("mapped_max_unpool", (d["gp"], d["gp"], d["m"], None, d["H"], d["W"], d["K"], 0), "int64"),
        ("resample_to_map", (d["x"], d["rm"], None, d["H"], d["W"], 1), "grid"),
        ("resample_from_map", (d["x"].half(), d["rm"].half(), None, 1), "dtype"),
    ]
    for name, args, what in bad:
        for fn in (getattr(ops.ops, name), ops.PYTHON_IMPL[name]):
            with pytest.raises(RuntimeError, match=what):
                fn(*args)
