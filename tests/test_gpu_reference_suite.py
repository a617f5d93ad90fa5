"""Replays the reference's own hot-path tests on the GPU through the nn layers: float64
known answers plus torch.autograd.gradcheck, as tests/utils.py:63-192 of the reference do
(its 'cuda' variants are these same tests with .cuda() tensors)."""
import numpy as np
import pytest
import torch
from torch.autograd import gradcheck

from conftest import ka_input, ka_kernel_map, ka_resample_map, ka_weight

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def _sizes(ka):
    s = ka["sizes"]
    return s["bs"], s["in_channels"], s["out_channels"], s["kernel_size"], s["bias"]


def _run(layer, args, grad_index=0):
    """Forward, backward with an all-ones upstream gradient, then gradcheck."""
    out = layer(*args)
    first = out[0] if isinstance(out, tuple) else out
    first.backward(torch.ones_like(first))
    assert args[grad_index].grad is not None
    assert gradcheck(layer, args)
    return first.detach().cpu().numpy()


@pytest.mark.parametrize("case", range(6))
def test_mapped_convolution(known_answers, case):
    from spherical_distortion.nn import MappedConvolution
    c = known_answers["mapped_convolution"][case]
    bs, cin, cout, K, bias = _sizes(known_answers)
    layer = MappedConvolution(cin, cout, kernel_size=K).double().to(DEV)
    layer.weight.data = _t(ka_weight(c["weight"], cout, cin, K))
    layer.bias.data = _t(np.full(cout, bias))
    x = _t(ka_input(c["input"], bs, cin)).requires_grad_()
    out = _run(layer, (x, _t(ka_kernel_map(known_answers, c["map"])), None))
    want = bias + cin * np.array(c["expected_core"])
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-7)


@pytest.mark.parametrize("case", range(3))
def test_mapped_transposed_convolution(known_answers, case):
    from spherical_distortion.nn import MappedTransposedConvolution
    c = known_answers["mapped_transposed_convolution"][case]
    bs, cin, cout, K, bias = _sizes(known_answers)
    layer = MappedTransposedConvolution(cin, cout, kernel_size=K).double().to(DEV)
    layer.weight.data = _t(np.ones((cin, cout, K)))
    layer.bias.data = _t(np.full(cout, bias))
    x = _t(ka_input(c["input"], bs, cin)).requires_grad_()
    out = _run(layer, (x, c["oh"], c["ow"], _t(ka_kernel_map(known_answers, c["map"])), None))
    want = bias + cin * np.array(c["expected_core"])
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-7)


@pytest.mark.parametrize("case", range(4))
def test_mapped_max_pool(known_answers, case):
    from spherical_distortion.nn import MappedMaxPool
    c = known_answers["mapped_max_pool"][case]
    bs, _, _, K, _ = _sizes(known_answers)
    layer = MappedMaxPool(kernel_size=K).double()
    x = _t(ka_input(c["input"], bs, 1)).requires_grad_()
    out = _run(layer, (x, _t(ka_kernel_map(known_answers, c["map"])), None))
    np.testing.assert_allclose(out, np.broadcast_to(np.array(c["expected"]), out.shape), rtol=1e-7)


def test_mapped_avg_pool(known_answers):
    """tests/test_mapped_pooling.py:110-132 of the reference, and the unpool module on the same
    map (forward of the adjoint, gradcheck)."""
    from spherical_distortion.nn import MappedAvgPool, MappedAvgUnpool
    c = known_answers["mapped_avg_pool"][0]
    bs, _, _, K, _ = _sizes(known_answers)
    x = _t(ka_input(c["input"], bs, 1)).requires_grad_(True)
    m = _t(ka_kernel_map(known_answers, c["map"]))
    out = _run(MappedAvgPool(kernel_size=K).double().to(DEV), (x, m))
    want = np.array(c["expected"], np.float64)
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-12)
    y = torch.rand(bs, 1, *m.shape[:2], dtype=torch.float64, device=DEV, requires_grad=True)
    layer = MappedAvgUnpool(kernel_size=K).double().to(DEV)
    h, w = x.shape[2:]
    spread = layer(y, h, w, m)
    assert spread.shape == (bs, 1, h, w)
    assert gradcheck(lambda t: layer(t, h, w, m), (y,))
    # adjoint of the pooling: <pool(x), y> = <x, unpool(y)>
    pooled = MappedAvgPool(kernel_size=K).double().to(DEV)(x.detach(), m)
    assert abs(float((pooled * y.detach()).sum()) - float((x.detach() * spread.detach()).sum())) < 1e-9


@pytest.mark.parametrize("case", range(10))
def test_unresample(known_answers, case):
    from spherical_distortion.nn import InterpolationType, Unresample
    c = known_answers["unresample"][case]
    bs = known_answers["sizes"]["bs"]
    layer = Unresample(InterpolationType(c["interp"]))
    x = _t(ka_input(c["input"], bs, 3)).requires_grad_()
    w = None
    if "weights" in c:
        w = _t(np.array(known_answers["resample_maps"][c["weights"]]["w"]))
    out = _run(layer, (x, _t(ka_resample_map(known_answers, c["map"])), w))
    np.testing.assert_allclose(out, np.broadcast_to(np.array(c["expected"]), out.shape),
                               rtol=1e-7, atol=1e-7)


def test_resample_forward_and_gradcheck(known_answers):
    """The scatter direction as a layer (the reference only exercises it as a backward)."""
    from spherical_distortion.nn import InterpolationType, Resample
    x = _t(ka_input("arange3x2", 2, 2)).requires_grad_()
    m = _t(ka_resample_map(known_answers, "sample_map7"))
    for interp in (0, 1, 2):
        layer = Resample(InterpolationType(interp))
        assert gradcheck(lambda t: layer(t, m, (3, 4)), (x,))


def test_three_dimensional_input_gets_a_batch_dimension(known_answers):
    from spherical_distortion import functional as F
    x = _t(ka_input("arange3x4", 1, 3))[0]
    m = _t(ka_resample_map(known_answers, "sample_map6"))
    out = F.unresample(x, m, 1)
    assert out.shape == (3, 3, 2) and x.dim() == 3
    back = F.resample(out, m, (3, 4), 1)
    assert back.shape == (3, 3, 4)
