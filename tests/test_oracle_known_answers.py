"""The CPU oracle replays every known-answer vector the reference's own tests hold
for this path (tests/golden/reference_known_answers.json), in float64 and float32."""
import numpy as np
import pytest

from conftest import ka_input, ka_kernel_map, ka_resample_map, ka_weight

BILINEAR = 1


def _sizes(ka):
    s = ka["sizes"]
    return s["bs"], s["in_channels"], s["out_channels"], s["kernel_size"], s["bias"]


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("case", range(6))
def test_mapped_convolution(oracle, known_answers, case, dtype):
    c = known_answers["mapped_convolution"][case]
    bs, cin, cout, K, bias = _sizes(known_answers)
    x = ka_input(c["input"], bs, cin, dtype)
    m = ka_kernel_map(known_answers, c["map"], dtype)
    w = ka_weight(c["weight"], cout, cin, K, dtype)
    b = np.full(cout, bias, dtype)
    out = oracle.mapped_conv_forward(x, m, w, b, K, BILINEAR)
    want = bias + cin * np.array(c["expected_core"], np.float64)
    assert out.shape == (bs, cout) + want.shape
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("case", range(3))
def test_mapped_transposed_convolution(oracle, known_answers, case, dtype):
    c = known_answers["mapped_transposed_convolution"][case]
    bs, cin, cout, K, bias = _sizes(known_answers)
    x = ka_input(c["input"], bs, cin, dtype)
    m = ka_kernel_map(known_answers, c["map"], dtype)
    w = np.ones((cin, cout, K), dtype)
    b = np.full(cout, bias, dtype)
    out = oracle.mapped_transposed_conv_forward(x, m, w, b, c["oh"], c["ow"], K, BILINEAR)
    want = bias + cin * np.array(c["expected_core"], np.float64)
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("case", range(4))
def test_mapped_max_pool_values(oracle, known_answers, case, dtype):
    c = known_answers["mapped_max_pool"][case]
    bs, _, _, K, _ = _sizes(known_answers)
    x = ka_input(c["input"], bs, 1, dtype)
    m = ka_kernel_map(known_answers, c["map"], dtype)
    for quirk in (False, True):
        out, idx = oracle.mapped_max_pool(x, m, K, BILINEAR, host_init_quirk=quirk)
        want = np.array(c["expected"], np.float64)
        np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-6)
        # the stored index names a sample of this pixel's own kernel
        pix = np.arange(want.size).reshape(want.shape)
        assert ((idx >= pix * K * 2) & (idx < (pix + 1) * K * 2) & (idx % 2 == 0)).all()


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_mapped_avg_pool_values(oracle, known_answers, dtype):
    c = known_answers["mapped_avg_pool"][0]
    bs, _, _, K, _ = _sizes(known_answers)
    x = ka_input(c["input"], bs, 1, dtype)
    m = ka_kernel_map(known_answers, c["map"], dtype)
    out = oracle.mapped_avg_pool(x, m, K, BILINEAR)
    want = np.array(c["expected"], np.float64)
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-6)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
@pytest.mark.parametrize("case", range(10))
def test_unresample(oracle, known_answers, case, dtype):
    c = known_answers["unresample"][case]
    bs = known_answers["sizes"]["bs"]
    x = ka_input(c["input"], bs, 3, dtype)
    m = ka_resample_map(known_answers, c["map"], dtype)
    w = None
    if "weights" in c:
        w = np.array(known_answers["resample_maps"][c["weights"]]["w"], dtype)
    out = oracle.resample_from_map(x, m, c["interp"], w)
    want = np.array(c["expected"], np.float64)
    np.testing.assert_allclose(out, np.broadcast_to(want, out.shape), rtol=1e-6, atol=1e-6)
