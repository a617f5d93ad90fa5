"""CPU check of the slicing identities tests/sampled_parity.py relies on: what the oracle
returns on a sliced map / on channel subsets equals the slice of its full evaluation."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import sampled_parity as sp  # noqa: E402
import workloads  # noqa: E402


def _small_cfg():
    rng = np.random.default_rng(9)
    H, W, B, Cin, Cout, K = 16, 32, 2, 6, 7, 9
    m = workloads.gnomonic_kernel_map(H, W, dtype=np.float64)
    m4, w4 = workloads.four_nearest_weighted(m, H, W)
    return {"x": rng.standard_normal((B, Cin, H, W)).astype(np.float32),
            "sample_map": m4.astype(np.float32), "interp_weights": w4.astype(np.float32),
            "weight": rng.standard_normal((Cout, Cin, K)).astype(np.float32),
            "bias": rng.standard_normal(Cout).astype(np.float32),
            "grad_output": rng.standard_normal((B, Cout, H, W)).astype(np.float32),
            "kernel_size": K, "interp": 2}


def test_sliced_oracle_answers_equal_slices_of_the_full_evaluation(oracle):
    c = _small_cfg()
    chk = sp.ConvOracle(oracle, c, n_random=40, n_targets=30, seed=3, n_weight_channels=3)
    K, it = c["kernel_size"], c["interp"]
    y = oracle.mapped_conv_forward(c["x"], c["sample_map"], c["weight"], c["bias"], K, it,
                                   c["interp_weights"])
    assert chk.check_forward(y) <= 1e-6
    gi, gw, gb = oracle.mapped_conv_backward(c["grad_output"], c["sample_map"], c["x"],
                                             c["weight"], c["bias"], K, it, c["interp_weights"])
    assert chk.check_backward_dense(gi) <= 1e-6
    assert len(chk.w_out) == 3 and len(chk.w_in) == 3
    assert chk.w_out[0] == 0 and chk.w_out[-1] == 6 and chk.w_in[-1] == 5
    assert chk.check_weight_dense(gw) <= 1e-6
    # a wrong channel pairing must show
    assert sp.relerr(gw[chk.w_out][:, chk.w_in[::-1]], chk.grad_weight_dense) > 1e-2
    gi_s, gw_s, gb_s = oracle.mapped_conv_backward(chk.g_sparse, c["sample_map"], c["x"],
                                                   c["weight"], c["bias"], K, it,
                                                   c["interp_weights"])
    assert max(sp.relerr(gi_s, chk.grad_input), sp.relerr(gw_s, chk.grad_weight),
               sp.relerr(gb_s, chk.grad_bias)) <= 1e-6
