import json
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "spherical-package_amd")
for p in (ROOT, PKG):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    """GPU tests are skipped, not failed, when collected without a GPU."""
    try:
        import torch
        have_gpu = torch.cuda.is_available()
    except Exception:
        have_gpu = False
    if have_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def known_answers():
    """The reference test-suite's known-answer vectors (tests/golden/*.json)."""
    with open(os.path.join(GOLDEN_DIR, "reference_known_answers.json")) as f:
        return json.load(f)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as _oracle
    _oracle.build()
    return _oracle


# ---------------------------------------------------------------------------------------------
# Builders shared by the oracle (CPU) and GPU replays of the reference's known-answer tests.
# ---------------------------------------------------------------------------------------------
def ka_kernel_map(ka, name, dtype=np.float64):
    """[OH,OW,K,2] map by name, resolving the +/-0.5 shifted variants."""
    dx = dy = 0.0
    if name in ka["derived_maps"] and name != "_comment":
        d = ka["derived_maps"][name]
        name, dx, dy = d["base"], d["dx"], d["dy"]
    m = ka["maps"][name]
    return np.ascontiguousarray(
        np.stack([np.array(m["x"], dtype) + dx, np.array(m["y"], dtype) + dy], -1))


def ka_resample_map(ka, name, dtype=np.float64):
    return np.ascontiguousarray(np.array(ka["resample_maps"][name]["xy"], dtype))


def ka_input(name, batch, channels, dtype=np.float64):
    """'arangeHxW' / 'onesHxW' planes tiled over batch and channels."""
    kind = "arange" if name.startswith("arange") else "ones"
    h, w = (int(v) for v in name[len(kind):].split("x"))
    plane = np.arange(h * w, dtype=dtype).reshape(h, w) if kind == "arange" \
        else np.ones((h, w), dtype)
    return np.ascontiguousarray(np.broadcast_to(plane, (batch, channels, h, w)))


def ka_weight(kind, out_channels, in_channels, K, dtype=np.float64):
    w = np.ones((out_channels, in_channels, K), dtype)
    if kind == "quarter_first_half":
        w[..., :K // 2] *= 0.25
    return w


def relerr(a, b):
    """Norm-relative error max|a-b| / max|b| (the tolerance definition used throughout)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))
