"""CPU-only checks of the host side: the C-ABI library exports what the header declares,
the Python layers mirror the reference's interface, and nothing runs without the GPU."""
import ctypes
import math
import os
import re

import pytest
import torch

from conftest import PKG, ROOT


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "sdk_mapped_ops.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sdk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib_path = os.path.join(PKG, "libsdk_mapped_ops.so")
    assert os.path.exists(lib_path), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    lib = ctypes.CDLL(lib_path)
    names = _declared_symbols()
    assert len(names) >= 17
    for n in names:
        assert hasattr(lib, n), "missing export " + n


def test_ctypes_table_matches_header():
    from _spherical_distortion_ext import _capi
    declared = set(_declared_symbols())
    bound = set(_capi.SIGNATURES) | set(_capi.OTHER_SYMBOLS)
    assert declared == bound
    assert _capi.load().sdk_version() >= 100


def test_enum_values_and_tensor_round_trip():
    from spherical_distortion.nn import InterpolationType as IT
    assert (int(IT.NEAREST), int(IT.BILINEAR), int(IT.BISPHERICAL)) == (0, 1, 2)
    assert IT(torch.tensor(2)) is IT.BISPHERICAL
    assert IT(torch.tensor(int(IT.NEAREST))) is IT.NEAREST


def test_module_parameters_follow_the_reference_layout():
    from spherical_distortion.nn import (MappedConvolution, MappedMaxPool,
                                         MappedTransposedConvolution)
    conv = MappedConvolution(6, 4, kernel_size=9)
    assert conv.weight.shape == (4, 6, 9) and conv.bias.shape == (4,)
    bound = 1 / math.sqrt(6 * 9)
    assert conv.weight.abs().max() <= bound and conv.bias.abs().max() <= bound
    assert conv.weight.std() > 0.3 * bound
    assert int(conv.interp) == 1
    nb = MappedConvolution(6, 4, kernel_size=9, bias=False)
    assert isinstance(nb.bias, torch.nn.Parameter) and (nb.bias == 0).all()
    t = MappedTransposedConvolution(6, 4, kernel_size=7)
    assert t.weight.shape == (6, 4, 7) and t.bias.shape == (4,)
    assert t.weight.abs().max() <= 1 / math.sqrt(6 * 7)
    assert set(dict(conv.state_dict())) == {"weight", "bias"}
    assert MappedMaxPool(4).return_indices is False


def test_check_args_assertions():
    from spherical_distortion import functional as F
    from spherical_distortion.layer_utils import check_args
    x = torch.zeros(1, 2, 4, 5)
    with pytest.raises(AssertionError, match="4 dimensions"):
        check_args(x[0], torch.zeros(4, 5, 3, 2), None, 2, 3)
    with pytest.raises(AssertionError, match="Sample map must have 4"):
        check_args(x, torch.zeros(4, 5, 2), None, 2, 3)
    with pytest.raises(AssertionError, match="Sample map must have 5"):
        check_args(x, torch.zeros(4, 5, 3, 2), torch.zeros(4, 5, 3, 2), 2, 3)
    with pytest.raises(AssertionError, match="size 2"):
        check_args(x, torch.zeros(4, 5, 3, 3), None, 2, 3)
    with pytest.raises(AssertionError, match="same dtype"):
        check_args(x, torch.zeros(4, 5, 3, 2).double(), None, 2, 3)
    with pytest.raises(AssertionError, match="input channels"):
        check_args(x, torch.zeros(4, 5, 3, 2), None, 3, 3)
    with pytest.raises(AssertionError, match="Kernel size"):
        check_args(x, torch.zeros(4, 5, 3, 2), None, 2, 4)
    with pytest.raises(AssertionError, match="interpolation points"):
        check_args(x, torch.zeros(4, 5, 3, 2, 2), torch.zeros(4, 5, 3, 3), 2, 3)
    check_args(x, torch.zeros(4, 5, 3, 2, 2), torch.zeros(4, 5, 3, 2), 2, 3)
    check_args(x, torch.zeros(7, 7, 2), None, None, None)  # resample: rank-3 map
    with pytest.raises(AssertionError, match="must match sample map"):
        F.mapped_transposed_convolution(x, torch.zeros(2, 3, 3), torch.zeros(3),
                                        torch.zeros(4, 6, 3, 2), 8, 8, 3, 1)
    with pytest.raises(AssertionError, match="3 or 4 dimensions"):
        F.unresample(torch.zeros(4, 5), torch.zeros(2, 2, 2), 1)


def test_cpu_tensors_are_refused_loudly():
    """There is no CPU path: the operators exist for the GPU dispatch key only."""
    from spherical_distortion.nn import MappedConvolution, MappedMaxPool, Unresample
    x = torch.zeros(1, 2, 4, 5)
    with pytest.raises((NotImplementedError, RuntimeError)):
        MappedConvolution(2, 3, 4)(x, torch.zeros(4, 5, 4, 2))
    with pytest.raises((NotImplementedError, RuntimeError)):
        MappedMaxPool(4)(x, torch.zeros(4, 5, 4, 2))
    with pytest.raises((NotImplementedError, RuntimeError)):
        Unresample()(x, torch.zeros(3, 3, 2))


def test_product_code_never_touches_the_oracle():
    bad = []
    for base, _, files in os.walk(PKG):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")) or f == "Makefile":
                text = open(os.path.join(base, f)).read()
                if re.search(r"\boracle\b|_ref\b|sdk_oracle", text):
                    bad.append(os.path.join(base, f))
    assert not bad, bad


def test_workload_generators_shapes():
    import numpy as np
    import workloads as wl
    m = wl.gnomonic_kernel_map(16, 32, stride=2, dilation=2)
    assert m.shape == (8, 16, 9, 2) and np.isfinite(m).all()
    assert np.array_equal(m[3, 5, 4], [10.0, 6.0])  # centre sample is the pixel itself
    m4, w4 = wl.four_nearest_weighted(wl.gnomonic_kernel_map(16, 32, dtype=np.float64), 16, 32)
    assert m4.shape == (16, 32, 9, 4, 2) and np.allclose(w4.sum(-1), 1, atol=1e-6)
    assert (m4 == np.round(m4)).all() and m4[..., 0].max() <= 31 and m4[..., 1].max() <= 15
    v, f = wl.icosphere(3)
    assert v.shape == (642, 3) and f.shape == (1280, 3)
    ring = wl.vertex_ring_map(3)
    assert ring.shape == (1, 642, 7, 2) and (ring[..., 1] == 0).all()
    nb = ring[0, :, 1:, 0].astype(int)
    assert all(v_ in nb[n] for v_ in range(40) for n in nb[v_])  # neighbourhood is symmetric
    assert wl.tangent_patch_map(64, 128, 1, 8).shape == (80, 64, 2)
    # the locality numbering is the same mesh: same vertex set, same neighbourhoods, and the
    # parent -> child map names the coarse vertices' own positions
    vh, fh = wl.icosphere(3, "hierarchical")
    assert np.allclose(np.sort(v, 0), np.sort(vh, 0)) and fh.shape == f.shape
    ring_h = wl.vertex_ring_map(3, order="hierarchical")[0, :, :, 0].astype(int)
    key = lambda pts: set(map(tuple, np.round(pts, 6)))
    for n in (0, 100, 641):
        old = int(np.argmin(np.abs(v - vh[n]).sum(1)))
        assert key(vh[ring_h[n]]) == key(v[ring[0, old, :, 0].astype(int)])
    c2f = wl.coarse_to_fine(3, "hierarchical")
    assert np.allclose(vh[c2f], wl.icosphere(2, "hierarchical")[0])
    assert np.array_equal(wl.coarse_to_fine(3), np.arange(162))
    spread = np.abs(ring_h[:, 1:] - ring_h[:, :1])
    assert np.median(spread) < 16   # neighbours are close in index


def test_entry_points_reject_bad_arguments_before_touching_the_device():
    """Argument checks come first in every entry point: status and message, no launch, so they
    can be exercised without a GPU."""
    from _spherical_distortion_ext import _capi
    lib = _capi.load()
    lib.sdk_last_error.restype = ctypes.c_char_p
    one = ctypes.c_void_p(16)   # a non-NULL pointer that is never dereferenced

    def rc(name, *args):
        return getattr(lib, name)(*args)

    def err():
        return lib.sdk_last_error().decode()

    # UV resampling: NULL pointers, no textures, empty planes
    assert rc("sdk_resample_from_uv_maps", None, one, one, one, 1, 1, 3, 4, 5, 6, 7, 1, 0, None) == -1
    assert "NULL" in err()
    assert rc("sdk_resample_from_uv_maps", one, one, one, one, 1, 1, 0, 4, 5, 6, 7, 1, 0, None) == -1
    assert "num_textures" in err()
    assert rc("sdk_resample_to_uv_maps", one, one, one, one, None, 0, 1, 1, 3, 0, 5, 6, 7, 1, 0,
              None) == -1
    assert rc("sdk_resample_to_uv_maps", one, one, one, one, None, 0, -1, 1, 3, 4, 5, 6, 7, 1, 0,
              None) == -1
    # an empty batch is a valid no-op, pointers or not
    assert rc("sdk_resample_from_uv_maps", None, None, None, None, 0, 4, 3, 4, 5, 6, 7, 1, 0,
              None) == 0
    assert lib.sdk_resample_to_uv_maps_workspace_bytes(80, 64, 64, 512, 1024, 0) > 512 * 1024 * 4
    assert lib.sdk_resample_to_uv_maps_workspace_bytes(3, 130, 140, 33, 47, 0) == 0   # too large for LDS
    assert lib.sdk_resample_to_uv_maps_workspace_bytes(0, 4, 4, 8, 8, 0) == 0
    # voting resample: the workspace is required
    assert rc("sdk_voting_resample_to_map", one, one, one, None, 0, 1, 1, 4, 5, 2, 3, 6, None) == -3
    assert "workspace" in err()
    assert rc("sdk_voting_resample_to_map", one, one, one, one, 1 << 20, 1, 1, 4, 5, 2, 3, 0,
              None) == -1
    assert lib.sdk_voting_resample_workspace_bytes(1, 2, 3, 6) >= 1 * 2 * 3 * 6 * 4
    # map generation
    assert rc("sdk_equirect_kernel_map", one, 1, 64, 3, 3, 1, 1, 1, 0, None) == -1
    assert "height" in err()
    assert rc("sdk_equirect_kernel_map", one, 32, 64, 3, 3, 0, 1, 1, 0, None) == -1
    assert rc("sdk_equirect_kernel_map", one, 32, 64, 3, 3, 1, 1, 7, 0, None) == -1
    assert "projection" in err()
    assert rc("sdk_equirect_kernel_map", None, 32, 64, 3, 3, 1, 1, 1, 0, None) == -1
    assert rc("sdk_gnomonic_kernel_at", None, None, 0, 3, 3, 0.1, 0.1, 0, 0, 0, None) == 0
    assert rc("sdk_four_nearest_weighted_map", None, None, None, 0, 8, 8, 1e-6, 0, None) == 0
    assert rc("sdk_four_nearest_weighted_map", one, one, one, 4, 1, 8, 1e-6, 0, None) == -1
    assert rc("sdk_four_nearest_weighted_map", one, one, one, 4, 8, 8, 0.0, 0, None) == -1
    assert rc("sdk_four_nearest_weighted_map", None, one, one, 4, 8, 8, 1e-6, 0, None) == -1
    assert rc("sdk_gnomonic_kernel_at", one, one, 5, 0, 3, 0.1, 0.1, 0, 0, 0, None) == -1
    assert rc("sdk_gnomonic_kernel_at", one, one, 5, 3, 3, 0.1, 0.1, 1, 8, 0, None) == -1
    # gather at index and average pooling share the mapped-operator checks
    assert rc("sdk_mapped_gather_at_index", one, None, one, None, one, 1, 1, 4, 5, 2, 3, 9, 0, 1, 0,
              None) == -1
    assert rc("sdk_mapped_avg_pool", one, one, None, one, 1, 1, 4, 5, 2, 3, 9, 2, 1, 0, None) == -1
    assert "interp_weights" in err()
    # unknown compute mode of a convolution call
    assert rc("sdk_mapped_conv_forward", one, one, None, one, one, one, None, 0, 1, 3, 8, 8, 4, 8, 8,
              9, 0, 1, 0, 9, None) == -1
    assert "compute" in err()
    assert lib.sdk_mapped_conv_workspace_bytes(1, 3, 4, 8, 8, 8, 8, 9, 0, 1, 0, 3) == \
        lib.sdk_mapped_conv_workspace_bytes(1, 3, 4, 8, 8, 8, 8, 9, 0, 1, 0, 0)


def test_compute_mode_override_is_scoped_and_per_thread():
    """conv_compute() overrides the mode for the block on the calling thread only and restores
    what was in force; set_conv_compute() sets the process default."""
    import threading
    from _spherical_distortion_ext import _ops
    assert _ops.get_conv_compute() == "native"
    with _ops.conv_compute("split"):
        assert _ops.get_conv_compute() == "split"
        seen = []
        th = threading.Thread(target=lambda: seen.append(_ops.get_conv_compute()))
        th.start()
        th.join()
        assert seen == ["native"]
        with _ops.conv_compute("bf16"):
            assert _ops.get_conv_compute() == "bf16"
        with _ops.conv_compute(None):
            assert _ops.get_conv_compute() == "split"
        assert _ops.get_conv_compute() == "split"
    assert _ops.get_conv_compute() == "native"
    _ops.set_conv_compute("unfused")
    try:
        assert _ops.get_conv_compute() == "unfused"
    finally:
        _ops.set_conv_compute("native")
    with pytest.raises(ValueError):
        with _ops.conv_compute("fp8"):
            pass


def test_native_override_under_a_non_native_default():
    """"native" is the C ABI's value 0: an override to it must still count as an override,
    and a mode recorded by a forward ("native") must be what conv_compute() restores for its
    backward after the process default has changed."""
    from _spherical_distortion_ext import _ops
    _ops.set_conv_compute("bf16")
    try:
        assert _ops.get_conv_compute() == "bf16"
        with _ops.conv_compute("native"):
            assert _ops.get_conv_compute() == "native"
            with _ops.conv_compute("split"):
                assert _ops.get_conv_compute() == "split"
            assert _ops.get_conv_compute() == "native"
        assert _ops.get_conv_compute() == "bf16"
    finally:
        _ops.set_conv_compute("native")
    # a forward that ran in native mode, its backward after the default moved to bf16
    recorded = _ops.get_conv_compute()
    assert recorded == "native"
    _ops.set_conv_compute("bf16")
    try:
        with _ops.conv_compute(recorded):
            assert _ops.get_conv_compute() == "native"
            assert _ops._current_mode() == 0
    finally:
        _ops.set_conv_compute("native")


def test_tensor_key_of_tensors_without_a_version_counter():
    """A tensor made under torch.inference_mode() has no version counter: the plan cache
    cannot see its in-place changes, so it gets the no-key marker and the operators go
    past the cache for it."""
    from _spherical_distortion_ext import _ops
    plain = torch.zeros(4, 5, 3, 2)
    key = _ops._tensor_key(plain)
    assert key == (plain.untyped_storage().data_ptr(), 0, plain._version, (4, 5, 3, 2))
    plain.add_(1)
    assert _ops._tensor_key(plain) != key           # an in-place change misses
    assert _ops._tensor_key(None) is None
    with torch.inference_mode():
        inf = torch.zeros(4, 5, 3, 2)
    assert inf.is_inference()
    assert _ops._tensor_key(inf) is _ops._NO_KEY
    assert _ops._uncacheable(key, _ops._NO_KEY) and not _ops._uncacheable(key, None)


def test_plan_cache_evicts_the_least_recently_used_entry():
    from _spherical_distortion_ext import _ops

    class Stream:          # stands in for a torch stream: identity and wait_stream only
        def __init__(self):
            self.waited = []

        def wait_stream(self, other):
            self.waited.append(other)

    s0, s1 = Stream(), Stream()
    saved, saved_max = dict(_ops._PLAN_CACHE), _ops._PLAN_CACHE_MAX
    _ops._PLAN_CACHE.clear()
    try:
        _ops.set_conv_plan_cache(True, max_entries=3)
        for k in "abc":
            _ops._cache_insert(k, _ops._PlanEntry(k.upper(), 1, None, s0))
        assert _ops._cache_lookup("a", s0).plan == "A" and s0.waited == []
        _ops._cache_insert("d", _ops._PlanEntry("D", 1, None, s0))     # evicts b, not a
        assert list(_ops._PLAN_CACHE) == ["c", "a", "d"]
        assert _ops._cache_lookup("b", s0) is None
        # a user on another stream is ordered behind the last user, which it then becomes
        ent = _ops._cache_lookup("c", s1)
        assert s1.waited == [s0] and ent.stream is s1
        assert _ops._cache_lookup("c", s1) is ent and s1.waited == [s0]
        assert _ops._cache_lookup("c", s0) is ent and s0.waited == [s1]
        _ops.set_conv_plan_cache(True, max_entries=1)
        assert list(_ops._PLAN_CACHE) == ["c"]
        with pytest.raises(ValueError):
            _ops.set_conv_plan_cache(True, max_entries=0)
    finally:
        _ops._PLAN_CACHE.clear()
        _ops._PLAN_CACHE.update(saved)
        _ops._PLAN_CACHE_MAX = saved_max
