"""Loader for the compiled reference CPU extensions under oracle/_ref.

TEST INFRASTRUCTURE ONLY.  `oracle/Makefile`'s `ref` target compiles the
reference's own C++ CPU sources (with -D__NO_CUDA__) into python extension
modules named as the reference's setup.py names them (setup.py:62-199).  This
module imports them when they have been built and reports their absence
otherwise; it is used to validate the restatement in oracle/sdk_oracle.cpp,
to write the fixtures under tests/golden and as the benchmark's CPU baseline.
"""
import importlib
import os
import sys

_HERE = os.path.dirname(os.path.abspath(__file__))
_REF_DIR = os.path.join(_HERE, "_ref")
_PKG = "_spherical_distortion_ext"

MODULES = ("_enums", "_resample", "_weighted_resample", "_mapped_convolution",
           "_weighted_mapped_convolution", "_mapped_transposed_convolution",
           "_weighted_mapped_transposed_convolution", "_mapped_max_pooling",
           "_weighted_mapped_max_pooling", "_mapped_avg_pooling",
           "_weighted_mapped_avg_pooling", "_uv_resample", "_voting_resample")


def available():
    d = os.path.join(_REF_DIR, _PKG)
    return os.path.isdir(d) and all(
        any(f.startswith(m + ".") for f in os.listdir(d)) for m in MODULES)


class _Ref(object):
    """Namespace holding the imported reference modules (attribute per module)."""


def load():
    """Import the compiled reference modules.  Raises ImportError when absent.

    The modules are imported under a private package path so that they can not
    be confused with the shipped `_spherical_distortion_ext` shim package."""
    if not available():
        raise ImportError("compiled reference not built (make -C oracle ref)")
    import torch  # noqa: F401  (the extensions link against libtorch)
    import importlib.util
    ns = _Ref()
    d = os.path.join(_REF_DIR, _PKG)
    for m in MODULES:  # _enums first: the other modules use its registered enum
        fn = [f for f in os.listdir(d) if f.startswith(m + ".")][0]
        spec = importlib.util.spec_from_file_location(m, os.path.join(d, fn))
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        setattr(ns, m, mod)
    ns.InterpolationType = ns._enums.InterpolationType
    return ns
