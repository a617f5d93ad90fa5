"""Drop-in for the reference's compiled extension package of the same name.

The reference builds one pybind11 module per operator family into the package
`_spherical_distortion_ext` (reference setup.py:62-199, :209).  This package
offers the mapped-operation subset of those modules, with the same module and
function names and argument orders, implemented by the hand-written gfx950 HIP
kernels in libsdk_mapped_ops.so:

    _enums, _resample, _weighted_resample, _mapped_convolution,
    _weighted_mapped_convolution, _mapped_transposed_convolution,
    _weighted_mapped_transposed_convolution, _mapped_max_pooling,
    _weighted_mapped_max_pooling, _mapped_avg_pooling, _weighted_mapped_avg_pooling,
    _uv_resample, _voting_resample

Importing the package loads the library and registers the operators; it raises
ImportError when the library has not been built.
"""
from . import _capi

_capi.load()

from . import _ops  # noqa: E402  (registers torch.ops.sdk_mapped_ops.*)
from . import _enums  # noqa: E402,F401
