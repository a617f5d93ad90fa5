"""Host-side layers of the mapped-operation backend.

Mirrors the part of the reference's `spherical_distortion` package (its
`layers/` directory, reference setup.py:211-228) that sits on the mapped
operation path: `nn.MappedConvolution`, `nn.MappedTransposedConvolution`,
`nn.MappedMaxPool`, `nn.MappedAvgPool`, `nn.MappedAvgUnpool`, `nn.Resample`, `nn.Unresample` and the matching
`functional` entry points, with the reference's names, signatures, parameter
shapes, initialisation and argument checks.  The arithmetic is done by the
gfx950 HIP kernels behind `_spherical_distortion_ext`.
"""
__version__ = "1.1.0+mi355x"
