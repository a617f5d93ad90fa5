from .mapped_ops import (mapped_convolution, mapped_transposed_convolution,  # noqa: F401
                         mapped_max_pool, resample, unresample,
                         MappedConvolutionFunction, MappedTransposedConvolutionFunction,
                         MappedMaxPoolFunction, ResampleFunction, UnresampleFunction)
