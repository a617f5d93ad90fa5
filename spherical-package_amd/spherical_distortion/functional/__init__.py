from .mapped_ops import (mapped_convolution, mapped_transposed_convolution,  # noqa: F401
                         mapped_max_pool, mapped_max_unpool, mapped_avg_pool,
                         mapped_avg_unpool, resample, unresample, uv_resample, voting_resample, MappedConvolutionFunction,
                         MappedTransposedConvolutionFunction, MappedMaxPoolFunction,
                         MappedMaxUnpoolFunction,
                         MappedAvgPoolFunction, MappedAvgUnpoolFunction, ResampleFunction,
                         UnresampleFunction, UVResampleFunction)
