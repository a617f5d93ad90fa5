"""`_mapped_avg_pooling` (reference: ext_modules/include/layers/mapped_avg_pooling_layer.h)."""
from ._ops import ops


def mapped_avg_pool(input, sample_map, kernel_size, interpolation):
    """-> pooled values: the mean of the K interpolated samples of every output pixel."""
    return ops.mapped_avg_pool(input, sample_map, None, int(kernel_size), int(interpolation))


def mapped_avg_unpool(input, sample_map, input_height, input_width, kernel_size, interpolation):
    """The adjoint: input / K splatted at every sample of its pixel."""
    return ops.mapped_avg_unpool(input, sample_map, None, int(input_height), int(input_width),
                                 int(kernel_size), int(interpolation))
