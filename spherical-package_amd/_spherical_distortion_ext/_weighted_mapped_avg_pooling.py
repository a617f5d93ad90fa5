"""`_weighted_mapped_avg_pooling`
(reference: ext_modules/include/layers/weighted_mapped_avg_pooling_layer.h)."""
from ._ops import ops


def weighted_mapped_avg_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    return ops.mapped_avg_pool(input, sample_map, interp_weights, int(kernel_size),
                               int(interpolation))


def weighted_mapped_avg_unpool(input, sample_map, interp_weights, input_height, input_width,
                               kernel_size, interpolation):
    return ops.mapped_avg_unpool(input, sample_map, interp_weights, int(input_height),
                                 int(input_width), int(kernel_size), int(interpolation))
