"""`_weighted_mapped_max_pooling`
(reference: ext_modules/include/layers/weighted_mapped_max_pooling_layer.h:101-104)."""
from ._ops import ops


def weighted_mapped_max_pool(input, sample_map, interp_weights, kernel_size, interpolation):
    return list(ops.mapped_max_pool(input, sample_map, interp_weights, int(kernel_size),
                                    int(interpolation)))


def weighted_mapped_max_unpool(input, idx_mask, sample_map, interp_weights, input_height,
                               input_width, kernel_size, interpolation):
    return ops.mapped_max_unpool(input, idx_mask, sample_map, interp_weights, int(input_height),
                                 int(input_width), int(kernel_size), int(interpolation))
