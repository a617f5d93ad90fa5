"""`_mapped_max_pooling` (reference: ext_modules/include/layers/mapped_max_pooling_layer.h:92-97)."""
from ._ops import ops


def mapped_max_pool(input, sample_map, kernel_size, interpolation):
    """-> [pooled values, int64 indices] (mapped_max_pooling_layer.h:42-62)."""
    return list(ops.mapped_max_pool(input, sample_map, None, int(kernel_size),
                                    int(interpolation)))


def mapped_max_unpool(input, idx_mask, sample_map, input_height, input_width, kernel_size,
                      interpolation):
    """(mapped_max_pooling_layer.h:64-88)."""
    return ops.mapped_max_unpool(input, idx_mask, sample_map, None, int(input_height),
                                 int(input_width), int(kernel_size), int(interpolation))
