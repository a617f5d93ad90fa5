"""`_mapped_convolution` (reference: ext_modules/include/layers/mapped_convolution_layer.h:138-143)."""
from ._ops import ops


def mapped_conv_forward(input, sample_map, weight, bias, kernel_size, interpolation):
    """(mapped_convolution_layer.h:62-87)."""
    return ops.mapped_conv_forward(input, sample_map, None, weight, bias, int(kernel_size),
                                   int(interpolation))


def mapped_conv_backward(grad_output, sample_map, input, weight, bias, kernel_size,
                         interpolation):
    """-> [grad_input, grad_weight, grad_bias] (mapped_convolution_layer.h:89-134)."""
    return list(ops.mapped_conv_backward(grad_output, sample_map, None, input, weight, bias,
                                         int(kernel_size), int(interpolation)))
