"""`_weighted_mapped_convolution`
(reference: ext_modules/include/layers/weighted_mapped_convolution_layer.h:157-162)."""
from ._ops import ops


def weighted_mapped_conv_forward(input, sample_map, interp_weights, weight, bias, kernel_size,
                                 interpolation):
    """(weighted_mapped_convolution_layer.h:69-101)."""
    return ops.mapped_conv_forward(input, sample_map, interp_weights, weight, bias,
                                   int(kernel_size), int(interpolation))


def weighted_mapped_conv_backward(grad_output, sample_map, interp_weights, input, weight, bias,
                                  kernel_size, interpolation):
    """(weighted_mapped_convolution_layer.h:103-153)."""
    return list(ops.mapped_conv_backward(grad_output, sample_map, interp_weights, input, weight,
                                         bias, int(kernel_size), int(interpolation)))
