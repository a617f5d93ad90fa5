"""`_weighted_mapped_transposed_convolution`
(reference: ext_modules/include/layers/weighted_mapped_transposed_convolution_layer.h:155-160)."""
from ._ops import ops


def weighted_mapped_transposed_conv_forward(input, sample_map, interp_weights, weight, bias,
                                            output_height, output_width, kernel_size,
                                            interpolation):
    return ops.mapped_transposed_conv_forward(input, sample_map, interp_weights, weight, bias,
                                              int(output_height), int(output_width),
                                              int(kernel_size), int(interpolation))


def weighted_mapped_transposed_conv_backward(grad_output, sample_map, interp_weights, input,
                                             weight, bias, kernel_size, interpolation):
    return list(ops.mapped_transposed_conv_backward(grad_output, sample_map, interp_weights,
                                                    input, weight, bias, int(kernel_size),
                                                    int(interpolation)))
