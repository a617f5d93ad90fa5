"""`_mapped_transposed_convolution`
(reference: ext_modules/include/layers/mapped_transposed_convolution_layer.h:144-149)."""
from ._ops import ops


def mapped_transposed_conv_forward(input, sample_map, weight, bias, output_height, output_width,
                                   kernel_size, interpolation):
    """(mapped_transposed_convolution_layer.h:62-93)."""
    return ops.mapped_transposed_conv_forward(input, sample_map, None, weight, bias,
                                              int(output_height), int(output_width),
                                              int(kernel_size), int(interpolation))


def mapped_transposed_conv_backward(grad_output, sample_map, input, weight, bias, kernel_size,
                                    interpolation):
    """(mapped_transposed_convolution_layer.h:95-140)."""
    return list(ops.mapped_transposed_conv_backward(grad_output, sample_map, None, input, weight,
                                                    bias, int(kernel_size), int(interpolation)))
