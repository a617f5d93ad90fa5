"""Argument validation shared by the functional entry points, and the enum.

Behaviour follows the reference's layers/layer_utils.py: the same assertions
fire for the same inputs (AssertionError), in the same order.
"""
from _spherical_distortion_ext._enums import InterpolationType  # noqa: F401


def _pair(value):
    """A scalar becomes a 2-tuple; an iterable is passed through (layer_utils.py:11-24)."""
    try:
        iter(value)
        return value
    except TypeError:
        return (value, value)


def check_input_dim(input):
    assert input.dim() == 4, 'Input must have 4 dimensions ({} != 4)'.format(input.dim())


def check_sample_map_dim(sample_map, interp_weights=None, kernel=True):
    """Map rank: [OH,OW,(K,)2] unweighted, [OH,OW,(K,)P,2] weighted (layer_utils.py:47-77)."""
    want = 3 + (1 if kernel else 0) + (0 if interp_weights is None else 1)
    assert sample_map.dim() == want, \
        'Sample map must have {} dimensions ({} != {})'.format(want, sample_map.dim(), want)
    assert sample_map.shape[-1] == 2, \
        'Last dimension of sample map must have size 2 ({} != 2)'.format(sample_map.shape[-1])


def check_interp_weights_dim(interp_weights, kernel=True):
    want = 4 if kernel else 3
    assert interp_weights.dim() == want, \
        'Interpolation weights must have {} dimensions ({} != {})'.format(
            want, interp_weights.dim(), want)


def check_type(input, sample_map, interp_weights=None):
    """Data, map and weights share one dtype (layer_utils.py:27-36)."""
    assert input.dtype == sample_map.dtype, \
        'Input and sample map must be the same dtype ({} != {})'.format(
            input.dtype, sample_map.dtype)
    if interp_weights is not None:
        assert input.dtype == interp_weights.dtype, \
            'Input and interpolation weights must be the same dtype ({} != {})'.format(
                input.dtype, interp_weights.dtype)


def check_input_shape(input, in_channels):
    assert input.shape[1] == in_channels, \
        'Number of input channels must match weight parameter ({} != {})'.format(
            input.shape[1], in_channels)


def check_sample_map_shape(sample_map, kernel_size):
    assert sample_map.shape[2] == kernel_size, \
        'Kernel size of sample map must match weight parameter ({} != {})'.format(
            sample_map.shape[2], kernel_size)


def check_interp_weights_shape(sample_map, interp_weights):
    assert sample_map.shape[-2] == interp_weights.shape[-1], \
        'Sample map and interpolation weights should have the same number of ' \
        'interpolation points ({} != {})'.format(sample_map.shape[-2], interp_weights.shape[-1])


def check_input_map_shape(input, sample_map):
    """The map grid equals the input's H x W (layer_utils.py:123-128)."""
    assert tuple(input.shape[2:4]) == tuple(sample_map.shape[0:2]), \
        'Input dimensions 2 and 3 must match sample map dimensions 0 and 1 ' \
        '({},{}) != ({},{})'.format(input.shape[2], input.shape[3],
                                    sample_map.shape[0], sample_map.shape[1])


def check_args(input, sample_map, interp_weights, in_channels, kernel_size):
    """Order as in layer_utils.py:131-154: ranks, dtypes, then sizes."""
    has_kernel = kernel_size is not None
    check_input_dim(input)
    check_sample_map_dim(sample_map, interp_weights, has_kernel)
    if interp_weights is not None:
        check_interp_weights_dim(interp_weights, has_kernel)
    check_type(input, sample_map, interp_weights)
    if in_channels is not None:
        check_input_shape(input, in_channels)
    if has_kernel:
        check_sample_map_shape(sample_map, kernel_size)
    if interp_weights is not None:
        check_interp_weights_shape(sample_map, interp_weights)
