"""`_weighted_resample` (reference: ext_modules/include/layers/weighted_resample_layer.h:105-110)."""
from ._ops import ops


def weighted_resample_to_map(input, sample_map, interp_weights, output_height, output_width,
                             interpolation):
    """sample_map [IH,IW,P,2], interp_weights [IH,IW,P] (weighted_resample_layer.h:49-74)."""
    return ops.resample_to_map(input, sample_map, interp_weights, int(output_height),
                               int(output_width), int(interpolation))


def weighted_resample_from_map(grad_output, sample_map, interp_weights, interpolation):
    """(weighted_resample_layer.h:76-101)."""
    return ops.resample_from_map(grad_output, sample_map, interp_weights, int(interpolation))
