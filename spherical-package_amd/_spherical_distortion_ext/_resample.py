"""`_resample` (reference: ext_modules/include/layers/resample_layer.h:84-88)."""
from ._ops import ops


def resample_to_map(input, sample_map, output_height, output_width, interpolation):
    """Scatter `input` [B,C,IH,IW] to [B,C,output_height,output_width] through
    `sample_map` [IH,IW,2] (resample_layer.h:40-60)."""
    return ops.resample_to_map(input, sample_map, None, int(output_height), int(output_width),
                               int(interpolation))


def resample_from_map(grad_output, sample_map, interpolation):
    """Gather from `grad_output` [B,C,OH,OW] at `sample_map` [IH,IW,2] -> [B,C,IH,IW]
    (resample_layer.h:62-80)."""
    return ops.resample_from_map(grad_output, sample_map, None, int(interpolation))
