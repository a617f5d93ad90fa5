"""`_voting_resample` (reference: ext_modules/include/layers/voting_resample_layer.h)."""
from ._ops import ops


def voting_resample_to_map(input, sample_map, output_height, output_width, num_candidates):
    """int64 labels [B, C, IH, IW] through an int64 map [IH, IW, 2] -> [B, C, OH, OW]: per output
    pixel the label most of its sources carry (voting_resample_layer.h:31-53)."""
    return ops.voting_resample_to_map(input, sample_map, int(output_height), int(output_width),
                                      int(num_candidates))
