"""`_uv_resample` (reference: ext_modules/include/layers/uv_resample_layer.h)."""
from ._ops import ops


def resample_from_uv_maps(grad_output, quad_idx, tex_uv, interpolation):
    """[B, C, T, TH, TW] textures -> [B, C, H, W]: every pixel reads texture quad_idx[y, x] at
    tex_uv[y, x] (uv_resample_layer.h:76-99)."""
    return ops.resample_from_uv_maps(grad_output, quad_idx, tex_uv, int(interpolation))


def resample_to_uv_maps(input, quad_idx, tex_uv, num_textures, tex_height, tex_width,
                        interpolation):
    """The adjoint: [B, C, H, W] splatted into [B, C, T, TH, TW] (uv_resample_layer.h:48-74)."""
    return ops.resample_to_uv_maps(input, quad_idx, tex_uv, int(num_textures), int(tex_height),
                                   int(tex_width), int(interpolation))
