"""nn.Module front-ends of the mapped operations.

Constructor and forward signatures, parameter shapes and initialisation follow
the reference's layers/nn/{mapped_convolution_layer,mapped_transposed_convolution_layer,
mapped_max_pooling_layer,resample_layer}.py.
"""
import math

import torch
import torch.nn as nn

from .. import functional as F
from ..layer_utils import InterpolationType


def _init_uniform(weight, bias, fan_in):
    """uniform(-1/sqrt(fan_in), +1/sqrt(fan_in)) for both parameters
    (mapped_convolution_layer.py:42-49)."""
    bound = 1.0 / math.sqrt(fan_in)
    with torch.no_grad():
        weight.uniform_(-bound, bound)
        bias.uniform_(-bound, bound)


class MappedConvolution(nn.Module):
    """Convolution whose K taps per output pixel are read where `sample_map`
    says.  weight [out_channels, in_channels, kernel_size]; `bias=False` keeps a
    zero bias parameter (mapped_convolution_layer.py:14-59).  compute (not in the reference):
    this layer's arithmetic, "native", "split", "bf16" or "unfused"; None follows
    set_conv_compute."""

    def __init__(self, in_channels, out_channels, kernel_size=1,
                 interpolation=InterpolationType.BILINEAR, bias=True, compute=None):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.interp = interpolation
        self.compute = compute
        self.weight = nn.Parameter(torch.empty(out_channels, in_channels, kernel_size))
        self.bias = nn.Parameter(torch.empty(out_channels))
        self.reset_parameters()
        if not bias:
            self.bias = nn.Parameter(torch.zeros(out_channels))

    def reset_parameters(self):
        _init_uniform(self.weight, self.bias, self.in_channels * self.kernel_size)

    def forward(self, x, sample_map, interp_weights=None):
        """x [B,Cin,H,W]; sample_map [OH,OW,K,2] or, with interp_weights [OH,OW,K,P],
        [OH,OW,K,P,2]."""
        return F.mapped_convolution(x, self.weight, self.bias, sample_map, self.kernel_size,
                                    self.interp, interp_weights, self.compute)


class MappedTransposedConvolution(nn.Module):
    """The map has the input's H x W and points into the [oh, ow] output.
    weight [in_channels, out_channels, kernel_size]
    (mapped_transposed_convolution_layer.py:10-56).  compute: as for MappedConvolution."""

    def __init__(self, in_channels, out_channels, kernel_size=1,
                 interpolation=InterpolationType.BILINEAR, bias=True, compute=None):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.interp = interpolation
        self.compute = compute
        self.weight = nn.Parameter(torch.empty(in_channels, out_channels, kernel_size))
        self.bias = nn.Parameter(torch.empty(out_channels))
        self.reset_parameters()
        if not bias:
            self.bias = nn.Parameter(torch.zeros(out_channels))

    def reset_parameters(self):
        _init_uniform(self.weight, self.bias, self.in_channels * self.kernel_size)

    def forward(self, x, oh, ow, sample_map, interp_weights=None):
        return F.mapped_transposed_convolution(x, self.weight, self.bias, sample_map, oh, ow,
                                               self.kernel_size, self.interp, interp_weights,
                                               self.compute)


class MappedMaxPool(nn.Module):
    """(mapped_max_pooling_layer.py:8-29)."""

    def __init__(self, kernel_size, interpolation=InterpolationType.BILINEAR,
                 return_indices=False):
        super().__init__()
        self.kernel_size = kernel_size
        self.interp = interpolation
        self.return_indices = return_indices

    def forward(self, x, sample_map, interp_weights=None):
        pooled, idx_mask = F.mapped_max_pool(x, sample_map, self.kernel_size, self.interp,
                                             interp_weights)
        return (pooled, idx_mask) if self.return_indices else pooled


class MappedMaxUnpool(nn.Module):
    """Pooled values back to the samples that won (mapped_max_pooling_layer.py:35-47, whose
    functional backend cannot run in the reference; `output_shape` = (H, W) of the unpooled
    image is an added argument)."""

    def __init__(self, kernel_size, interpolation=InterpolationType.BILINEAR):
        super().__init__()
        self.kernel_size = kernel_size
        self.interp = interpolation

    def forward(self, x, idx_mask, sample_map, output_shape, interp_weights=None):
        return F.mapped_max_unpool(x, idx_mask, sample_map, output_shape, self.kernel_size,
                                   self.interp, interp_weights)


class MappedAvgPool(nn.Module):
    """(mapped_avg_pooling_layer.py:7-19)."""

    def __init__(self, kernel_size, interpolation=InterpolationType.BILINEAR):
        super().__init__()
        self.kernel_size = kernel_size
        self.interp = interpolation

    def forward(self, x, sample_map, interp_weights=None):
        return F.mapped_avg_pool(x, sample_map, self.kernel_size, self.interp, interp_weights)


class MappedAvgUnpool(nn.Module):
    """x on the map's grid is spread, divided by the kernel size, over the samples of each of
    its pixels in an oh x ow image (mapped_avg_pooling_layer.py:22-44)."""

    def __init__(self, kernel_size, interpolation=InterpolationType.BILINEAR):
        super().__init__()
        self.kernel_size = kernel_size
        self.interp = interpolation

    def forward(self, x, oh, ow, sample_map, interp_weights=None):
        return F.mapped_avg_unpool(x, oh, ow, sample_map, self.kernel_size, self.interp,
                                   interp_weights)


class Resample(nn.Module):
    """Scatter: integer input locations go to the real-valued output locations
    the map gives (resample_layer.py:13-32)."""

    def __init__(self, interpolation=InterpolationType.BILINEAR):
        super().__init__()
        self.interp = interpolation

    def forward(self, x, sample_map, output_shape, interp_weights=None):
        return F.resample(x, sample_map, output_shape, self.interp, interp_weights)


class Unresample(nn.Module):
    """Gather: each map location is read from the input by interpolation
    (resample_layer.py:35-52)."""

    def __init__(self, interpolation=InterpolationType.BILINEAR):
        super().__init__()
        self.interp = interpolation

    def forward(self, x, sample_map, interp_weights=None):
        return F.unresample(x, sample_map, self.interp, interp_weights)


class UVResample(nn.Module):
    """Tangent images (a stack of textures) back to one image: the resampling step of the
    reference's TangentImagesToEquirectangular (layers/nn/tangent_image_layer.py:42-70), with
    the per-pixel texture index and UV coordinates handed in as tensors instead of being
    generated from an icosphere in the constructor."""

    def __init__(self, quad_idx, tex_uv, interpolation=InterpolationType.BILINEAR):
        super().__init__()
        self.register_buffer('quad', quad_idx)
        self.register_buffer('uv', tex_uv)
        self.interp = interpolation

    def forward(self, x):
        return F.uv_resample(x, self.quad, self.uv, self.interp)
