"""Autograd functions and functional entry points of the mapped operations.

Counterpart of the reference's layers/functional/{mapped_convolution,
mapped_pooling,resample}.py: same call signatures, same choice between the
weighted and unweighted extension modules, same gradient tuple arity.
"""
import torch

import _spherical_distortion_ext._mapped_avg_pooling as _mapped_avg_pool
import _spherical_distortion_ext._mapped_convolution as _mapped_conv
import _spherical_distortion_ext._mapped_max_pooling as _mapped_max_pool
import _spherical_distortion_ext._mapped_transposed_convolution as _mapped_transposed_conv
import _spherical_distortion_ext._resample as _resample
import _spherical_distortion_ext._uv_resample as _uv_resample
import _spherical_distortion_ext._voting_resample as _voting_resample
import _spherical_distortion_ext._weighted_mapped_avg_pooling as _weighted_mapped_avg_pool
import _spherical_distortion_ext._weighted_mapped_convolution as _weighted_mapped_conv
import _spherical_distortion_ext._weighted_mapped_max_pooling as _weighted_mapped_max_pool
import _spherical_distortion_ext._weighted_mapped_transposed_convolution as _weighted_mapped_transposed_conv
import _spherical_distortion_ext._weighted_resample as _weighted_resample

from _spherical_distortion_ext._ops import conv_compute, get_conv_compute, ops as _sdk_ops

from ..layer_utils import InterpolationType, check_args, check_input_map_shape


class MappedConvolutionFunction(torch.autograd.Function):
    """layers/functional/mapped_convolution.py:14-61."""

    @staticmethod
    def forward(ctx, input, weight, bias, sample_map, kernel_size, interp, interp_weights=None):
        ctx.save_for_backward(input, weight, bias, sample_map, interp_weights)
        ctx.kernel_size = int(kernel_size)
        ctx.interp = InterpolationType(interp)
        ctx.compute = get_conv_compute()   # the backward runs in the arithmetic of the forward
        if interp_weights is None:
            return _mapped_conv.mapped_conv_forward(input, sample_map, weight, bias,
                                                    ctx.kernel_size, ctx.interp)
        return _weighted_mapped_conv.weighted_mapped_conv_forward(
            input, sample_map, interp_weights, weight, bias, ctx.kernel_size, ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        input, weight, bias, sample_map, interp_weights = ctx.saved_tensors
        with conv_compute(ctx.compute):
            if interp_weights is None:
                grads = _mapped_conv.mapped_conv_backward(grad_output, sample_map, input, weight,
                                                          bias, ctx.kernel_size, ctx.interp)
            else:
                grads = _weighted_mapped_conv.weighted_mapped_conv_backward(
                    grad_output, sample_map, interp_weights, input, weight, bias,
                    ctx.kernel_size, ctx.interp)
        grad_input, grad_weight, grad_bias = grads
        return grad_input, grad_weight, grad_bias, None, None, None, None


class MappedTransposedConvolutionFunction(torch.autograd.Function):
    """layers/functional/mapped_convolution.py:64-113."""

    @staticmethod
    def forward(ctx, input, weight, bias, sample_map, output_height, output_width, kernel_size,
                interp, interp_weights=None):
        ctx.save_for_backward(input, sample_map, weight, bias, interp_weights)
        ctx.kernel_size = int(kernel_size)
        ctx.interp = InterpolationType(interp)
        ctx.compute = get_conv_compute()
        if interp_weights is None:
            return _mapped_transposed_conv.mapped_transposed_conv_forward(
                input, sample_map, weight, bias, output_height, output_width, ctx.kernel_size,
                ctx.interp)
        return _weighted_mapped_transposed_conv.weighted_mapped_transposed_conv_forward(
            input, sample_map, interp_weights, weight, bias, output_height, output_width,
            ctx.kernel_size, ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        input, sample_map, weight, bias, interp_weights = ctx.saved_tensors
        with conv_compute(ctx.compute):
            if interp_weights is None:
                grads = _mapped_transposed_conv.mapped_transposed_conv_backward(
                    grad_output, sample_map, input, weight, bias, ctx.kernel_size, ctx.interp)
            else:
                grads = _weighted_mapped_transposed_conv.weighted_mapped_transposed_conv_backward(
                    grad_output, sample_map, interp_weights, input, weight, bias,
                    ctx.kernel_size, ctx.interp)
        grad_input, grad_weight, grad_bias = grads
        return grad_input, grad_weight, grad_bias, None, None, None, None, None, None


class MappedMaxPoolFunction(torch.autograd.Function):
    """layers/functional/mapped_pooling.py:106-153: returns (pooled, idx_mask);
    idx_mask is not differentiable."""

    @staticmethod
    def forward(ctx, input, sample_map, kernel_size, interp, interp_weights=None):
        interp = InterpolationType(interp)
        if interp_weights is None:
            pooled, idx_mask = _mapped_max_pool.mapped_max_pool(input, sample_map, kernel_size,
                                                                interp)
        else:
            pooled, idx_mask = _weighted_mapped_max_pool.weighted_mapped_max_pool(
                input, sample_map, interp_weights, kernel_size, interp)
        ctx.mark_non_differentiable(idx_mask)
        ctx.save_for_backward(idx_mask, sample_map, interp_weights)
        ctx.in_hw = (int(input.shape[2]), int(input.shape[3]))
        ctx.kernel_size = int(kernel_size)
        ctx.interp = interp
        return pooled, idx_mask

    @staticmethod
    def backward(ctx, grad_output, idx_mask_grad=None):
        idx_mask, sample_map, interp_weights = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if interp_weights is None:
            grad_input = _mapped_max_pool.mapped_max_unpool(
                grad_output, idx_mask, sample_map, ctx.in_hw[0], ctx.in_hw[1], ctx.kernel_size,
                ctx.interp)
        else:
            grad_input = _weighted_mapped_max_pool.weighted_mapped_max_unpool(
                grad_output, idx_mask, sample_map, interp_weights, ctx.in_hw[0], ctx.in_hw[1],
                ctx.kernel_size, ctx.interp)
        return grad_input, None, None, None, None


class MappedMaxUnpoolFunction(torch.autograd.Function):
    """Unpooling as a layer of its own: the pooled values go back to the samples `idx_mask`
    names, on an output of the given size; the gradient reads `grad_output` at those samples.
    The reference's class of this name (layers/functional/mapped_pooling.py:156-199) refers to
    undefined variables and pools the gradient again; this is the working form of it, with the
    output size as an explicit argument."""

    @staticmethod
    def forward(ctx, input, idx_mask, sample_map, output_height, output_width, kernel_size,
                interp, interp_weights=None):
        interp = InterpolationType(interp)
        ctx.save_for_backward(idx_mask, sample_map, interp_weights)
        ctx.kernel_size = int(kernel_size)
        ctx.interp = interp
        if interp_weights is None:
            return _mapped_max_pool.mapped_max_unpool(input, idx_mask, sample_map, output_height,
                                                      output_width, kernel_size, interp)
        return _weighted_mapped_max_pool.weighted_mapped_max_unpool(
            input, idx_mask, sample_map, interp_weights, output_height, output_width, kernel_size,
            interp)

    @staticmethod
    def backward(ctx, grad_output):
        idx_mask, sample_map, interp_weights = ctx.saved_tensors
        grad = _sdk_ops.mapped_gather_at_index(grad_output.contiguous(), idx_mask, sample_map,
                                               interp_weights, ctx.kernel_size, int(ctx.interp))
        return grad, None, None, None, None, None, None, None


def _avg_pool(input, sample_map, interp_weights, kernel_size, interp):
    if interp_weights is None:
        return _mapped_avg_pool.mapped_avg_pool(input, sample_map, kernel_size, interp)
    return _weighted_mapped_avg_pool.weighted_mapped_avg_pool(input, sample_map, interp_weights,
                                                              kernel_size, interp)


def _avg_unpool(input, sample_map, interp_weights, height, width, kernel_size, interp):
    if interp_weights is None:
        return _mapped_avg_pool.mapped_avg_unpool(input, sample_map, height, width, kernel_size,
                                                  interp)
    return _weighted_mapped_avg_pool.weighted_mapped_avg_unpool(
        input, sample_map, interp_weights, height, width, kernel_size, interp)


class MappedAvgPoolFunction(torch.autograd.Function):
    """Forward mean of the K samples, backward its adjoint
    (layers/functional/mapped_pooling.py:10-57)."""

    @staticmethod
    def forward(ctx, input, sample_map, kernel_size, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.in_hw = (int(input.shape[2]), int(input.shape[3]))
        ctx.kernel_size = int(kernel_size)
        ctx.interp = InterpolationType(interp)
        return _avg_pool(input, sample_map, interp_weights, ctx.kernel_size, ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        grad = _avg_unpool(grad_output.contiguous(), sample_map, interp_weights, ctx.in_hw[0],
                           ctx.in_hw[1], ctx.kernel_size, ctx.interp)
        return grad, None, None, None, None


class MappedAvgUnpoolFunction(torch.autograd.Function):
    """Forward the adjoint of average pooling onto an oh x ow image, backward the pooling
    (layers/functional/mapped_pooling.py:60-103)."""

    @staticmethod
    def forward(ctx, input, oh, ow, sample_map, kernel_size, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.kernel_size = int(kernel_size)
        ctx.interp = InterpolationType(interp)
        return _avg_unpool(input, sample_map, interp_weights, int(oh), int(ow), ctx.kernel_size,
                           ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        grad = _avg_pool(grad_output.contiguous(), sample_map, interp_weights, ctx.kernel_size,
                         ctx.interp)
        return grad, None, None, None, None, None, None


class ResampleFunction(torch.autograd.Function):
    """Forward scatter, backward gather (layers/functional/resample.py:11-48)."""

    @staticmethod
    def forward(ctx, input, sample_map, output_shape, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.interp = InterpolationType(interp)
        if interp_weights is None:
            return _resample.resample_to_map(input, sample_map, output_shape[0], output_shape[1],
                                             ctx.interp)
        return _weighted_resample.weighted_resample_to_map(
            input, sample_map, interp_weights, output_shape[0], output_shape[1], ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if interp_weights is None:
            grad = _resample.resample_from_map(grad_output, sample_map, ctx.interp)
        else:
            grad = _weighted_resample.weighted_resample_from_map(grad_output, sample_map,
                                                                 interp_weights, ctx.interp)
        return grad, None, None, None, None


class UnresampleFunction(torch.autograd.Function):
    """Forward gather, backward scatter (layers/functional/resample.py:51-83)."""

    @staticmethod
    def forward(ctx, input, sample_map, interp, interp_weights=None):
        ctx.save_for_backward(sample_map, interp_weights)
        ctx.interp = InterpolationType(interp)
        ctx.in_hw = (int(input.shape[2]), int(input.shape[3]))
        if interp_weights is None:
            return _resample.resample_from_map(input, sample_map, ctx.interp)
        return _weighted_resample.weighted_resample_from_map(input, sample_map, interp_weights,
                                                             ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        sample_map, interp_weights = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if interp_weights is None:
            grad = _resample.resample_to_map(grad_output, sample_map, ctx.in_hw[0], ctx.in_hw[1],
                                             ctx.interp)
        else:
            grad = _weighted_resample.weighted_resample_to_map(
                grad_output, sample_map, interp_weights, ctx.in_hw[0], ctx.in_hw[1], ctx.interp)
        return grad, None, None, None


class UVResampleFunction(torch.autograd.Function):
    """Forward gather from a stack of textures, backward the splat into it
    (layers/functional/resample.py:86-110)."""

    @staticmethod
    def forward(ctx, input, quad_idx, tex_uv, interp):
        ctx.save_for_backward(quad_idx, tex_uv)
        ctx.interp = InterpolationType(interp)
        ctx.tex_shape = tuple(int(v) for v in input.shape[-3:])
        return _uv_resample.resample_from_uv_maps(input, quad_idx, tex_uv, ctx.interp)

    @staticmethod
    def backward(ctx, grad_output):
        quad_idx, tex_uv = ctx.saved_tensors
        grad = _uv_resample.resample_to_uv_maps(grad_output.contiguous(), quad_idx, tex_uv,
                                                ctx.tex_shape[0], ctx.tex_shape[1],
                                                ctx.tex_shape[2], ctx.interp)
        return grad, None, None, None


# ----------------------------------------------------------------------------- entry points
def mapped_convolution(input, weight, bias, sample_map, kernel_size, interp,
                       interp_weights=None, compute=None):
    """layers/functional/mapped_convolution.py:121-131.  compute (not in the reference): the
    arithmetic of this call and of its backward ("native", "split", "bf16", "unfused"); None
    takes the mode in force (set_conv_compute / conv_compute)."""
    check_args(input, sample_map, interp_weights, weight.shape[1], weight.shape[2])
    with conv_compute(compute):
        return MappedConvolutionFunction.apply(input, weight, bias, sample_map, kernel_size,
                                               interp, interp_weights)


def mapped_transposed_convolution(input, weight, bias, sample_map, output_height, output_width,
                                  kernel_size, interp, interp_weights=None, compute=None):
    """layers/functional/mapped_convolution.py:134-148.  compute: as for mapped_convolution."""
    check_args(input, sample_map, interp_weights, weight.shape[0], weight.shape[2])
    check_input_map_shape(input, sample_map)
    with conv_compute(compute):
        return MappedTransposedConvolutionFunction.apply(input, weight, bias, sample_map,
                                                         output_height, output_width,
                                                         kernel_size, interp, interp_weights)


def mapped_max_pool(input, sample_map, kernel_size, interp, interp_weights=None):
    """-> (pooled, idx_mask); layers/functional/mapped_pooling.py:225-232."""
    check_args(input, sample_map, interp_weights, None, kernel_size)
    return MappedMaxPoolFunction.apply(input, sample_map, kernel_size, interp, interp_weights)


def mapped_max_unpool(input, idx_mask, sample_map, output_shape, kernel_size, interp,
                      interp_weights=None):
    """Pooled values back onto an `output_shape` = (H, W) image at the samples `idx_mask` names
    (the reference's function of this name, layers/functional/mapped_pooling.py:235-242, calls
    the pooling function with these arguments and cannot run)."""
    check_args(input, sample_map, interp_weights, None, kernel_size)
    check_input_map_shape(input, sample_map)
    return MappedMaxUnpoolFunction.apply(input, idx_mask, sample_map, output_shape[0],
                                         output_shape[1], kernel_size, interp, interp_weights)


def mapped_avg_pool(input, sample_map, kernel_size, interp, interp_weights=None):
    """layers/functional/mapped_pooling.py:202-209."""
    check_args(input, sample_map, interp_weights, None, kernel_size)
    return MappedAvgPoolFunction.apply(input, sample_map, kernel_size, interp, interp_weights)


def mapped_avg_unpool(input, oh, ow, sample_map, kernel_size, interp, interp_weights=None):
    """layers/functional/mapped_pooling.py:212-222."""
    check_args(input, sample_map, interp_weights, None, kernel_size)
    check_input_map_shape(input, sample_map)
    return MappedAvgUnpoolFunction.apply(input, oh, ow, sample_map, kernel_size, interp,
                                         interp_weights)


def _with_batch_dim(input):
    assert input.dim() in [3, 4], \
        'Input must have 3 or 4 dimensions (input.dim() == {})'.format(input.dim())
    return (input.unsqueeze(0), True) if input.dim() == 3 else (input, False)


def resample(input, sample_map, output_shape, interp, interp_weights=None):
    """Scatter `input` through the map; a 3-D input is treated as one batch element
    (layers/functional/resample.py:113-134)."""
    batched, added = _with_batch_dim(input)
    check_args(batched, sample_map, interp_weights, None, None)
    check_input_map_shape(batched, sample_map)
    out = ResampleFunction.apply(batched, sample_map, output_shape, interp, interp_weights)
    return out.squeeze(0) if added else out


def unresample(input, sample_map, interp, interp_weights=None):
    """Gather from `input` at the map (layers/functional/resample.py:137-157)."""
    batched, added = _with_batch_dim(input)
    check_args(batched, sample_map, interp_weights, None, None)
    out = UnresampleFunction.apply(batched, sample_map, interp, interp_weights)
    return out.squeeze(0) if added else out


def uv_resample(input, quad_idx, tex_uv, interp):
    """[B, C, T, TH, TW] (or [C, T, TH, TW]) textures -> [B, C, H, W] image: pixel (y, x) reads
    texture quad_idx[y, x] at tex_uv[y, x] (layers/functional/resample.py:192-209)."""
    assert input.dim() in [4, 5], \
        'Input must have 4 or 5 dimensions (input.dim() == {})'.format(input.dim())
    added = input.dim() == 4
    out = UVResampleFunction.apply(input.unsqueeze(0) if added else input, quad_idx, tex_uv,
                                   interp)
    return out.squeeze(0) if added else out


def voting_resample(input, sample_map, interp_weights, output_shape, num_candidates):
    """Labels scattered through the map, every output pixel keeping the label with the most
    votes; input and map are cast to int64 as the reference does, `interp_weights` is accepted
    and unused as there (layers/functional/resample.py:160-189)."""
    batched, added = _with_batch_dim(input)
    check_input_map_shape(batched, sample_map)
    out = _voting_resample.voting_resample_to_map(batched.long().contiguous(),
                                                  sample_map.long().contiguous(),
                                                  output_shape[0], output_shape[1],
                                                  num_candidates)
    return out.squeeze(0) if added else out
