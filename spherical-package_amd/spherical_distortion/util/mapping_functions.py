"""Sample-map builders, computed on the GPU.

Counterpart of the reference's layers/util/mapping_functions.py (equirectangular kernel maps,
:43-160) and of `gnomonic_kernel` in layers/util/icosahedron_functions.py:47-103: same names,
arguments and output layouts.  The reference evaluates these with tensor operations on the host;
here one kernel launch writes the map straight into device memory, where the mapped operations
read it.  Maps that need a mesh (icosphere vertices and faces) take the points as a tensor.
"""
import math

import torch

from _spherical_distortion_ext import _ops

GRID, INVERSE_GNOMONIC, INVERSE_EQUIRECTANGULAR = 0, 1, 2


def get_equirectangular_grid_resolution(shape):
    """(res_lon, res_lat) between neighbouring pixels (layers/util/grids.py:5-10)."""
    H, W = shape
    return 2 * math.pi / W, math.pi / (H - 1)


def _kernel_map(shape, kernel_size, stride, dilation, projection, dtype, device):
    H, W = shape
    kh, kw = kernel_size
    return _ops.equirect_kernel_map(H, W, kh, kw, stride, dilation, projection, dtype, device)


def grid_projection_map(shape, kernel_size, stride=1, dilation=1, dtype=torch.float32,
                        device="cuda"):
    """H/stride x W/stride x kh*kw x 2 map of the plain pixel-grid kernel
    (layers/util/mapping_functions.py:43-75)."""
    return _kernel_map(shape, kernel_size, stride, dilation, GRID, dtype, device)


def inverse_gnomonic_projection_map(shape, kernel_size, stride=1, dilation=1,
                                    dtype=torch.float32, device="cuda"):
    """The kernel laid on the plane tangent at every pixel and projected back onto the sphere
    (layers/util/mapping_functions.py:78-120)."""
    return _kernel_map(shape, kernel_size, stride, dilation, INVERSE_GNOMONIC, dtype, device)


def inverse_equirectangular_projection_map(shape, kernel_size, stride=1, dilation=1,
                                           dtype=torch.float32, device="cuda"):
    """Longitude steps widened by 1 / cos(latitude) (layers/util/mapping_functions.py:123-160)."""
    return _kernel_map(shape, kernel_size, stride, dilation, INVERSE_EQUIRECTANGULAR, dtype,
                       device)


def gnomonic_kernel(spherical_coords, kh, kw, res_lat, res_lon):
    """(1, N, kh*kw, 2) gnomonic kernels in (lon, lat) about the N points of `spherical_coords`
    [N, 2] (layers/util/icosahedron_functions.py:47-103)."""
    pts = spherical_coords.reshape(-1, 2).contiguous()
    return _ops.gnomonic_kernel_at(pts, kh, kw, res_lat, res_lon).unsqueeze(0)


def gnomonic_kernel_pixels(spherical_coords, kh, kw, res_lat, res_lon, image_shape):
    """`gnomonic_kernel` followed by `convert_spherical_to_image`
    (layers/util/conversions.py:33-52) in one launch: [N, kh*kw, 2] pixel coordinates of an
    equirectangular image, the sample map of tangent images and icosphere kernels
    (layers/util/tangent_images.py:59-109)."""
    pts = spherical_coords.reshape(-1, 2).contiguous()
    return _ops.gnomonic_kernel_at(pts, kh, kw, res_lat, res_lon, image_shape[0], image_shape[1])


def four_nearest_weighted(sample_map, image_shape, eps=1e-6):
    """(map [..., 4, 2], weights [..., 4]) from a map of single points [..., 2]: the four pixel
    centres around every sample of an equirectangular image (columns wrap, rows clamp) and
    weights proportional to 1 / (great-circle distance + eps), normalised to one.  No
    counterpart in the reference, whose weighted maps come from its mesh code."""
    return _ops.four_nearest_weighted_map(sample_map.contiguous(), image_shape[0], image_shape[1],
                                          eps)
