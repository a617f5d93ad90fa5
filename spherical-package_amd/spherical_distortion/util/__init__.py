from .mapping_functions import (get_equirectangular_grid_resolution,  # noqa: F401
                                grid_projection_map, inverse_gnomonic_projection_map,
                                inverse_equirectangular_projection_map, gnomonic_kernel,
                                gnomonic_kernel_pixels, four_nearest_weighted)
