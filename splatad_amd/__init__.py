"""MI355X-native rendering hot path of SplatAD behind the gsplat operator API.

Exports the operators and end-to-end functions of the reference's gsplat/__init__.py:3-24 that
lie on the path projection -> tile intersection -> rasterization, and the lidar point binning
that prepares the points to render.
"""
from .hip._torch_impl import accumulate, accumulate_lidar
from .hip._wrapper import (
    compute_lidar_velocity,
    compute_pix_velocity,
    lidar_proj,
    persp_proj,
    quat_scale_to_covar_preci,
    world_to_cam,
    fully_fused_lidar_projection,
    fully_fused_projection,
    isect_lidar_tiles,
    isect_offset_encode,
    isect_tiles,
    map_points_to_lidar_tiles,
    points_mapping_offset_encode,
    populate_image_from_points,
    rasterize_to_indices_in_range,
    rasterize_to_indices_in_range_lidar,
    rasterize_to_pixels,
    rasterize_to_points,
    spherical_harmonics,
)
from .rendering import lidar_rasterization, rasterization

__version__ = "0.1.0"

__all__ = [
    "rasterization",
    "lidar_rasterization",
    "fully_fused_projection",
    "fully_fused_lidar_projection",
    "isect_tiles",
    "isect_lidar_tiles",
    "isect_offset_encode",
    "rasterize_to_pixels",
    "rasterize_to_points",
    "spherical_harmonics",
    "quat_scale_to_covar_preci",
    "world_to_cam",
    "persp_proj",
    "lidar_proj",
    "compute_pix_velocity",
    "compute_lidar_velocity",
    "map_points_to_lidar_tiles",
    "points_mapping_offset_encode",
    "populate_image_from_points",
    "rasterize_to_indices_in_range",
    "rasterize_to_indices_in_range_lidar",
    "accumulate",
    "accumulate_lidar",
]
