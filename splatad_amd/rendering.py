"""End-to-end rasterization of 3D Gaussians to camera images and lidar sweeps.

`rasterization()` and `lidar_rasterization()` keep the signatures, defaults, return values and
`meta` keys of the reference's gsplat/rendering.py (:22-440 and :443-819); each stage runs a
hand-written gfx950 kernel through the operators of `splatad_amd.hip._wrapper`.
"""
import math
from typing import Dict, Optional, Tuple, Union

import torch
from torch import Tensor
from typing_extensions import Literal

from ._helper_stream import HelperStream, InPlace
from .hip._wrapper import (
    MIN_OPACITY_PER_TILE,
    fully_fused_lidar_projection,
    fully_fused_projection,
    isect_lidar_tiles,
    isect_offset_encode,
    isect_tiles,
    rasterize_to_pixels,
    rasterize_to_pixels_with_sh,
    rasterize_to_points,
    spherical_harmonics,
    view_dependent_color_cache,
    view_dependent_colors,
)


def _sensor_motion(C, device, linear_velocity, angular_velocity, rolling_shutter_time):
    """Shape checks and zero defaults of the ego-motion arguments (rendering.py:215-226)."""
    if linear_velocity is not None:
        assert linear_velocity.shape == (C, 3), linear_velocity.shape
    else:
        linear_velocity = torch.zeros(C, 3, device=device)
    if angular_velocity is not None:
        assert angular_velocity.shape == (C, 3), angular_velocity.shape
    else:
        angular_velocity = torch.zeros(C, 3, device=device)
    if rolling_shutter_time is not None:
        assert rolling_shutter_time.shape == (C,), rolling_shutter_time.shape
    else:
        rolling_shutter_time = torch.zeros(C, device=device)
    return linear_velocity, angular_velocity, rolling_shutter_time


# Whether rasterization() puts the work that only depends on the projection (colour kernel,
# packed rows, their opacities) on a helper stream beside the tile intersection.  Off: measured
# on the 1M-Gaussian 1080p frame, that work enqueued on the caller's stream behind the sort costs
# the same or 6-9 us less in every mode but one (packed, colours from spherical harmonics and
# gradients wanted: 0.468 against 0.462 ms) -- kernels that share the GPU share its wave slots
# and memory system, and a fork and a join cost 20 us of their own -- and a call then uses one
# stream only.
HELPER_STREAM = False
# rows (sensors x Gaussians) up to which the colour cache is made beside the sort, see rasterization()
CACHE_BESIDE_SORT_ROWS = 1_500_000


class _CameraPlan:
    """What a `rasterization()` call does beyond the fixed stages, decided up front from its
    arguments alone:

    colors            who makes the per-row colours: "given" (post-activation features),
                      "view_kernel" (one kernel: directions, SH, activation, depth channel),
                      "while_compositing" (the compositing kernel evaluates the colours of the
                      entries it stages, and its backward pass takes them from what that left
                      in the colour cache) or "sh_operators" (view matrices that
                      take a gradient: directions and SH by differentiable operators);
    depth_in_colors   the colour maker appends the depth channel itself;
    requests          what a packed projection is asked to make of its rows besides the rows:
                      their opacities, their colours, their colour cache;
    helper_stream     whether that work runs on a helper stream beside the tile intersection.
    """

    def __init__(self, packed, sh_degree, render_mode, tile, means, quats, scales, opacities, colors,
                 velocities, viewmats, backgrounds):
        def wanted(*tensors):  # does any of them take a gradient in this call?
            return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)

        with_depth = render_mode in ("RGB+D", "RGB+ED")
        if sh_degree is None:
            self.colors = "given"
        elif viewmats.requires_grad:
            self.colors = "sh_operators"
        elif (means.is_cuda and render_mode in ("RGB", "RGB+D", "RGB+ED") and colors.dtype == torch.float32
              and opacities.dtype == torch.float32):
            self.colors = "while_compositing"
        else:
            self.colors = "view_kernel"
        self.depth_in_colors = with_depth and self.colors in ("view_kernel", "while_compositing")
        self.helper_stream = HELPER_STREAM and self.colors != "while_compositing"
        self.requests = {}
        if packed:
            if self.colors == "view_kernel" and colors.is_contiguous():
                self.requests["colors"] = (sh_degree, colors, self.depth_in_colors)
            # the gather opacities[gaussian_ids] (* compensations), where no gradient passes through it
            if (not wanted(means, quats, scales, opacities, velocities, viewmats) and opacities.is_contiguous()
                    and opacities.dtype == torch.float32):
                self.requests["opacities"] = opacities
                if self.colors == "while_compositing" and colors.is_contiguous():
                    self.requests["color_cache"] = (sh_degree, colors, self.depth_in_colors, *tile,
                                                    MIN_OPACITY_PER_TILE)


def rasterization(
    means: Tensor,  # [N, 3]
    quats: Tensor,  # [N, 4]
    scales: Tensor,  # [N, 3]
    opacities: Tensor,  # [N]
    colors: Tensor,  # [(C,) N, D] or [(C,) N, K, 3]
    velocities: Optional[Tensor],  # [N, 3]
    viewmats: Tensor,  # [C, 4, 4]
    Ks: Tensor,  # [C, 3, 3]
    width: int,
    height: int,
    linear_velocity: Optional[Tensor] = None,  # [C, 3]
    angular_velocity: Optional[Tensor] = None,  # [C, 3]
    rolling_shutter_time: Optional[Tensor] = None,  # [C]
    near_plane: float = 0.01,
    far_plane: float = 1e10,
    radius_clip: float = 0.0,
    eps2d: float = 0.3,
    sh_degree: Optional[int] = None,
    packed: bool = True,
    tile_size: int = 16,
    backgrounds: Optional[Tensor] = None,
    render_mode: Literal["RGB", "D", "ED", "RGB+D", "RGB+ED"] = "RGB",
    sparse_grad: bool = False,
    absgrad: bool = False,
    rasterize_mode: Literal["classic", "antialiased"] = "classic",
    channel_chunk: int = 32,
) -> Tuple[Tensor, Tensor, Dict]:
    """Renders N Gaussians into C pinhole images.

    `colors` are either post-activation features [(C,) N, D] (`sh_degree=None`) or SH
    coefficients [(C,) N, K, 3] evaluated up to `sh_degree`.  `render_mode` selects colour,
    accumulated depth ("D"), expected depth ("ED") or colour plus depth as the last channel.
    `linear_velocity` (world frame), `angular_velocity` (sensor frame) and
    `rolling_shutter_time` describe the ego motion during the row-wise readout; `velocities`
    are per-Gaussian world velocities.  `packed=True` keeps only visible (camera, Gaussian)
    pairs between the stages; `rasterize_mode="antialiased"` scales opacities by
    sqrt(det(Sigma) / det(Sigma + eps2d I)); `absgrad=True` leaves the accumulated absolute
    image-plane gradients in `meta["means2d"].absgrad` after backward.

    Reproducibility: forward results are the same bits from run to run.  Gradients that add up
    contributions of many pixels (those of the compositing stage) are summed with float atomics,
    so they differ in the last bits between runs; with `packed=True` and more than one camera
    this also holds for the sums over the cameras that see a Gaussian (opacities, colours or SH
    coefficients, projection inputs), which the unpacked call adds in a fixed order.

    Returns (render_colors [C, H, W, X], render_alphas [C, H, W, 1], meta).
    """
    N = means.shape[0]
    C = viewmats.shape[0]
    assert means.shape == (N, 3), means.shape
    assert quats.shape == (N, 4), quats.shape
    assert scales.shape == (N, 3), scales.shape
    assert opacities.shape == (N,), opacities.shape
    if velocities is not None:
        assert velocities.shape == (N, 3), velocities.shape
    assert viewmats.shape == (C, 4, 4), viewmats.shape
    assert Ks.shape == (C, 3, 3), Ks.shape
    linear_velocity, angular_velocity, rolling_shutter_time = _sensor_motion(
        C, means.device, linear_velocity, angular_velocity, rolling_shutter_time
    )
    assert render_mode in ["RGB", "D", "ED", "RGB+D", "RGB+ED"], render_mode

    if sh_degree is None:
        assert (colors.dim() == 2 and colors.shape[0] == N) or (
            colors.dim() == 3 and colors.shape[:2] == (C, N)
        ), colors.shape
    else:
        assert (colors.dim() == 3 and colors.shape[0] == N and colors.shape[2] == 3) or (
            colors.dim() == 4 and colors.shape[:2] == (C, N) and colors.shape[3] == 3
        ), colors.shape
        assert (sh_degree + 1) ** 2 <= colors.shape[-2], colors.shape

    # 1. projection (packed: it also counts the intersections with the tile grid of step 2,
    # so that the host waits for the GPU once per call, not twice, makes the lists of step 2
    # on its dense rows, and is asked for what else only needs the projection: see the plan)
    tile_width = math.ceil(width / float(tile_size))
    tile_height = math.ceil(height / float(tile_size))
    plan = _CameraPlan(packed, sh_degree, render_mode, (tile_size, tile_width, tile_height), means, quats,
                       scales, opacities, colors, velocities, viewmats, backgrounds)
    beside = HelperStream(means.device, plan.requests) if plan.helper_stream else InPlace(plan.requests)
    proj = fully_fused_projection(
        means, None, quats, scales, velocities, viewmats, Ks, width, height, linear_velocity,
        angular_velocity, rolling_shutter_time, eps2d=eps2d, packed=packed, near_plane=near_plane,
        far_plane=far_plane, radius_clip=radius_clip, sparse_grad=sparse_grad,
        calc_compensations=(rasterize_mode == "antialiased"),
        isect_grid=(tile_size, tile_width, tile_height) if packed else None,
        beside=beside if packed else None,
    )
    if packed:
        camera_ids, gaussian_ids, radii, means2d, depths, conics, compensations, pix_vels = proj
    else:
        radii, means2d, depths, conics, compensations, pix_vels = proj
        camera_ids, gaussian_ids = None, None
        beside.refork()  # everything the colours need is enqueued

    # 2. tile intersection, sort, offsets.  (Work beside it is enqueued behind it: the kernel then
    # meets the segment sort; enqueued first, its launch would stand between the host and the
    # launches the GPU is waiting for.)  The colour cache of a call that evaluates its colours
    # while compositing needs the projection only: its two short launches are made from inside
    # the intersection call, on a stream that the sort forks and joins anyway (unpacked calls;
    # a packed projection has made the cache of its rows the same way).  That stream has about
    # 14 us to spare on a frame of a million rows, and clearing the cache takes 9 us per million
    # rows: beyond a million and a half the launches stay behind the sort (measured: 1M rows
    # 0.3675 -> 0.3585 ms beside the sort, 2M 0.639 -> 0.643, 4M 0.966 -> 0.996).
    cache_beside_sort = None
    if (plan.colors == "while_compositing" and not packed and "color_cache" not in beside.results
            and C * N <= CACHE_BESIDE_SORT_ROWS
            and all(t.is_contiguous() for t in (means, viewmats, colors, radii, depths, opacities))):
        made = []
        cache_depths = depths if plan.depth_in_colors else None

        def cache_beside_sort():
            made.append(view_dependent_color_cache(
                sh_degree, means, viewmats, colors, radii, cache_depths, opacities, tile_size, tile_width,
                tile_height, None, None))

    tiles_per_gauss, isect_ids, flatten_ids = isect_tiles(
        means2d, radii, depths, tile_size, tile_width, tile_height, packed=packed, n_cameras=C,
        camera_ids=camera_ids, gaussian_ids=gaussian_ids, beside_work=cache_beside_sort,
    )
    if cache_beside_sort is not None:
        beside.results["color_cache"] = made[0]
    isect_offsets = isect_offset_encode(isect_ids, C, tile_width, tile_height)

    # per-row opacities: [nnz], or [C, N] (a view, copied by the first operator that needs it
    # when C > 1).  (index_select: its backward adds with atomics where that of
    # opacities[gaussian_ids] sorts the indices first, 0.1 ms for a million rows; the sums can
    # differ in the last bit from run to run where a Gaussian is seen by several cameras.)
    opacities_per_gaussian = opacities

    def per_row_opacities():
        # (one sensor: a view whose backward is a view; expand's is a sum, a kernel even over one row)
        o = (opacities_per_gaussian.index_select(0, gaussian_ids) if packed
             else opacities_per_gaussian[None] if C == 1 else opacities_per_gaussian.expand(C, -1))
        return o if compensations is None else o * compensations

    if "opacities" in beside.results:
        opacities = beside.results["opacities"]
    elif packed and not opacities.requires_grad:
        with beside:  # (not for a leaf that takes a gradient: autograd would accumulate it there)
            opacities = per_row_opacities()
    else:
        if packed:
            beside.join()  # the gather reads the packed rows' ids
        opacities = per_row_opacities()

    # 3. per-(camera, Gaussian) colours
    color_cache = None
    depths_for_colors = depths if plan.depth_in_colors else None
    if plan.colors == "view_kernel":
        colors = view_dependent_colors(sh_degree, means, viewmats, colors, radii, depths_for_colors, camera_ids,
                                       gaussian_ids, launch_context=beside,
                                       precomputed=beside.results.get("colors"))
    beside.join(colors, opacities)  # from here on everything is on the caller's stream
    if plan.colors == "while_compositing":
        # the empty cache through which the tiles share the colours they evaluate, or, for a
        # scene whose tiles will not saturate early, all colours after all: what the packed
        # projection made of its rows, or two short launches here
        color_cache = beside.results.get("color_cache")
        if color_cache is None:
            color_cache = view_dependent_color_cache(
                sh_degree, means, viewmats, colors, radii, depths_for_colors, opacities_per_gaussian,
                tile_size, tile_width, tile_height, camera_ids, gaussian_ids)
    elif plan.colors == "given":
        if packed:
            colors = colors.index_select(0, gaussian_ids) if colors.dim() == 2 else colors[camera_ids, gaussian_ids]
        elif colors.dim() == 2:
            colors = colors.expand(C, -1, -1)
    elif plan.colors == "sh_operators":
        camtoworlds = torch.inverse(viewmats)  # [C, 4, 4]
        if packed:
            dirs = means[gaussian_ids, :] - camtoworlds[camera_ids, :3, 3]  # [nnz, 3]
            shs = (colors[gaussian_ids, :, :] if colors.dim() == 3
                   else colors[camera_ids, gaussian_ids, :, :])  # [nnz, K, 3]
        else:
            dirs = means[None, :, :] - camtoworlds[:, None, :3, 3]  # [C, N, 3]
            shs = colors.expand(C, -1, -1, -1) if colors.dim() == 3 else colors  # [C, N, K, 3]
        colors = spherical_harmonics(sh_degree, dirs, shs, masks=radii[..., 0] > 0)
        colors = torch.clamp_min(colors + 0.5, 0.0)

    # 4. channels to composite
    if render_mode in ["RGB+D", "RGB+ED"]:
        if not plan.depth_in_colors:
            colors = torch.cat((colors, depths[..., None]), dim=-1)
        if backgrounds is not None:
            backgrounds = torch.cat(
                [backgrounds, torch.zeros(C, 1, device=backgrounds.device)], dim=-1
            )
    elif render_mode in ["D", "ED"]:
        colors = depths[..., None]
        if backgrounds is not None:
            backgrounds = torch.zeros(C, 1, device=backgrounds.device)

    def composite(cols, bgs):
        return rasterize_to_pixels(
            means2d, conics, cols, opacities, pix_vels, width, height, tile_size, isect_offsets,
            flatten_ids, rolling_shutter_time, backgrounds=bgs, packed=packed, absgrad=absgrad,
        )

    # The reference composites channel_chunk channels per call (rendering.py:362-391), copying
    # a slice of the colours for each; the kernel here takes all channels in one call (in
    # passes of 32 over the same lists), which renders the same images without the copies.
    if plan.colors == "while_compositing":
        render_colors, render_alphas = rasterize_to_pixels_with_sh(
            sh_degree, means, viewmats, colors, depths_for_colors, means2d, conics,
            opacities, pix_vels, width, height, tile_size, isect_offsets, flatten_ids,
            rolling_shutter_time, backgrounds=backgrounds, gaussian_ids=gaussian_ids,
            color_cache=color_cache, radii=radii, camera_ids=camera_ids, absgrad=absgrad)
    else:
        render_colors, render_alphas = composite(colors, backgrounds)

    if render_mode in ["ED", "RGB+ED"]:
        render_colors = torch.cat(
            [render_colors[..., :-1], render_colors[..., -1:] / render_alphas.clamp(min=1e-10)],
            dim=-1,
        )

    meta = {
        "camera_ids": camera_ids,
        "gaussian_ids": gaussian_ids,
        "radii": radii,
        "means2d": means2d,
        "depths": depths,
        "conics": conics,
        "opacities": opacities,
        "pix_vels": pix_vels,
        "tile_width": tile_width,
        "tile_height": tile_height,
        "tiles_per_gauss": tiles_per_gauss,
        "isect_ids": isect_ids,
        "flatten_ids": flatten_ids,
        "isect_offsets": isect_offsets,
        "width": width,
        "height": height,
        "tile_size": tile_size,
        "n_cameras": C,
    }
    return render_colors, render_alphas, meta


def lidar_rasterization(
    means: Tensor,  # [N, 3]
    quats: Tensor,  # [N, 4]
    scales: Tensor,  # [N, 3]
    opacities: Tensor,  # [N]
    lidar_features: Tensor,  # [C, N, D]
    velocities: Optional[Tensor],  # [N, 3]
    viewmats: Tensor,  # [C, 4, 4]
    raster_pts: Tensor,  # [C, H, W, 4]
    tile_elevation_boundaries: Tensor,  # [ceil(n_elevation_channels / tile_height) + 1]
    linear_velocity: Optional[Tensor] = None,  # [C, 3]
    angular_velocity: Optional[Tensor] = None,  # [C, 3]
    rolling_shutter_time: Optional[Tensor] = None,  # [C]
    min_azimuth: float = -180,
    max_azimuth: float = 180,
    min_elevation: float = -80,
    max_elevation: float = 80,
    n_elevation_channels: int = 32,
    azimuth_resolution: float = 0.1,
    tile_width: int = 32,
    tile_height: int = 8,
    near_plane: float = 0.01,
    far_plane: float = 1e10,
    radius_clip: float = 0.0,
    eps2d: float = 0.017,
    compute_alpha_sum_until_points: bool = True,
    compute_alpha_sum_until_points_threshold: float = 0.2,
    packed: bool = False,
    sparse_grad: bool = False,
    absgrad: bool = False,
    rasterize_mode: Literal["classic", "antialiased"] = "classic",
    channel_chunk: int = 32,
    use_depth_compensation: bool = True,
) -> Tuple[Tensor, Tensor, Union[Tensor, None], Dict]:
    """Renders N Gaussians onto the points of C spinning-lidar sweeps.

    `raster_pts[c, i, j] = (azimuth deg, elevation deg, range m, time s)` are the points to
    render, laid out so that rows group into elevation tiles of `tile_height` beams bounded by
    `tile_elevation_boundaries` and columns into azimuth tiles of
    `tile_width * azimuth_resolution` degrees starting at `min_azimuth`; points with range <= 0
    are skipped.  The per-point time shifts every Gaussian along its spherical velocity
    (rolling shutter).  The output has the D features plus the expected range as last channel.
    `alpha_sum_until_points` sums the alphas of Gaussians closer than the point's range minus
    the threshold; `meta["median_depths"]` is the range at which transmittance crosses 0.5.

    Returns (render_lidar_features [C, H, W, D+1], render_alphas [C, H, W, 1],
    alpha_sum_until_points [C, H, W, 1] | None, meta).
    """
    N = means.shape[0]
    C = viewmats.shape[0]
    D = lidar_features.shape[-1]
    assert means.shape == (N, 3), means.shape
    assert quats.shape == (N, 4), quats.shape
    assert scales.shape == (N, 3), scales.shape
    assert opacities.shape == (N,), opacities.shape
    if velocities is not None:
        assert velocities.shape == (N, 3), velocities.shape
    assert viewmats.shape == (C, 4, 4), viewmats.shape
    assert lidar_features.shape == (C, N, D), lidar_features.shape
    assert min_azimuth < max_azimuth, (min_azimuth, max_azimuth)
    assert min_elevation < max_elevation, (min_elevation, max_elevation)
    assert min_azimuth >= -180.0 and max_azimuth <= 180.0, (min_azimuth, max_azimuth)
    # the spherical Jacobian degenerates towards the poles
    assert min_elevation >= -85.0 and max_elevation <= 85.0, (min_elevation, max_elevation)
    assert tile_width * tile_height <= 256, (tile_width, tile_height)
    assert n_elevation_channels > 0, n_elevation_channels
    assert tile_elevation_boundaries.shape == (
        math.ceil(n_elevation_channels / tile_height) + 1,
    ), tile_elevation_boundaries.shape
    assert azimuth_resolution > 0.0, azimuth_resolution
    linear_velocity, angular_velocity, rolling_shutter_time = _sensor_motion(
        C, means.device, linear_velocity, angular_velocity, rolling_shutter_time
    )
    assert raster_pts.shape == (C, *raster_pts.shape[1:]), raster_pts.shape
    assert raster_pts.shape[-1] == 4, raster_pts.shape

    proj = fully_fused_lidar_projection(
        means, None, quats, scales, velocities, viewmats, linear_velocity, angular_velocity,
        rolling_shutter_time, min_elevation=min_elevation, max_elevation=max_elevation,
        min_azimuth=min_azimuth, max_azimuth=max_azimuth, eps2d=eps2d, packed=packed,
        near_plane=near_plane, far_plane=far_plane, radius_clip=radius_clip,
        sparse_grad=sparse_grad, calc_compensations=(rasterize_mode == "antialiased"),
    )
    if packed:
        raise NotImplementedError("Packed mode is not supported for lidar_rasterization")
    radii, means2d, depths, conics, compensations, pix_vels, depth_compensations = proj
    opacities = opacities[None] if C == 1 else opacities.expand(C, -1)  # [C, N], as above
    camera_ids, gaussian_ids = None, None

    if not use_depth_compensation:
        depth_compensations = depth_compensations * 0
    if compensations is not None:
        opacities = opacities * compensations

    n_elevation_tiles = math.ceil(n_elevation_channels / tile_height)
    tile_azimuth_resolution = azimuth_resolution * tile_width
    n_azimuth_tiles = math.ceil((max_azimuth - min_azimuth) / tile_azimuth_resolution)
    # Features to composite.  The reference composites chunks of channel_chunk-1 features plus
    # the range, each a concatenated copy (rendering.py:733-771), because its kernels take 32
    # channels at most; the kernels here take any number of channels in one call (in passes
    # of 32 over the same lists) and read features and ranges where they are, so one call
    # renders what the reference's loop renders: the features its chunks cover -- those beyond
    # n_chunks*(channel_chunk-1) are not rendered, e.g. D=63 with channel_chunk=32 -- then the
    # range, and one median column per chunk (the chunks' medians are equal: they depend on
    # the opacities alone).
    n_chunks = (D + channel_chunk) // channel_chunk if (D + 1) > channel_chunk else 1
    n_feats = min(D, n_chunks * (channel_chunk - 1)) if n_chunks > 1 else D
    tiles_per_gauss, isect_ids, flatten_ids = isect_lidar_tiles(
        means2d, radii, depths, elev_boundaries=tile_elevation_boundaries,
        tile_azim_resolution=tile_azimuth_resolution, min_azim=min_azimuth, packed=packed,
        n_cameras=C, camera_ids=camera_ids, gaussian_ids=gaussian_ids,
    )
    isect_offsets = isect_offset_encode(isect_ids, C, n_azimuth_tiles, n_elevation_tiles)

    image_width = raster_pts.shape[-2]
    image_height = raster_pts.shape[-3]
    if n_feats > 0:
        feats = lidar_features if n_feats == D else lidar_features[..., :n_feats]
        ranges = depths
    else:
        feats, ranges = depths[..., None], None  # the range alone is a one-channel call
    render_lidar_features, render_alphas, alpha_sum_until_points, median_depths = rasterize_to_points(
        means2d, conics, feats, opacities, pix_vels,
        depth_compensations, raster_pts, image_width, image_height, tile_width, tile_height,
        isect_offsets, flatten_ids,
        compute_alpha_sum_until_points=compute_alpha_sum_until_points,
        compute_alpha_sum_until_points_threshold=compute_alpha_sum_until_points_threshold,
        packed=packed, absgrad=absgrad, ranges=ranges,
    )
    if n_chunks > 1:
        median_depths = median_depths.repeat(1, 1, 1, n_chunks)

    meta = {
        "camera_ids": camera_ids,
        "gaussian_ids": gaussian_ids,
        "radii": radii,
        "means2d": means2d,
        "depths": depths,
        "conics": conics,
        "opacities": opacities,
        "pix_vels": pix_vels,
        "tile_grid_width": n_azimuth_tiles,
        "tile_grid_height": n_elevation_tiles,
        "tiles_per_gauss": tiles_per_gauss,
        "isect_ids": isect_ids,
        "flatten_ids": flatten_ids,
        "isect_offsets": isect_offsets,
        "width": image_width,
        "height": image_height,
        "tile_width": tile_width,
        "tile_height": tile_height,
        "n_cameras": C,
        "median_depths": median_depths,
    }
    return render_lidar_features, render_alphas, alpha_sum_until_points, meta
