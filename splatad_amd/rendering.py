"""End-to-end rasterization of 3D Gaussians to camera images and lidar sweeps.

`rasterization()` and `lidar_rasterization()` keep the signatures, defaults, return values and
`meta` keys of the reference's gsplat/rendering.py (:22-440 and :443-819); each stage runs a
hand-written gfx950 kernel through the operators of `splatad_amd.hip._wrapper`.
"""
import math
import threading
from typing import Dict, Optional, Tuple, Union

import torch
from torch import Tensor
from typing_extensions import Literal

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

# one helper stream per (device, host thread): calls from different threads do not wait for one
# another's helper work
_HELPER_STREAMS: Dict[Tuple[int, int], "torch.cuda.Stream"] = {}


class _Beside:
    """Runs the work of `with` blocks on a helper stream, beside what the caller's stream does
    between the creation of the object (the fork) and `join()`.

    The tile intersection ends with a segment sort whose few long workgroups leave most of the
    GPU idle; work that only depends on the projection -- the colours of the Gaussians -- is
    enqueued on a helper stream (default priority) to run meanwhile.  Create the object when
    the inputs of that work are enqueued on the caller's stream: the helper stream waits for
    that point only, not for what the caller's stream is given afterwards.  `join()` makes the
    caller's stream wait for the helper and tells the allocator that the tensors made there
    are used on the caller's stream from now on.  On a CPU device, or while a graph is being
    captured, the blocks simply run in place.
    """

    def __init__(self, device, enabled=True):
        # enabled=False: no helper stream; the blocks run in place, the requests to the packed
        # projection are served on the caller's stream
        self.main = self.side = self.fork = self._ctx = self._waited = None
        # what the packed projection is asked to make on the helper stream, and what it made
        self.requests: Dict[str, object] = {}
        self.results: Dict[str, Tensor] = {}
        if enabled and device.type == "cuda" and not torch.cuda.is_current_stream_capturing():
            idx = device.index if device.index is not None else torch.cuda.current_device()
            key = (idx, threading.get_ident())
            if key not in _HELPER_STREAMS:
                _HELPER_STREAMS[key] = torch.cuda.Stream(device=idx)
            self.main = torch.cuda.current_stream(idx)
            self.side = _HELPER_STREAMS[key]
            self.fork = self.main.record_event()

    def __enter__(self):
        if self.side is not None:
            if self._waited is not self.fork:  # once per fork: the helper stream runs in order
                self.side.wait_event(self.fork)
                self._waited = self.fork
            self._ctx = torch.cuda.stream(self.side)
            self._ctx.__enter__()
        return self

    def __exit__(self, *exc):
        if self._ctx is not None:
            self._ctx.__exit__(*exc)
            self._ctx = None
        return False

    def refork(self):
        """Moves the fork to what the caller's stream holds now."""
        if self.side is not None:
            self.fork = self.main.record_event()

    def join(self, *tensors):
        if self.side is not None:
            self.main.wait_stream(self.side)
            for t in tensors:
                if t is not None:
                    t.record_stream(self.main)


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
    # so that the host waits for the GPU once per call, not twice)
    tile_width = math.ceil(width / float(tile_size))
    tile_height = math.ceil(height / float(tile_size))
    # (packed, in a call that wants gradients: the kernels that write the packed rows go to the
    # helper stream, and with them what else only needs the projection, the colours of step 3 and
    # the rows' opacities; the tile intersection works on the projection's dense rows and does
    # not wait for any of it)
    fused_colors = sh_degree is not None and not viewmats.requires_grad
    depth_appended = fused_colors and render_mode in ["RGB+D", "RGB+ED"]
    # Colours from spherical harmonics and no gradient wanted: the compositing kernel evaluates
    # the colours of the entries it stages itself (step 3 below falls away).
    colors_while_compositing = (
        fused_colors and means.is_cuda and render_mode in ["RGB", "RGB+D", "RGB+ED"]
        and colors.dtype == torch.float32 and opacities.dtype == torch.float32
        and not (torch.is_grad_enabled() and any(
            t is not None and t.requires_grad
            for t in (means, quats, scales, opacities, colors, velocities, viewmats, backgrounds))))
    colors_beside = fused_colors and (packed or not colors_while_compositing)  # step 3 joins the helper stream
    beside = _Beside(means.device, enabled=HELPER_STREAM and not colors_while_compositing)
    if packed:
        if fused_colors and not colors_while_compositing and colors.is_contiguous():
            beside.requests["colors"] = (sh_degree, colors, depth_appended)
        # the gather opacities[gaussian_ids] (* compensations), where no gradient passes through it
        no_grad = not torch.is_grad_enabled() or not any(
            t is not None and t.requires_grad for t in (means, quats, scales, opacities, velocities, viewmats))
        if no_grad and opacities.is_contiguous() and opacities.dtype == torch.float32:
            beside.requests["opacities"] = opacities
            if colors_while_compositing and colors.is_contiguous():
                beside.requests["color_cache"] = (sh_degree, colors, depth_appended, tile_size, tile_width,
                                                  tile_height, MIN_OPACITY_PER_TILE)
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

    opacities_per_gaussian = opacities

    def per_row_opacities():
        # Compositing is the first to need these: [nnz], or [C, N] (a view, copied by the first
        # operator that needs it when C > 1).
        # (index_select: its backward adds with atomics where that of opacities[gaussian_ids]
        # sorts the indices first, 0.1 ms for a million rows; the sums can differ in the last
        # bit from run to run where a Gaussian is seen by several cameras)
        o = opacities.index_select(0, gaussian_ids) if packed else opacities.expand(C, -1)
        return o if compensations is None else o * compensations

    # 2. tile intersection, sort, offsets
    if not packed and not colors_while_compositing:
        beside.refork()  # fork: everything the colours need is enqueued

    def fused_view_colors():
        # one kernel for directions, masks, SH, activation and the depth channel
        return view_dependent_colors(sh_degree, means, viewmats, colors, radii,
                                     depths if depth_appended else None, camera_ids,
                                     gaussian_ids, launch_context=beside,
                                     precomputed=beside.results.get("colors"))

    # The colours run on a helper stream beside the intersection, enqueued behind it: the kernel
    # then meets the segment sort, whose long workgroups leave part of the GPU idle (enqueued
    # first, it would compete with the binning chain that everything else waits for, and its
    # launch would stand between the host and the launches the GPU is waiting for).
    tiles_per_gauss, isect_ids, flatten_ids = isect_tiles(
        means2d, radii, depths, tile_size, tile_width, tile_height, packed=packed, n_cameras=C,
        camera_ids=camera_ids, gaussian_ids=gaussian_ids,
    )
    isect_offsets = isect_offset_encode(isect_ids, C, tile_width, tile_height)
    beside_opacities = packed and not opacities.requires_grad
    if "opacities" in beside.results:
        opacities = beside.results["opacities"]
        if not colors_beside:
            beside.join()
    elif beside_opacities:
        # the gather (and the product with the compensations) goes beside the sort too: on the
        # caller's stream it would stand alone between the sort and the compositing.  (Not for a
        # leaf that takes a gradient: autograd would accumulate it on the helper stream.)
        with beside:
            opacities = per_row_opacities()
        if not colors_beside:
            beside.join(opacities)
    else:
        if packed:
            beside.join()  # the packed rows are written on the helper stream
        opacities = per_row_opacities()

    # 3. per-(camera, Gaussian) colours
    color_cache = None
    if colors_while_compositing:
        # the empty cache through which the tiles share the colours they evaluate, or, for a
        # scene whose tiles will not saturate early, all colours after all (on the caller's
        # stream: two short launches cost less there than a helper stream's fork and join)
        color_cache = beside.results.get("color_cache")  # what the packed projection made of its rows
        if color_cache is None:
            color_cache = view_dependent_color_cache(
                sh_degree, means, viewmats, colors, radii, depths if depth_appended else None,
                opacities_per_gaussian, tile_size, tile_width, tile_height, camera_ids, gaussian_ids)
    elif fused_colors:
        colors = fused_view_colors()
        made_beside = "colors" not in beside.results  # (what the projection made was allocated here)
        beside.join(colors if made_beside else None,
                    opacities if beside_opacities and "opacities" not in beside.results else None)
    elif sh_degree is None:
        if packed:
            colors = colors.index_select(0, gaussian_ids) if colors.dim() == 2 else colors[camera_ids, gaussian_ids]
        elif colors.dim() == 2:
            colors = colors.expand(C, -1, -1)
    else:
        camtoworlds = torch.inverse(viewmats)  # [C, 4, 4]
        masks = radii[..., 0] > 0
        if packed:
            dirs = means[gaussian_ids, :] - camtoworlds[camera_ids, :3, 3]  # [nnz, 3]
            shs = (colors[gaussian_ids, :, :] if colors.dim() == 3
                   else colors[camera_ids, gaussian_ids, :, :])  # [nnz, K, 3]
        else:
            dirs = means[None, :, :] - camtoworlds[:, None, :3, 3]  # [C, N, 3]
            shs = colors.expand(C, -1, -1, -1) if colors.dim() == 3 else colors  # [C, N, K, 3]
        colors = spherical_harmonics(sh_degree, dirs, shs, masks=masks)
        colors = torch.clamp_min(colors + 0.5, 0.0)

    # 4. channels to composite
    if render_mode in ["RGB+D", "RGB+ED"]:
        if not depth_appended and not colors_while_compositing:
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
    if colors_while_compositing:
        render_colors, render_alphas = rasterize_to_pixels_with_sh(
            sh_degree, means, viewmats, colors, depths if depth_appended else None, means2d, conics,
            opacities, pix_vels, width, height, tile_size, isect_offsets, flatten_ids,
            rolling_shutter_time, backgrounds=backgrounds, gaussian_ids=gaussian_ids,
            color_cache=color_cache)
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
    opacities = opacities.expand(C, -1)  # [C, N], as above
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
