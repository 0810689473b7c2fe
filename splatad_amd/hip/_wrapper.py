"""Operator wrappers and autograd glue over the HIP kernels.

Same public names, argument order, defaults and return values as the reference's
gsplat/cuda/_wrapper.py (functions at :17, :230, :390, :533, :606, :680, :811, :951; autograd
classes at :1495-2351), so code written against those operators runs unchanged.  Differences,
all on the permissive side:
  * channel counts are passed to the kernels as they are (no host-side zero padding);
  * rows of culled Gaussians and masked SH rows are zeros instead of uninitialised memory;
  * the fused projections return a gradient for per-Gaussian `velocities` (the reference
    computes it and drops it, gsplat/cuda/csrc/projection.cu:874-877).
"""
import contextlib
from typing import Callable, Optional, Tuple

import torch
from torch import Tensor

MAX_CHANNELS = 513  # same ceiling as the reference (gsplat/cuda/_wrapper.py:878)


def _make_lazy_hip_func(name: str) -> Callable:
    """Late lookup in the op table, so importing this module needs no GPU and no library."""

    def call_hip(*args, **kwargs):
        from ._backend import _C

        return getattr(_C, name)(*args, **kwargs)

    return call_hip


class _NoGradContext:
    """Takes the place of the autograd context when no gradient can be asked for."""

    needs_input_grad = ()

    def save_for_backward(self, *tensors):
        pass

    def mark_non_differentiable(self, *tensors):
        pass

    def set_materialize_grads(self, value):
        pass


def _apply(function, *args):
    """`function.apply(*args)`, or just its forward when gradients are switched off or no
    argument takes one (the bookkeeping of autograd costs as much host time as a kernel launch)."""
    if torch.is_grad_enabled():
        for a in args:
            if isinstance(a, Tensor) and a.requires_grad:
                return function.apply(*args)
    return function.forward(_NoGradContext(), *args)


def _c(t: Optional[Tensor]) -> Optional[Tensor]:
    return None if t is None else t.contiguous()


def _check_gaussians(means, covars, quats, scales, velocities):
    N = means.size(0)
    assert means.size() == (N, 3), means.size()
    if covars is not None:
        assert covars.size() == (N, 6), covars.size()
    else:
        assert quats is not None, "covars or quats is required"
        assert scales is not None, "covars or scales is required"
        assert quats.size() == (N, 4), quats.size()
        assert scales.size() == (N, 3), scales.size()
    if velocities is not None:
        assert velocities.size() == (N, 3), velocities.size()
    return N


def spherical_harmonics(
    degrees_to_use: int,
    dirs: Tensor,  # [..., 3]
    coeffs: Tensor,  # [..., K, 3]
    masks: Optional[Tensor] = None,  # [...]
) -> Tensor:
    """Evaluates real spherical harmonics of degree `degrees_to_use` (0..4) in the directions
    `dirs` (need not be unit length) with coefficients `coeffs`; returns [..., 3].  Rows whose
    mask is False are skipped (zeros)."""
    assert (degrees_to_use + 1) ** 2 <= coeffs.shape[-2], coeffs.shape
    assert dirs.shape[:-1] == coeffs.shape[:-2], (dirs.shape, coeffs.shape)
    assert dirs.shape[-1] == 3, dirs.shape
    assert coeffs.shape[-1] == 3, coeffs.shape
    if masks is not None:
        assert masks.shape == dirs.shape[:-1], masks.shape
        masks = masks.contiguous()
    return _apply(_SphericalHarmonics, degrees_to_use, dirs.contiguous(), coeffs.contiguous(), masks)


def view_dependent_colors(
    degrees_to_use: int,
    means: Tensor,  # [N, 3]
    viewmats: Tensor,  # [C, 4, 4]
    coeffs: Tensor,  # [N, K, 3] or [C, N, K, 3]
    radii: Tensor,  # [C, N, 2] or [nnz, 2], int32
    depths: Optional[Tensor] = None,  # [C, N] or [nnz]
    camera_ids: Optional[Tensor] = None,  # [nnz]
    gaussian_ids: Optional[Tensor] = None,  # [nnz]
    launch_context=None,
    precomputed: Optional[Tensor] = None,
) -> Tensor:
    """Activated view-dependent colours of every (sensor, Gaussian) pair in one kernel:
    max(SH(mean - sensor position) + 1/2, 0) for pairs with a positive projected radius
    (1/2 for the others), with `depths` appended as fourth channel when given.  Same values as
    inverting the view matrices, forming the directions and masks, `spherical_harmonics`,
    the activation and the concatenation (gsplat/rendering.py:325-351 of the reference),
    without materialising any of them.  Differentiable in `means`, `coeffs` and `depths`;
    `viewmats` are treated as constants (rows [A | t], last row (0, 0, 0, 1)).
    `launch_context`, if given, is a context manager entered around the forward kernel launch
    only (e.g. a helper stream); the autograd node, and with it the backward pass, stays on the
    caller's stream.  `precomputed`: the result of this very call, made elsewhere (by the packed
    projection, see `fully_fused_projection`); it is taken instead of running the kernel.

    Returns [C, N, 3 or 4], or [nnz, 3 or 4] for packed input.
    """
    N, C = means.shape[0], viewmats.shape[0]
    packed = radii.dim() == 2
    assert means.shape == (N, 3), means.shape
    assert viewmats.shape == (C, 4, 4), viewmats.shape
    assert coeffs.shape[-1] == 3 and (degrees_to_use + 1) ** 2 <= coeffs.shape[-2], coeffs.shape
    assert coeffs.shape[:-2] in ((N,), (C, N)), coeffs.shape
    if packed:
        assert camera_ids is not None and gaussian_ids is not None
        assert camera_ids.shape == gaussian_ids.shape == radii.shape[:1], radii.shape
        camera_ids, gaussian_ids = camera_ids.contiguous(), gaussian_ids.contiguous()
    else:
        assert radii.shape == (C, N, 2), radii.shape
        camera_ids, gaussian_ids = None, None
    if depths is not None:
        assert depths.shape == radii.shape[:-1], depths.shape
        depths = depths.contiguous()
    return _apply(_ViewColors, degrees_to_use, means.contiguous(), viewmats.contiguous(),
                  coeffs.contiguous(), radii.contiguous(), depths, camera_ids, gaussian_ids,
                  launch_context, precomputed)


def fully_fused_projection(
    means: Tensor,  # [N, 3]
    covars: Optional[Tensor],  # [N, 6] or None
    quats: Optional[Tensor],  # [N, 4] or None
    scales: Optional[Tensor],  # [N, 3] or None
    velocities: Optional[Tensor],  # [N, 3] or None
    viewmats: Tensor,  # [C, 4, 4]
    Ks: Tensor,  # [C, 3, 3]
    width: int,
    height: int,
    linear_velocity: Tensor,  # [C, 3]
    angular_velocity: Tensor,  # [C, 3]
    rolling_shutter_time: Tensor,  # [C]
    eps2d: float = 0.3,
    near_plane: float = 0.01,
    far_plane: float = 1e10,
    radius_clip: float = 0.0,
    packed: bool = False,
    sparse_grad: bool = False,
    calc_compensations: bool = False,
    isect_grid: Optional[Tuple[int, int, int]] = None,
    beside=None,
):
    """Projects Gaussians onto C pinhole image planes (EWA splatting) with rolling-shutter
    pixel velocities.

    `isect_grid` = (tile_size, tile_width, tile_height) (not in the reference; packed only) says
    that `isect_tiles` on that grid follows: the projection, which waits for its row count
    anyway, then counts the tile intersections of the rows it keeps as well, and `isect_tiles`
    on the returned (unmodified) `means2d` and `radii` starts without a wait of its own.
    `beside` (packed with `isect_grid` only, not in the reference): an object with `side` (a
    torch stream or None), `requests` and `results` (dicts).  The kernels that write the packed
    outputs then run on that stream beside the sort of the tile intersection, and the caller
    joins it before anything but `isect_tiles` reads the outputs.  requests["colors"] =
    (degrees_to_use, coeffs, with_depth) and requests["opacities"] = opacities [N] ask for the
    result of `view_dependent_colors` and of opacities[gaussian_ids] (* compensations) on the
    returned rows; they are made on the same stream, without a gradient, and left in `results`.

    Returns, unpacked: (radii int32[C,N,2], means2d[C,N,2], depths[C,N], conics[C,N,3],
    compensations[C,N] | None, pix_vels[C,N,2]); a zero radius marks a culled Gaussian.
    Packed: (camera_ids[nnz], gaussian_ids[nnz], radii[nnz,2], means2d[nnz,2], depths[nnz],
    conics[nnz,3], compensations[nnz] | None, pix_vels[nnz,2]) in (camera, gaussian) order.
    """
    C = viewmats.size(0)
    _check_gaussians(means, covars, quats, scales, velocities)
    assert viewmats.size() == (C, 4, 4), viewmats.size()
    assert Ks.size() == (C, 3, 3), Ks.size()
    assert linear_velocity.size() == (C, 3), linear_velocity.size()
    assert angular_velocity.size() == (C, 3), angular_velocity.size()
    assert rolling_shutter_time.size() == (C,), rolling_shutter_time.size()
    if sparse_grad:
        assert packed, "sparse_grad is only supported when packed is True"
    args = (
        means.contiguous(), _c(covars), _c(quats), _c(scales), _c(velocities),
        viewmats.contiguous(), Ks.contiguous(), width, height, linear_velocity.contiguous(),
        angular_velocity.contiguous(), rolling_shutter_time.contiguous(), eps2d, near_plane,
        far_plane, radius_clip,
    )
    if packed:
        return _apply(_FullyFusedProjectionPacked, *args, sparse_grad, calc_compensations, isect_grid,
                      beside)
    return _apply(_FullyFusedProjection, *args, calc_compensations)


def fully_fused_lidar_projection(
    means: Tensor,  # [N, 3]
    covars: Optional[Tensor],  # [N, 6] or None
    quats: Optional[Tensor],  # [N, 4] or None
    scales: Optional[Tensor],  # [N, 3] or None
    velocities: Optional[Tensor],  # [N, 3] or None
    viewmats: Tensor,  # [C, 4, 4]
    linear_velocity: Tensor,  # [C, 3]
    angular_velocity: Tensor,  # [C, 3]
    rolling_shutter_time: Tensor,  # [C]
    min_elevation: float = -45,
    max_elevation: float = 45,
    min_azimuth: float = -180,
    max_azimuth: float = 180,
    eps2d: float = 0.01,
    near_plane: float = 0.01,
    far_plane: float = 1e10,
    radius_clip: float = 0.0,
    packed: bool = False,
    sparse_grad: bool = False,
    calc_compensations: bool = False,
):
    """Projects Gaussians into the spherical frame (azimuth deg, elevation deg, range) of C
    lidars.

    Returns (radii float[C,N,2] in degrees, means2d[C,N,2] in degrees, depths[C,N] = range,
    conics[C,N,3], compensations[C,N] | None, pix_vels[C,N,3] = (deg/s, deg/s, m/s),
    depth_compensations[C,N,2] = change of range per degree of angular offset).
    Packed mode does not exist for lidars.
    """
    C = viewmats.size(0)
    _check_gaussians(means, covars, quats, scales, velocities)
    assert viewmats.size() == (C, 4, 4), viewmats.size()
    if sparse_grad:
        assert packed, "sparse_grad is only supported when packed is True"
    if packed:
        raise NotImplementedError("FullyFusedLidarProjectionPacked is not implemented yet")
    return _apply(_FullyFusedLidarProjection,
        means.contiguous(), _c(covars), _c(quats), _c(scales), _c(velocities),
        viewmats.contiguous(), min_elevation, max_elevation, min_azimuth, max_azimuth,
        linear_velocity.contiguous(), angular_velocity.contiguous(),
        rolling_shutter_time.contiguous(), eps2d, near_plane, far_plane, radius_clip,
        calc_compensations,
    )


def _check_projected(means2d, radii, depths, packed, n_cameras, camera_ids, gaussian_ids):
    if packed:
        nnz = means2d.size(0)
        assert means2d.shape == (nnz, 2), means2d.size()
        assert radii.shape == (nnz, 2), radii.size()
        assert depths.shape == (nnz,), depths.size()
        assert camera_ids is not None, "camera_ids is required if packed is True"
        assert gaussian_ids is not None, "gaussian_ids is required if packed is True"
        assert n_cameras is not None, "n_cameras is required if packed is True"
        return n_cameras, camera_ids.contiguous(), gaussian_ids.contiguous()
    C, N, _ = means2d.shape
    assert means2d.shape == (C, N, 2), means2d.size()
    assert radii.shape == (C, N, 2), radii.size()
    assert depths.shape == (C, N), depths.size()
    return C, camera_ids, gaussian_ids


@torch.no_grad()
def isect_tiles(
    means2d: Tensor,  # [C, N, 2] or [nnz, 2]
    radii: Tensor,  # [C, N, 2] or [nnz, 2]
    depths: Tensor,  # [C, N] or [nnz]
    tile_size: int,
    tile_width: int,
    tile_height: int,
    sort: bool = True,
    packed: bool = False,
    n_cameras: Optional[int] = None,
    camera_ids: Optional[Tensor] = None,
    gaussian_ids: Optional[Tensor] = None,
    beside_work=None,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Lists the image tiles every projected Gaussian touches.

    Returns (tiles_per_gauss int32[C,N] | [nnz], isect_ids int64[n_isects] with layout
    camera | tile | float bits of depth, flatten_ids int32[n_isects]); sorted by isect id
    (ties in emission order) when `sort`.

    beside_work (not in the reference): a callable without arguments that is called once before
    this returns, where possible from inside the call with the library's launches redirected to
    a stream that runs beside the sort and is joined with it.  It may call operators of this
    package that need only what was enqueued before this call, on contiguous tensors (no torch
    kernel may be launched inside), e.g. `view_dependent_color_cache`.
    """
    C, camera_ids, gaussian_ids = _check_projected(
        means2d, radii, depths, packed, n_cameras, camera_ids, gaussian_ids
    )
    more = {} if beside_work is None else {"beside_work": beside_work}
    return _make_lazy_hip_func("isect_tiles")(
        means2d.contiguous(), radii.contiguous(), depths.contiguous(), camera_ids, gaussian_ids,
        C, tile_size, tile_width, tile_height, sort, True, **more,
    )


@torch.no_grad()
def isect_lidar_tiles(
    means2d: Tensor,  # [C, N, 2] or [nnz, 2]
    radii: Tensor,  # [C, N, 2] or [nnz, 2]
    depths: Tensor,  # [C, N] or [nnz]
    elev_boundaries: Tensor,
    tile_azim_resolution: float,
    min_azim: float,
    sort: bool = True,
    packed: bool = False,
    n_cameras: Optional[int] = None,
    camera_ids: Optional[Tensor] = None,
    gaussian_ids: Optional[Tensor] = None,
) -> Tuple[Tensor, Tensor, Tensor]:
    """Lists the lidar tiles (uniform in azimuth with wrap-around, `elev_boundaries` in
    elevation) every projected Gaussian touches.  Same outputs as :func:`isect_tiles`."""
    C, camera_ids, gaussian_ids = _check_projected(
        means2d, radii, depths, packed, n_cameras, camera_ids, gaussian_ids
    )
    return _make_lazy_hip_func("isect_lidar_tiles")(
        means2d.contiguous(), radii.contiguous(), depths.contiguous(), camera_ids, gaussian_ids,
        C, elev_boundaries.contiguous(), tile_azim_resolution, min_azim, sort, True,
    )


@torch.no_grad()
def isect_offset_encode(isect_ids: Tensor, n_cameras: int, tile_width: int, tile_height: int) -> Tensor:
    """Start of every (camera, tile) segment in the sorted intersection list,
    int32 [C, tile_height, tile_width]."""
    return _make_lazy_hip_func("isect_offset_encode")(
        isect_ids.contiguous(), n_cameras, tile_width, tile_height
    )


@torch.no_grad()
def map_points_to_lidar_tiles(
    points2d: Tensor,  # [C, N, 2] or [nnz, 2]
    elev_boundaries: Tensor,
    tile_azim_resolution: float,
    min_azim: float,
    packed: bool = False,
    n_cameras: Optional[int] = None,
    camera_ids: Optional[Tensor] = None,
    sort: bool = True,
) -> Tuple[Tensor, Tensor]:
    """Tile of every lidar point (no extent), `gsplat/cuda/_wrapper.py:698-757`.

    Returns (tile ids int64 [total]: camera << 32 | tile, flatten ids int32 [total]); with
    `sort` the ids ascend and the points of one tile keep their order."""
    if packed:
        nnz = points2d.size(0)
        assert points2d.shape == (nnz, 2), points2d.size()
        assert camera_ids is not None, "camera_ids is required if packed is True"
        assert n_cameras is not None, "n_cameras is required if packed is True"
        camera_ids = camera_ids.contiguous()
        C = n_cameras
    else:
        C, N, _ = points2d.shape
        assert points2d.shape == (C, N, 2), points2d.size()
    return _make_lazy_hip_func("map_points_to_lidar_tiles")(
        points2d.contiguous(), camera_ids, C, elev_boundaries.contiguous(), tile_azim_resolution,
        min_azim, sort, True)


@torch.no_grad()
def points_mapping_offset_encode(point_ids: Tensor, n_lidars: int, tile_width: int,
                                 tile_height: int) -> Tensor:
    """Offsets [n_lidars, tile_height, tile_width] of sorted point tile ids,
    `gsplat/cuda/_wrapper.py:759-776`."""
    return _make_lazy_hip_func("points_mapping_offset_encode")(
        point_ids.contiguous(), n_lidars, tile_width, tile_height)


@torch.no_grad()
def populate_image_from_points(points: Tensor, image_width: int, image_height: int,
                               tile_width: int, tile_height: int, tile_offsets: Tensor,
                               flatten_id: Tensor) -> Tensor:
    """Image [C, image_height, image_width, 5] whose tiles are filled, in order, with the
    points binned into them (`gsplat/cuda/_wrapper.py:778-809`)."""
    return _make_lazy_hip_func("populate_image_from_points")(
        points.contiguous(), image_width, image_height, tile_width, tile_height,
        tile_offsets.contiguous(), flatten_id.contiguous())


def rasterize_to_pixels(
    means2d: Tensor,  # [C, N, 2] or [nnz, 2]
    conics: Tensor,  # [C, N, 3] or [nnz, 3]
    colors: Tensor,  # [C, N, channels] or [nnz, channels]
    opacities: Tensor,  # [C, N] or [nnz]
    pix_vels: Tensor,  # [C, N, 2] or [nnz, 2]
    image_width: int,
    image_height: int,
    tile_size: int,
    isect_offsets: Tensor,  # [C, tile_height, tile_width]
    flatten_ids: Tensor,  # [n_isects]
    rolling_shutter_time: Optional[Tensor] = None,  # [C]
    backgrounds: Optional[Tensor] = None,  # [C, channels]
    packed: bool = False,
    absgrad: bool = False,
) -> Tuple[Tensor, Tensor]:
    """Front-to-back alpha compositing of the sorted per-tile Gaussian lists onto the pixel
    grid, with a per-row rolling-shutter shift of the Gaussian centres.

    Returns (render_colors[C,H,W,channels], render_alphas[C,H,W,1]).
    """
    C = isect_offsets.size(0)
    device = means2d.device
    if packed:
        nnz = means2d.size(0)
        assert means2d.shape == (nnz, 2), means2d.shape
        assert conics.shape == (nnz, 3), conics.shape
        assert colors.shape[0] == nnz, colors.shape
        assert opacities.shape == (nnz,), opacities.shape
        assert pix_vels.shape == (nnz, 2), pix_vels.shape
    else:
        N = means2d.size(1)
        assert means2d.shape == (C, N, 2), means2d.shape
        assert conics.shape == (C, N, 3), conics.shape
        assert colors.shape[:2] == (C, N), colors.shape
        assert opacities.shape == (C, N), opacities.shape
        assert pix_vels.shape == (C, N, 2), pix_vels.shape
    if rolling_shutter_time is not None:
        assert rolling_shutter_time.shape == (C,), rolling_shutter_time.shape
    else:
        rolling_shutter_time = torch.zeros(C, device=device)
    if backgrounds is not None:
        assert backgrounds.shape == (C, colors.shape[-1]), backgrounds.shape
        backgrounds = backgrounds.contiguous()
    channels = colors.shape[-1]
    if channels > MAX_CHANNELS or channels == 0:
        raise ValueError(f"Unsupported number of color channels: {channels}")
    tile_height, tile_width = isect_offsets.shape[1:3]
    assert tile_height * tile_size >= image_height, f"Assert Failed: {tile_height} * {tile_size} >= {image_height}"
    assert tile_width * tile_size >= image_width, f"Assert Failed: {tile_width} * {tile_size} >= {image_width}"

    return _apply(_RasterizeToPixels,
        means2d.contiguous(), conics.contiguous(), colors.contiguous(), opacities.contiguous(),
        pix_vels.contiguous(), rolling_shutter_time.contiguous(), backgrounds, image_width,
        image_height, tile_size, isect_offsets.contiguous(), flatten_ids.contiguous(), absgrad,
    )


def rasterize_to_pixels_with_sh(
    sh_degree: int,
    means: Tensor,  # [N, 3]
    viewmats: Tensor,  # [C, 4, 4]
    sh_coeffs: Tensor,  # [N, K, 3] or [C, N, K, 3]
    depths: Optional[Tensor],  # [C, N] or [nnz]: rendered as a fourth channel
    means2d: Tensor,  # [C, N, 2] or [nnz, 2]
    conics: Tensor,  # [C, N, 3] or [nnz, 3]
    opacities: Tensor,  # [C, N] or [nnz]
    pix_vels: Tensor,  # [C, N, 2] or [nnz, 2]
    image_width: int,
    image_height: int,
    tile_size: int,
    isect_offsets: Tensor,  # [C, tile_height, tile_width]
    flatten_ids: Tensor,  # [n_isects]
    rolling_shutter_time: Optional[Tensor] = None,  # [C]
    backgrounds: Optional[Tensor] = None,  # [C, 3 or 4]
    gaussian_ids: Optional[Tensor] = None,  # [nnz]: the rows are packed
    color_cache: Optional[Tensor] = None,  # [C, N, 4] or [nnz, 4], from view_dependent_color_cache
    radii: Optional[Tensor] = None,  # [C, N, 2] or [nnz, 2]: needed where a gradient is wanted
    camera_ids: Optional[Tensor] = None,  # [nnz], with gaussian_ids and radii
    absgrad: bool = False,
) -> Tuple[Tensor, Tensor]:
    """`view_dependent_colors` and `rasterize_to_pixels` in one kernel: the compositing kernel
    evaluates the colour of the list entries it stages (the ones tiles reach before they
    saturate) instead of reading colours made for every visible Gaussian beforehand.  Same
    images, bit for bit, as the two operators one after the other.  Differentiable in what the
    two operators are differentiable in (not the view matrices) when `radii` is given: the
    backward pass takes the colours from what the forward pass left in the cache.

    color_cache: where the first tiles to stage a row leave its colour for the others; made by
    `view_dependent_color_cache`, which also decides whether to evaluate all rows beforehand
    after all (scenes whose lists are consumed to their ends).  Without one, the call makes an
    empty cache.  Its contents after the call are of no use.

    Returns (render_colors[C,H,W,3 or 4], render_alphas[C,H,W,1]).
    """
    C = isect_offsets.size(0)
    N = means.size(0)
    rows = (C, N) if gaussian_ids is None else (gaussian_ids.size(0),)
    assert gaussian_ids is None or gaussian_ids.dim() == 1, gaussian_ids.shape
    assert means2d.shape == rows + (2,), means2d.shape
    assert conics.shape == rows + (3,), conics.shape
    assert opacities.shape == rows, opacities.shape
    assert pix_vels.shape == rows + (2,), pix_vels.shape
    assert viewmats.shape == (C, 4, 4), viewmats.shape
    assert sh_coeffs.shape[-1] == 3 and sh_coeffs.shape[:-2] in ((N,), (C, N)), sh_coeffs.shape
    assert (sh_degree + 1) ** 2 <= sh_coeffs.shape[-2], sh_coeffs.shape
    assert depths is None or depths.shape == rows, depths.shape
    channels = 3 if depths is None else 4
    if rolling_shutter_time is not None:
        assert rolling_shutter_time.shape == (C,), rolling_shutter_time.shape
    else:
        rolling_shutter_time = torch.zeros(C, device=means2d.device)
    if backgrounds is not None:
        assert backgrounds.shape == (C, channels), backgrounds.shape
        backgrounds = backgrounds.contiguous()
    tile_height, tile_width = isect_offsets.shape[1:3]
    assert tile_height * tile_size >= image_height, f"Assert Failed: {tile_height} * {tile_size} >= {image_height}"
    assert tile_width * tile_size >= image_width, f"Assert Failed: {tile_width} * {tile_size} >= {image_width}"
    tensors = (means, viewmats, sh_coeffs, depths, means2d, conics, opacities, pix_vels, backgrounds)
    if torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors):
        if viewmats.requires_grad or radii is None:
            raise ValueError("rasterize_to_pixels_with_sh: gradients need `radii` and view matrices "
                             "that take none; use view_dependent_colors and rasterize_to_pixels otherwise")
        assert radii.shape == rows + (2,), radii.shape
        assert (camera_ids is None) == (gaussian_ids is None)
        if color_cache is None:
            color_cache = torch.full(rows + (4,), float("nan"), dtype=torch.float32, device=means2d.device)
        return _RasterizeToPixelsWithSH.apply(
            sh_degree, means.contiguous(), viewmats.contiguous(), sh_coeffs.contiguous(), _c(depths),
            radii.contiguous(), _c(camera_ids), _c(gaussian_ids), means2d.contiguous(), conics.contiguous(),
            opacities.contiguous(), pix_vels.contiguous(), rolling_shutter_time.contiguous(), backgrounds,
            image_width, image_height, tile_size, isect_offsets.contiguous(), flatten_ids.contiguous(),
            color_cache, absgrad)
    render_colors, render_alphas, _ = _make_lazy_hip_func("rasterize_to_pixels_sh_fwd")(
        sh_degree, means.contiguous(), viewmats.contiguous(), sh_coeffs.contiguous(), _c(gaussian_ids),
        _c(depths), means2d.contiguous(), conics.contiguous(), opacities.contiguous(), pix_vels.contiguous(),
        rolling_shutter_time.contiguous(), backgrounds, image_width, image_height, tile_size,
        isect_offsets.contiguous(), flatten_ids.contiguous(), cache=color_cache, want_last_ids=False)
    return render_colors, render_alphas


# Opacity that a tile's list has to carry, by the estimate of view_dependent_color_cache, for the
# colours to be left to the compositing kernel.  Measured on a 1080p frame of 1M Gaussians
# whose opacities were scaled (estimate: colour kernel + compositing / compositing with the
# colours left to it / with all colours put into the cache beforehand, in ms):
# 1399: 0.159 / 0.139 / 0.178; 560: 0.284 / 0.274 / 0.294; 280: 0.445 / 0.456 / 0.453;
# 140: 0.702 / 0.813 / 0.724; 70: 1.173 / 1.444 / 1.193.
MIN_OPACITY_PER_TILE = 200.0


def view_dependent_color_cache(
    degrees_to_use: int,
    means: Tensor,  # [N, 3]
    viewmats: Tensor,  # [C, 4, 4]
    coeffs: Tensor,  # [N, K, 3] or [C, N, K, 3]
    radii: Tensor,  # [C, N, 2] or [nnz, 2], int32
    depths: Optional[Tensor],  # [C, N] or [nnz]: what rasterize_to_pixels_with_sh is given
    opacities: Tensor,  # [N]
    tile_size: int,
    tile_width: int,
    tile_height: int,
    camera_ids: Optional[Tensor] = None,  # [nnz]
    gaussian_ids: Optional[Tensor] = None,  # [nnz]
    min_opacity_per_tile: Optional[float] = None,
) -> Tensor:
    """The colour cache for `rasterize_to_pixels_with_sh` ([C, N, 4] or [nnz, 4]; NaN = colour
    not evaluated yet).  Where the visible Gaussians carry little opacity per tile (their
    opacities times the tiles they meet, summed and divided by the number of tiles, below
    `min_opacity_per_tile`, default MIN_OPACITY_PER_TILE), tiles will not saturate early and
    the colours of all visible rows are evaluated here, as `view_dependent_colors` does."""
    if min_opacity_per_tile is None:
        min_opacity_per_tile = MIN_OPACITY_PER_TILE
    return _make_lazy_hip_func("view_colors_cache")(
        degrees_to_use, means.contiguous(), viewmats.contiguous(), _c(camera_ids), _c(gaussian_ids),
        radii.contiguous(), coeffs.contiguous(), _c(depths), opacities.contiguous(), tile_size, tile_width,
        tile_height, float(min_opacity_per_tile))


def rasterize_to_points(
    means2d: Tensor,  # [C, N, 2] or [nnz, 2]
    conics: Tensor,  # [C, N, 3] or [nnz, 3]
    lidar_features: Tensor,  # [C, N, channels] or [nnz, channels]; last channel = range
    opacities: Tensor,  # [C, N] or [nnz]
    pix_vels: Tensor,  # [C, N, 3] or [nnz, 3]
    depth_compensations: Tensor,  # [C, N, 2] or [nnz, 2]
    raster_pts: Tensor,  # [C, H, W, 4] = (azimuth, elevation, range, time)
    image_width: int,
    image_height: int,
    tile_width: int,
    tile_height: int,
    isect_offsets: Tensor,  # [C, tile_grid_height, tile_grid_width]
    flatten_ids: Tensor,  # [n_isects]
    compute_alpha_sum_until_points: bool,
    compute_alpha_sum_until_points_threshold: float,
    backgrounds: Optional[Tensor] = None,  # [C, channels]
    packed: bool = False,
    absgrad: bool = False,
    ranges: Optional[Tensor] = None,  # [C, N] or [nnz]
) -> Tuple[Tensor, Tensor, Optional[Tensor], Tensor]:
    """Alpha compositing onto a grid of lidar points given in spherical coordinates; the last
    feature channel is the Gaussian's range and receives the depth-compensation and range-rate
    terms.  Points with range <= 0 are skipped (zeros).

    `ranges` (not in the reference) spares the caller the concatenation of features and
    ranges: given it, `lidar_features` holds channels - 1 features per Gaussian and the range
    channel is read from `ranges`; results and gradients are those of the concatenated call.

    Returns (render_features[C,H,W,channels], render_alphas[C,H,W,1],
    alpha_sum_until_points[C,H,W,1] | None, median_depths[C,H,W,1]).
    """
    C = isect_offsets.size(0)
    if packed:
        nnz = means2d.size(0)
        assert means2d.shape == (nnz, 2), means2d.shape
        assert conics.shape == (nnz, 3), conics.shape
        assert lidar_features.shape[0] == nnz, lidar_features.shape
        assert opacities.shape == (nnz,), opacities.shape
        assert pix_vels.shape == (nnz, 3), pix_vels.shape
        assert depth_compensations.shape == (nnz, 2), depth_compensations.shape
        assert ranges is None or ranges.shape == (nnz,), ranges.shape
    else:
        N = means2d.size(1)
        assert means2d.shape == (C, N, 2), means2d.shape
        assert conics.shape == (C, N, 3), conics.shape
        assert lidar_features.shape[:2] == (C, N), lidar_features.shape
        assert opacities.shape == (C, N), opacities.shape
        assert pix_vels.shape == (C, N, 3), pix_vels.shape
        assert depth_compensations.shape == (C, N, 2), depth_compensations.shape
        assert ranges is None or ranges.shape == (C, N), ranges.shape
    channels = lidar_features.shape[-1] + (ranges is not None)
    if backgrounds is not None:
        assert backgrounds.shape == (C, channels), backgrounds.shape
        backgrounds = backgrounds.contiguous()
    depth_channel_idx = channels - 1
    if ranges is not None and channels < 2:
        raise ValueError("ranges needs at least one feature channel beside it")
    if channels > MAX_CHANNELS or channels == 0:
        raise ValueError(f"Unsupported number of lidar_features channels: {channels}")
    tile_grid_height, tile_grid_width = isect_offsets.shape[1:3]
    assert tile_grid_height * tile_height >= image_height, f"Assert Failed: {tile_grid_height} * {tile_height} >= {image_height}"
    assert tile_grid_width * tile_width >= image_width, f"Assert Failed: {tile_grid_width} * {tile_width} >= {image_width}"
    assert raster_pts.shape == (C, image_height, image_width, 4), "raster_pts does not have the correct shape"

    return _apply(_RasterizeToPoints,
        means2d.contiguous(), conics.contiguous(), lidar_features.contiguous(),
        opacities.contiguous(), pix_vels.contiguous(), depth_compensations.contiguous(),
        backgrounds, raster_pts.contiguous(), image_width, image_height, tile_width, tile_height,
        isect_offsets.contiguous(), flatten_ids.contiguous(), compute_alpha_sum_until_points,
        compute_alpha_sum_until_points_threshold, absgrad, depth_channel_idx,
        None if ranges is None else ranges.contiguous(),
    )


@torch.no_grad()
def rasterize_to_indices_in_range(
    range_start: int,
    range_end: int,
    transmittances: Tensor,  # [C, image_height, image_width]
    means2d: Tensor,  # [C, N, 2]
    conics: Tensor,  # [C, N, 3]
    opacities: Tensor,  # [C, N]
    pix_vels: Tensor,  # [C, N, 2]
    image_width: int,
    image_height: int,
    tile_size: int,
    isect_offsets: Tensor,  # [C, tile_height, tile_width]
    flatten_ids: Tensor,  # [n_isects]
    rolling_shutter_time: Optional[Tensor] = None,  # [C]
) -> Tuple[Tensor, Tensor, Tensor]:
    """Lists the (Gaussian, pixel, camera) triples that take part in compositing, for batches
    `[range_start, range_end)` of every tile's depth-sorted list (a batch is tile_size**2
    Gaussians), starting from the transmittance reached so far.  A very large `range_end`
    walks every list to its end in one call.  (Reference: gsplat/cuda/_wrapper.py:1115-1198.)

    Returns (gaussian_ids[M], pixel_ids[M] (row-major), camera_ids[M]), int64; within a pixel
    front to back, pixels in row-major order, camera by camera.
    """
    C, N, _ = means2d.shape
    assert conics.shape == (C, N, 3), conics.shape
    assert opacities.shape == (C, N), opacities.shape
    assert isect_offsets.shape[0] == C, isect_offsets.shape
    assert pix_vels.shape == (C, N, 2), pix_vels.shape
    assert transmittances.shape == (C, image_height, image_width), transmittances.shape
    if rolling_shutter_time is not None:
        assert rolling_shutter_time.shape == (C,), rolling_shutter_time.shape
    else:
        rolling_shutter_time = torch.zeros(C, device=means2d.device)
    tile_height, tile_width = isect_offsets.shape[1:3]
    assert tile_height * tile_size >= image_height, f"Assert Failed: {tile_height} * {tile_size} >= {image_height}"
    assert tile_width * tile_size >= image_width, f"Assert Failed: {tile_width} * {tile_size} >= {image_width}"

    out_gauss_ids, out_indices = _make_lazy_hip_func("rasterize_to_indices_in_range")(
        range_start, range_end, transmittances.contiguous(), means2d.contiguous(),
        conics.contiguous(), opacities.contiguous(), pix_vels.contiguous(),
        rolling_shutter_time.contiguous(), image_width, image_height, tile_size,
        isect_offsets.contiguous(), flatten_ids.contiguous(),
    )
    out_pixel_ids = out_indices % (image_width * image_height)
    out_camera_ids = out_indices // (image_width * image_height)
    return out_gauss_ids, out_pixel_ids, out_camera_ids


@torch.no_grad()
def rasterize_to_indices_in_range_lidar(
    range_start: int,
    range_end: int,
    transmittances: Tensor,  # [C, image_height, image_width]
    means2d: Tensor,  # [C, N, 2]
    conics: Tensor,  # [C, N, 3]
    opacities: Tensor,  # [C, N]
    pix_vels: Tensor,  # [C, N, 3]
    raster_pts: Tensor,  # [C, image_height, image_width, 4]
    image_width: int,
    image_height: int,
    tile_width: int,
    tile_height: int,
    isect_offsets: Tensor,  # [C, tile_grid_height, tile_grid_width]
    flatten_ids: Tensor,  # [n_isects]
) -> Tuple[Tensor, Tensor, Tensor]:
    """`rasterize_to_indices_in_range` for lidar points given as (azimuth, elevation, range,
    time); a batch is tile_width * tile_height Gaussians and points with range <= 0 take
    nothing.  (Reference: gsplat/cuda/_wrapper.py:1200-1281.)
    """
    C, N, _ = means2d.shape
    assert conics.shape == (C, N, 3), conics.shape
    assert opacities.shape == (C, N), opacities.shape
    assert isect_offsets.shape[0] == C, isect_offsets.shape
    assert pix_vels.shape == (C, N, 3), pix_vels.shape
    assert transmittances.shape == (C, image_height, image_width), transmittances.shape
    assert raster_pts.shape == (C, image_height, image_width, 4), raster_pts.shape
    tile_grid_height, tile_grid_width = isect_offsets.shape[1:3]
    assert tile_grid_height * tile_height >= image_height, f"Assert Failed: {tile_grid_height} * {tile_height} >= {image_height}"
    assert tile_grid_width * tile_width >= image_width, f"Assert Failed: {tile_grid_width} * {tile_width} >= {image_width}"

    out_gauss_ids, out_indices = _make_lazy_hip_func("rasterize_to_indices_in_range_lidar")(
        range_start, range_end, transmittances.contiguous(), means2d.contiguous(),
        conics.contiguous(), opacities.contiguous(), pix_vels.contiguous(),
        raster_pts.contiguous(), image_width, image_height, tile_width, tile_height,
        isect_offsets.contiguous(), flatten_ids.contiguous(),
    )
    out_pixel_ids = out_indices % (image_width * image_height)
    out_camera_ids = out_indices // (image_width * image_height)
    return out_gauss_ids, out_pixel_ids, out_camera_ids


# ---------------------------------------------------------------------------------------------
# autograd pairing of the forward and backward kernels
# ---------------------------------------------------------------------------------------------
def _gate(grads, needs):
    return tuple(g if n else None for g, n in zip(grads, needs))


def _given(v: Optional[Tensor], like: Tensor, *last) -> Tensor:
    """The incoming gradient, contiguous, or zeros of shape like.shape[:-1] + last where autograd
    has none.  (The projections switch off autograd's own zero-filling of absent gradients: it
    would also clear a tensor for the integer radii on every backward pass.)"""
    return torch.zeros(like.shape[:-1] + last, dtype=torch.float32, device=like.device) if v is None else v.contiguous()


class _FullyFusedProjection(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means, covars, quats, scales, velocities, viewmats, Ks, width, height,
                linear_velocity, angular_velocity, rolling_shutter_time, eps2d, near_plane,
                far_plane, radius_clip, calc_compensations):
        radii, means2d, depths, conics, compensations, pix_vels = _make_lazy_hip_func(
            "fully_fused_projection_fwd"
        )(means, covars, quats, scales, velocities, viewmats, Ks, width, height, linear_velocity,
          angular_velocity, rolling_shutter_time, eps2d, near_plane, far_plane, radius_clip,
          calc_compensations)
        if not calc_compensations:
            compensations = None
        ctx.save_for_backward(means, covars, quats, scales, velocities, viewmats, Ks,
                              linear_velocity, angular_velocity, rolling_shutter_time, radii,
                              conics, compensations)
        ctx.width, ctx.height, ctx.eps2d = width, height, eps2d
        ctx.mark_non_differentiable(radii)
        ctx.set_materialize_grads(False)
        return radii, means2d, depths, conics, compensations, pix_vels

    @staticmethod
    def backward(ctx, v_radii, v_means2d, v_depths, v_conics, v_compensations, v_pix_vels):
        (means, covars, quats, scales, velocities, viewmats, Ks, linear_velocity,
         angular_velocity, rolling_shutter_time, radii, conics, compensations) = ctx.saved_tensors
        want_vel = velocities is not None and ctx.needs_input_grad[4]
        out = _make_lazy_hip_func("fully_fused_projection_bwd")(
            means, covars, quats, scales, velocities, viewmats, Ks, ctx.width, ctx.height,
            linear_velocity, angular_velocity, rolling_shutter_time, ctx.eps2d, radii, conics,
            compensations, _given(v_means2d, conics, 2), _given(v_depths, conics), _given(v_conics, conics, 3),
            _c(v_compensations), _given(v_pix_vels, conics, 2), ctx.needs_input_grad[5], want_vel)
        v_means, v_covars, v_quats, v_scales, v_viewmats = out[:5]
        v_velocities = out[5] if want_vel else None
        grads = _gate((v_means, v_covars, v_quats, v_scales, v_velocities, v_viewmats),
                      ctx.needs_input_grad[:6])
        return grads + (None,) * 11


class _FullyFusedLidarProjection(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means, covars, quats, scales, velocities, viewmats, min_elevation,
                max_elevation, min_azimuth, max_azimuth, linear_velocity, angular_velocity,
                rolling_shutter_time, eps2d, near_plane, far_plane, radius_clip,
                calc_compensations):
        (radii, means2d, depths, conics, compensations, pix_vels,
         depth_compensations) = _make_lazy_hip_func("fully_fused_lidar_projection_fwd")(
            means, covars, quats, scales, velocities, viewmats, min_elevation, max_elevation,
            min_azimuth, max_azimuth, linear_velocity, angular_velocity, rolling_shutter_time,
            eps2d, near_plane, far_plane, radius_clip, calc_compensations)
        if not calc_compensations:
            compensations = None
        ctx.save_for_backward(means, covars, quats, scales, velocities, viewmats,
                              linear_velocity, angular_velocity, rolling_shutter_time, radii,
                              conics, compensations)
        ctx.bounds = (min_elevation, max_elevation, min_azimuth, max_azimuth)
        ctx.eps2d = eps2d
        ctx.mark_non_differentiable(radii)
        ctx.set_materialize_grads(False)
        return radii, means2d, depths, conics, compensations, pix_vels, depth_compensations

    @staticmethod
    def backward(ctx, v_radii, v_means2d, v_depths, v_conics, v_compensations, v_pix_vels,
                 v_depth_compensations):
        (means, covars, quats, scales, velocities, viewmats, linear_velocity, angular_velocity,
         rolling_shutter_time, radii, conics, compensations) = ctx.saved_tensors
        want_vel = velocities is not None and ctx.needs_input_grad[4]
        out = _make_lazy_hip_func("fully_fused_lidar_projection_bwd")(
            means, covars, quats, scales, velocities, viewmats, *ctx.bounds, linear_velocity,
            angular_velocity, rolling_shutter_time, ctx.eps2d, radii, conics, compensations,
            _given(v_means2d, conics, 2), _given(v_depths, conics), _given(v_conics, conics, 3),
            _c(v_compensations), _given(v_pix_vels, conics, 3), _given(v_depth_compensations, conics, 2),
            ctx.needs_input_grad[5], want_vel)
        v_means, v_covars, v_quats, v_scales, v_viewmats = out[:5]
        v_velocities = out[5] if want_vel else None
        grads = _gate((v_means, v_covars, v_quats, v_scales, v_velocities, v_viewmats),
                      ctx.needs_input_grad[:6])
        return grads + (None,) * 12


class _FullyFusedProjectionPacked(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means, covars, quats, scales, velocities, viewmats, Ks, width, height,
                linear_velocity, angular_velocity, rolling_shutter_time, eps2d, near_plane,
                far_plane, radius_clip, sparse_grad, calc_compensations, isect_grid=None,
                beside=None):
        (indptr, camera_ids, gaussian_ids, radii, means2d, depths, conics, compensations,
         pix_vels) = _make_lazy_hip_func("fully_fused_projection_packed_fwd")(
            means, covars, quats, scales, velocities, viewmats, Ks, width, height,
            linear_velocity, angular_velocity, rolling_shutter_time, eps2d, near_plane, far_plane,
            radius_clip, calc_compensations, isect_grid, beside)
        if not calc_compensations:
            compensations = None
        ctx.save_for_backward(camera_ids, gaussian_ids, means, covars, quats, scales, velocities,
                              viewmats, Ks, linear_velocity, angular_velocity,
                              rolling_shutter_time, conics, compensations, pix_vels)
        ctx.width, ctx.height, ctx.eps2d, ctx.sparse_grad = width, height, eps2d, sparse_grad
        ctx.mark_non_differentiable(camera_ids, gaussian_ids, radii)
        ctx.set_materialize_grads(False)
        return camera_ids, gaussian_ids, radii, means2d, depths, conics, compensations, pix_vels

    @staticmethod
    def backward(ctx, v_camera_ids, v_gaussian_ids, v_radii, v_means2d, v_depths, v_conics,
                 v_compensations, v_pix_vels):
        (camera_ids, gaussian_ids, means, covars, quats, scales, velocities, viewmats, Ks,
         linear_velocity, angular_velocity, rolling_shutter_time, conics, compensations,
         pix_vels) = ctx.saved_tensors
        sparse_grad = ctx.sparse_grad
        want_vel = velocities is not None and ctx.needs_input_grad[4]
        out = _make_lazy_hip_func("fully_fused_projection_packed_bwd")(
            means, covars, quats, scales, velocities, viewmats, Ks, ctx.width, ctx.height,
            linear_velocity, angular_velocity, rolling_shutter_time, ctx.eps2d, camera_ids,
            gaussian_ids, conics, compensations, pix_vels, _given(v_means2d, conics, 2),
            _given(v_depths, conics), _given(v_conics, conics, 3), _c(v_compensations),
            _given(v_pix_vels, conics, 2), ctx.needs_input_grad[5], sparse_grad, want_vel)
        v_means, v_covars, v_quats, v_scales, v_viewmats = out[:5]
        v_velocities = out[5] if want_vel else None

        def coo(values, like):
            # rows of `values` belong to gaussian_ids; duplicates (several cameras) are summed
            # by the sparse tensor's consumer
            return torch.sparse_coo_tensor(indices=gaussian_ids[None], values=values, size=like.size())

        if sparse_grad:
            if ctx.needs_input_grad[0]:
                v_means = coo(v_means, means)
            if covars is not None and ctx.needs_input_grad[1]:
                v_covars = coo(v_covars, covars)
            if quats is not None and ctx.needs_input_grad[2]:
                v_quats = coo(v_quats, quats)
            if scales is not None and ctx.needs_input_grad[3]:
                v_scales = coo(v_scales, scales)
        grads = _gate((v_means, v_covars, v_quats, v_scales, v_velocities, v_viewmats),
                      ctx.needs_input_grad[:6])
        return grads + (None,) * 14


class _RasterizeToPixels(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means2d, conics, colors, opacities, pix_vels, rolling_shutter_time,
                backgrounds, width, height, tile_size, isect_offsets, flatten_ids, absgrad):
        render_colors, render_alphas, last_ids = _make_lazy_hip_func("rasterize_to_pixels_fwd")(
            means2d, conics, colors, opacities, pix_vels, rolling_shutter_time, backgrounds, width,
            height, tile_size, isect_offsets, flatten_ids)
        ctx.save_for_backward(means2d, conics, colors, opacities, pix_vels, rolling_shutter_time,
                              backgrounds, isect_offsets, flatten_ids, render_alphas, last_ids)
        ctx.width, ctx.height, ctx.tile_size, ctx.absgrad = width, height, tile_size, absgrad
        return render_colors, render_alphas.float()

    @staticmethod
    def backward(ctx, v_render_colors, v_render_alphas):
        (means2d, conics, colors, opacities, pix_vels, rolling_shutter_time, backgrounds,
         isect_offsets, flatten_ids, render_alphas, last_ids) = ctx.saved_tensors
        (v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities,
         v_pix_vels) = _make_lazy_hip_func("rasterize_to_pixels_bwd")(
            means2d, conics, colors, opacities, pix_vels, rolling_shutter_time, backgrounds,
            ctx.width, ctx.height, ctx.tile_size, isect_offsets, flatten_ids, render_alphas,
            last_ids, v_render_colors.contiguous(), v_render_alphas.contiguous(), ctx.absgrad)
        if ctx.absgrad:
            means2d.absgrad = v_means2d_abs
        v_backgrounds = None
        if ctx.needs_input_grad[6]:
            v_backgrounds = (v_render_colors * (1.0 - render_alphas).float()).sum(dim=(1, 2))
        return (v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, None, v_backgrounds,
                None, None, None, None, None, None)


class _RasterizeToPoints(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means2d, conics, colors, opacities, pix_vels, depth_compensations,
                backgrounds, raster_pts, width, height, tile_width, tile_height, isect_offsets,
                flatten_ids, compute_alpha_sum_until_points,
                compute_alpha_sum_until_points_threshold, absgrad, depth_channel_idx,
                ranges=None):
        (render_colors, render_alphas, last_ids, alpha_sum_until_points,
         median_depths) = _make_lazy_hip_func("rasterize_to_points_fwd")(
            means2d, conics, colors, opacities, pix_vels, depth_compensations, backgrounds,
            raster_pts, width, height, tile_width, tile_height, compute_alpha_sum_until_points,
            compute_alpha_sum_until_points_threshold, isect_offsets, flatten_ids,
            depth_channel_idx, range_channel=ranges)
        ctx.save_for_backward(means2d, conics, colors, opacities, pix_vels, depth_compensations,
                              backgrounds, raster_pts, isect_offsets, flatten_ids, render_alphas,
                              last_ids, ranges)
        ctx.geom = (width, height, tile_width, tile_height)
        ctx.absgrad = absgrad
        ctx.alpha_sum = (compute_alpha_sum_until_points, compute_alpha_sum_until_points_threshold)
        ctx.depth_channel_idx = depth_channel_idx
        ctx.mark_non_differentiable(median_depths)
        alpha_sum_until_points = (
            alpha_sum_until_points.float() if compute_alpha_sum_until_points else None
        )
        return render_colors, render_alphas.float(), alpha_sum_until_points, median_depths

    @staticmethod
    def backward(ctx, v_render_colors, v_render_alphas, v_alpha_sum_until_points, v_median_depths):
        (means2d, conics, colors, opacities, pix_vels, depth_compensations, backgrounds,
         raster_pts, isect_offsets, flatten_ids, render_alphas, last_ids,
         ranges) = ctx.saved_tensors
        compute_sum, threshold = ctx.alpha_sum
        if compute_sum and v_alpha_sum_until_points is not None:
            v_sum = v_alpha_sum_until_points.contiguous()
        else:
            v_sum = torch.zeros_like(v_render_alphas)
        grads = _make_lazy_hip_func("rasterize_to_points_bwd")(
            means2d, conics, colors, opacities, pix_vels, depth_compensations, backgrounds,
            raster_pts, *ctx.geom, isect_offsets, flatten_ids, render_alphas, last_ids,
            v_render_colors.contiguous(), v_render_alphas.contiguous(), v_sum, ctx.absgrad,
            compute_sum, threshold, ctx.depth_channel_idx, range_channel=ranges)
        (v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities, v_pix_vels,
         v_depth_compensations) = grads[:7]
        v_ranges = grads[7] if ranges is not None else None
        if ctx.absgrad:
            means2d.absgrad = v_means2d_abs
        v_backgrounds = None
        if ctx.needs_input_grad[6]:
            v_backgrounds = (v_render_colors * (1.0 - render_alphas).float()).sum(dim=(1, 2))
        return (v_means2d, v_conics, v_colors, v_opacities, v_pix_vels, v_depth_compensations,
                v_backgrounds) + (None,) * 11 + (v_ranges,)


# ---------------------------------------------------------------------------
# the unfused projection operators (gsplat/cuda/_wrapper.py:46-228, 1283-1493)
# ---------------------------------------------------------------------------
def quat_scale_to_covar_preci(
    quats: Tensor,  # [N, 4]
    scales: Tensor,  # [N, 3]
    compute_covar: bool = True,
    compute_preci: bool = True,
    triu: bool = False,
) -> Tuple[Optional[Tensor], Optional[Tensor]]:
    """Covariances R S S R^T and precisions R S^-1 S^-1 R^T of (unnormalised) quaternions and
    scales, [N, 3, 3] each or upper triangles [N, 6] with `triu`; a matrix that is not asked
    for is None."""
    assert quats.dim() == 2 and quats.size(1) == 4, quats.size()
    assert scales.dim() == 2 and scales.size(1) == 3, scales.size()
    covars, precis = _apply(_QuatScaleToCovarPreci,
        quats.contiguous(), scales.contiguous(), compute_covar, compute_preci, triu)
    return covars if compute_covar else None, precis if compute_preci else None


def persp_proj(means: Tensor, covars: Tensor, Ks: Tensor, width: int, height: int) -> Tuple[Tensor, Tensor]:
    """Pinhole projection of sensor-frame means [C, N, 3] and covariances [C, N, 3, 3]:
    means2d [C, N, 2] and covars2d [C, N, 2, 2]."""
    C, N, _ = means.shape
    assert means.shape == (C, N, 3), means.size()
    assert covars.shape == (C, N, 3, 3), covars.size()
    assert Ks.shape == (C, 3, 3), Ks.size()
    return _apply(_PerspProj, means.contiguous(), covars.contiguous(), Ks.contiguous(), width, height)


def compute_pix_velocity(p_view: Tensor, lin_vel: Tensor, ang_vel: Tensor, velocities: Tensor,
                         Ks: Tensor, width: int, height: int) -> Tensor:
    """Image-space velocity [C, N, 2] of sensor-frame points [C, N, 3] moving with
    `velocities` [C, N, 3] while the camera moves with `lin_vel`, `ang_vel` [C, 3]."""
    C, N, _ = p_view.shape
    assert p_view.shape == (C, N, 3), p_view.size()
    assert lin_vel.shape == (C, 3), lin_vel.size()
    assert ang_vel.shape == (C, 3), ang_vel.size()
    assert velocities.shape == (C, N, 3), velocities.size()
    assert Ks.shape == (C, 3, 3), Ks.size()
    return _apply(_ComputePixVelocity, p_view.contiguous(), lin_vel.contiguous(), ang_vel.contiguous(),
                                     velocities.contiguous(), Ks.contiguous(), width, height)


def world_to_cam(means: Tensor, covars: Tensor, viewmats: Tensor) -> Tuple[Tensor, Tensor]:
    """World-frame means [N, 3] and covariances [N, 3, 3] in the frames of C sensors:
    [C, N, 3] and [C, N, 3, 3]."""
    C = viewmats.size(0)
    N = means.size(0)
    assert means.size() == (N, 3), means.size()
    assert covars.size() == (N, 3, 3), covars.size()
    assert viewmats.size() == (C, 4, 4), viewmats.size()
    return _apply(_WorldToCam, means.contiguous(), covars.contiguous(), viewmats.contiguous())


def lidar_proj(means: Tensor, covars: Tensor, eps2d: float) -> Tuple[Tensor, Tensor, Tensor]:
    """Spherical projection of sensor-frame Gaussians: means2d (azimuth, elevation above the
    xy-plane, degrees) [C, N, 2], covars2d [C, N, 2, 2], depth compensations [C, N, 2]."""
    C, N, _ = means.shape
    assert means.shape == (C, N, 3), means.size()
    assert covars.shape == (C, N, 3, 3), covars.size()
    return _apply(_LidarProj, means.contiguous(), covars.contiguous(), eps2d)


def compute_lidar_velocity(p_view: Tensor, lin_vel: Tensor, ang_vel: Tensor, velocities: Tensor) -> Tensor:
    """Spherical velocity (azimuth rate, elevation rate, range rate) [C, N, 3] of sensor-frame
    points under sensor motion."""
    C, N, _ = p_view.shape
    assert p_view.shape == (C, N, 3), p_view.size()
    assert lin_vel.shape == (C, 3), lin_vel.size()
    assert ang_vel.shape == (C, 3), ang_vel.size()
    assert velocities.shape == (C, N, 3), velocities.size()
    return _apply(_ComputeLidarVelocity, p_view.contiguous(), lin_vel.contiguous(), ang_vel.contiguous(),
                                       velocities.contiguous())


class _QuatScaleToCovarPreci(torch.autograd.Function):
    @staticmethod
    def forward(ctx, quats, scales, compute_covar=True, compute_preci=True, triu=False):
        covars, precis = _make_lazy_hip_func("quat_scale_to_covar_preci_fwd")(
            quats, scales, compute_covar, compute_preci, triu)
        ctx.save_for_backward(quats, scales)
        ctx.compute_covar, ctx.compute_preci, ctx.triu = compute_covar, compute_preci, triu
        return covars, precis

    @staticmethod
    def backward(ctx, v_covars, v_precis):
        quats, scales = ctx.saved_tensors
        if ctx.compute_covar and v_covars is not None and v_covars.is_sparse:
            v_covars = v_covars.to_dense()
        if ctx.compute_preci and v_precis is not None and v_precis.is_sparse:
            v_precis = v_precis.to_dense()
        v_quats, v_scales = _make_lazy_hip_func("quat_scale_to_covar_preci_bwd")(
            quats, scales,
            v_covars.contiguous() if ctx.compute_covar and v_covars is not None else None,
            v_precis.contiguous() if ctx.compute_preci and v_precis is not None else None, ctx.triu)
        return v_quats, v_scales, None, None, None


class _PerspProj(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means, covars, Ks, width, height):
        means2d, covars2d = _make_lazy_hip_func("persp_proj_fwd")(means, covars, Ks, width, height)
        ctx.save_for_backward(means, covars, Ks)
        ctx.width, ctx.height = width, height
        return means2d, covars2d

    @staticmethod
    def backward(ctx, v_means2d, v_covars2d):
        means, covars, Ks = ctx.saved_tensors
        v_means, v_covars = _make_lazy_hip_func("persp_proj_bwd")(
            means, covars, Ks, ctx.width, ctx.height, v_means2d.contiguous(), v_covars2d.contiguous())
        return v_means, v_covars, None, None, None


class _ComputePixVelocity(torch.autograd.Function):
    @staticmethod
    def forward(ctx, p_view, lin_vel, ang_vel, velocities, Ks, width, height):
        vel = _make_lazy_hip_func("compute_pix_velocity_fwd")(p_view, lin_vel, ang_vel, velocities, Ks,
                                                              width, height)
        ctx.save_for_backward(p_view, lin_vel, ang_vel, velocities, Ks)
        ctx.width, ctx.height = width, height
        return vel

    @staticmethod
    def backward(ctx, v_vel):
        p_view, lin_vel, ang_vel, velocities, Ks = ctx.saved_tensors
        v_p_view, v_velocities = _make_lazy_hip_func("compute_pix_velocity_bwd")(
            p_view, lin_vel, ang_vel, velocities, Ks, ctx.width, ctx.height, v_vel.contiguous())
        return v_p_view, None, None, v_velocities, None, None, None


class _WorldToCam(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means, covars, viewmats):
        means_c, covars_c = _make_lazy_hip_func("world_to_cam_fwd")(means, covars, viewmats)
        ctx.save_for_backward(means, covars, viewmats)
        return means_c, covars_c

    @staticmethod
    def backward(ctx, v_means_c, v_covars_c):
        means, covars, viewmats = ctx.saved_tensors
        return _make_lazy_hip_func("world_to_cam_bwd")(
            means, covars, viewmats, v_means_c.contiguous(), v_covars_c.contiguous(),
            ctx.needs_input_grad[0], ctx.needs_input_grad[1], ctx.needs_input_grad[2])


class _LidarProj(torch.autograd.Function):
    @staticmethod
    def forward(ctx, means, covars, eps2d):
        means2d, covars2d, depth_compensations = _make_lazy_hip_func("lidar_proj_fwd")(means, covars, eps2d)
        ctx.save_for_backward(means, covars)
        ctx.eps2d = eps2d
        return means2d, covars2d, depth_compensations

    @staticmethod
    def backward(ctx, v_means2d, v_covars2d, v_depth_compensations):
        means, covars = ctx.saved_tensors
        v_means, v_covars = _make_lazy_hip_func("lidar_proj_bwd")(
            means, covars, ctx.eps2d, v_means2d.contiguous(), v_covars2d.contiguous(),
            v_depth_compensations.contiguous())
        return v_means, v_covars, None


class _ComputeLidarVelocity(torch.autograd.Function):
    @staticmethod
    def forward(ctx, p_view, lin_vel, ang_vel, velocities):
        vel = _make_lazy_hip_func("compute_lidar_velocity_fwd")(p_view, lin_vel, ang_vel, velocities)
        ctx.save_for_backward(p_view, lin_vel, ang_vel, velocities)
        return vel

    @staticmethod
    def backward(ctx, v_vel):
        p_view, lin_vel, ang_vel, velocities = ctx.saved_tensors
        v_p_view, v_velocities = _make_lazy_hip_func("compute_lidar_velocity_bwd")(
            p_view, lin_vel, ang_vel, velocities, v_vel.contiguous())
        return v_p_view, None, None, v_velocities


class _ViewColors(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sh_degree, means, viewmats, coeffs, radii, depths, camera_ids, gaussian_ids,
                launch_context, precomputed=None):
        if precomputed is not None:
            assert precomputed.shape == radii.shape[:-1] + (4 if depths is not None else 3,), precomputed.shape
            colors = precomputed
        else:
            with (launch_context if launch_context is not None else contextlib.nullcontext()):
                colors = _make_lazy_hip_func("view_colors_fwd")(
                    sh_degree, means, viewmats, camera_ids, gaussian_ids, radii, coeffs, depths)
        ctx.save_for_backward(means, viewmats, coeffs, radii, camera_ids, gaussian_ids, colors)
        ctx.sh_degree = sh_degree
        ctx.has_depths = depths is not None
        return colors

    @staticmethod
    def backward(ctx, v_colors):
        means, viewmats, coeffs, radii, camera_ids, gaussian_ids, colors = ctx.saved_tensors
        v_means, v_coeffs = _view_colors_backward(
            ctx.sh_degree, means, viewmats, coeffs, radii, camera_ids, gaussian_ids, colors, v_colors,
            ctx.needs_input_grad[1], ctx.needs_input_grad[3])
        v_depths = v_colors[..., 3] if ctx.has_depths and ctx.needs_input_grad[5] else None
        return None, v_means, None, v_coeffs, None, v_depths, None, None, None, None


def _view_colors_backward(sh_degree, means, viewmats, coeffs, radii, camera_ids, gaussian_ids, colors,
                          v_colors, need_means, need_coeffs):
    """Gradients of the view-dependent colours with respect to the means and the coefficients,
    summed over the sensors that see a Gaussian; (None, None) where neither is wanted."""
    v_means = v_coeffs = None
    if need_means or need_coeffs:
        # rows of one Gaussian seen by several sensors add up; for packed rows the kernel adds
        # the coefficient gradients at their Gaussians itself (one pass over them instead of
        # a [nnz, K, 3] tensor and an index_add_ over it)
        packed = camera_ids is not None
        scatter = packed and need_coeffs
        v_rows, v_dirs = _make_lazy_hip_func("view_colors_bwd")(
            sh_degree, means, viewmats, camera_ids, gaussian_ids, radii, coeffs, colors,
            v_colors.contiguous(), need_means, scatter)
        if need_coeffs:
            if scatter:
                v_coeffs = v_rows
            elif coeffs.dim() == 4:
                v_coeffs = (torch.zeros_like(coeffs).index_put_((camera_ids, gaussian_ids), v_rows, accumulate=True)
                            if packed else v_rows)
            elif packed:
                v_coeffs = torch.zeros_like(coeffs).index_add_(0, gaussian_ids, v_rows)
            else:
                v_coeffs = v_rows[0] if v_rows.shape[0] == 1 else v_rows.sum(0)
        if need_means:
            if packed:
                v_means = torch.zeros_like(means).index_add_(0, gaussian_ids, v_dirs)
            else:
                v_means = v_dirs[0] if v_dirs.shape[0] == 1 else v_dirs.sum(0)
    return v_means, v_coeffs


class _RasterizeToPixelsWithSH(torch.autograd.Function):
    """rasterize_to_pixels_with_sh for calls that want gradients: the forward pass is the kernel
    that evaluates the colours of the entries it stages; what it leaves in the colour cache --
    the colour (and depth) of every row some tile staged -- is all the backward pass needs of the
    colours, because a row that no tile staged was composited nowhere and takes no gradient."""

    @staticmethod
    def forward(ctx, sh_degree, means, viewmats, coeffs, depths, radii, camera_ids, gaussian_ids, means2d,
                conics, opacities, pix_vels, rolling_shutter_time, backgrounds, width, height, tile_size,
                isect_offsets, flatten_ids, color_cache, absgrad):
        render_colors, render_alphas, last_ids = _make_lazy_hip_func("rasterize_to_pixels_sh_fwd")(
            sh_degree, means, viewmats, coeffs, gaussian_ids, depths, means2d, conics, opacities, pix_vels,
            rolling_shutter_time, backgrounds, width, height, tile_size, isect_offsets, flatten_ids,
            cache=color_cache, want_last_ids=True)
        ctx.save_for_backward(means, viewmats, coeffs, radii, camera_ids, gaussian_ids, means2d, conics,
                              opacities, pix_vels, rolling_shutter_time, backgrounds, isect_offsets, flatten_ids,
                              render_alphas, last_ids, color_cache)
        ctx.sh_degree, ctx.has_depths = sh_degree, depths is not None
        ctx.width, ctx.height, ctx.tile_size, ctx.absgrad = width, height, tile_size, absgrad
        return render_colors, render_alphas.float()

    @staticmethod
    def backward(ctx, v_render_colors, v_render_alphas):
        (means, viewmats, coeffs, radii, camera_ids, gaussian_ids, means2d, conics, opacities, pix_vels,
         rolling_shutter_time, backgrounds, isect_offsets, flatten_ids, render_alphas, last_ids,
         cache) = ctx.saved_tensors
        # the rows' colours as the forward pass evaluated them; rows it never staged hold NaN,
        # are read by no pixel that composited them, and count as zero in both kernels below
        # (the SH backward only asks whether a colour is positive)
        colors = cache if ctx.has_depths else cache[..., :3].contiguous()
        # (with the depth channel: its gradient as a contiguous tensor of its own, which the
        # projection's backward pass takes as it is)
        (v_means2d_abs, v_means2d, v_conics, v_colors, v_opacities, v_pix_vels,
         *v_depth_channel) = _make_lazy_hip_func("rasterize_to_pixels_bwd")(
            means2d, conics, colors, opacities, pix_vels, rolling_shutter_time, backgrounds,
            ctx.width, ctx.height, ctx.tile_size, isect_offsets, flatten_ids, render_alphas,
            last_ids, v_render_colors.contiguous(), v_render_alphas.contiguous(), ctx.absgrad,
            colors_from_cache=True)
        if ctx.absgrad:
            means2d.absgrad = v_means2d_abs
        v_means, v_coeffs = _view_colors_backward(
            ctx.sh_degree, means, viewmats, coeffs, radii, camera_ids, gaussian_ids, colors, v_colors,
            ctx.needs_input_grad[1], ctx.needs_input_grad[3])
        v_depths = v_depth_channel[0] if ctx.has_depths and ctx.needs_input_grad[4] else None
        v_backgrounds = None
        if ctx.needs_input_grad[13]:
            v_backgrounds = (v_render_colors * (1.0 - render_alphas).float()).sum(dim=(1, 2))
        return (None, v_means, None, v_coeffs, v_depths, None, None, None, v_means2d, v_conics, v_opacities,
                v_pix_vels, None, v_backgrounds, None, None, None, None, None, None, None)


class _SphericalHarmonics(torch.autograd.Function):
    @staticmethod
    def forward(ctx, sh_degree, dirs, coeffs, masks):
        colors = _make_lazy_hip_func("compute_sh_fwd")(sh_degree, dirs, coeffs, masks)
        ctx.save_for_backward(dirs, coeffs, masks)
        ctx.sh_degree = sh_degree
        ctx.num_bases = coeffs.shape[-2]
        return colors

    @staticmethod
    def backward(ctx, v_colors):
        dirs, coeffs, masks = ctx.saved_tensors
        compute_v_dirs = ctx.needs_input_grad[1]
        v_coeffs, v_dirs = _make_lazy_hip_func("compute_sh_bwd")(
            ctx.num_bases, ctx.sh_degree, dirs, coeffs, masks, v_colors.contiguous(),
            compute_v_dirs)
        return None, (v_dirs if compute_v_dirs else None), v_coeffs, None
