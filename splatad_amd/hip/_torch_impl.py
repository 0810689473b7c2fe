"""Compositing written in plain tensor operations over (Gaussian, pixel, sensor) index lists.

Counterpart of `accumulate`, `accumulate_lidar`, `_rasterize_to_pixels` and
`_rasterize_to_points` of the reference (gsplat/cuda/_torch_impl.py:610-1022): the index lists
come from the HIP kernels behind `rasterize_to_indices_in_range[_lidar]`, everything after that
is ordinary torch, so gradients come from autograd and every intermediate can be inspected.
Much slower and hungrier for memory than the fused kernels; meant for experiments and as a
cross-check of them.

The reference delegates two steps to the third-party package `nerfacc`
(`render_weight_from_alpha`, `accumulate_along_rays`; no version is pinned by the reference),
which is not a dependency here.  Their published definitions are restated below:

  * per ray, the transmittance in front of sample k is the product of (1 - alpha) over the
    samples of that ray before k, and the weight of sample k is that transmittance times its
    alpha (`_weights_along_rays`);
  * a ray's value is the sum of weight * value over its samples (`_sum_along_rays`).

As in nerfacc, samples of one ray must be contiguous and ordered front to back, which is how
`rasterize_to_indices_in_range[_lidar]` emits them.
"""
from typing import Optional, Tuple

import torch
from torch import Tensor


def _weights_along_rays(alphas: Tensor, ray_indices: Tensor) -> Tuple[Tensor, Tensor]:
    """(weights, transmittances) of the samples of contiguous rays: T_k = prod_{j<k} (1 - a_j)
    within a ray, w_k = T_k a_k.

    The running product is a running sum of logarithms taken in float64, so that one cumulative
    sum over all samples serves every ray (the part before a ray's first sample is subtracted)
    without losing the float32 accuracy of the result.  alpha <= 0.999 keeps the logarithms finite.
    """
    if alphas.numel() == 0:
        return alphas, alphas
    log_keep = torch.log1p(-alphas.double())
    before = torch.cumsum(log_keep, dim=0) - log_keep  # exclusive, over all rays
    new_ray = torch.ones_like(ray_indices, dtype=torch.bool)
    new_ray[1:] = ray_indices[1:] != ray_indices[:-1]
    first = torch.nonzero(new_ray).squeeze(-1)  # first sample of every ray present
    ray_of_sample = torch.cumsum(new_ray.long(), dim=0) - 1
    trans = torch.exp(before - before[first][ray_of_sample]).to(alphas.dtype)
    return trans * alphas, trans


def _sum_along_rays(weights: Tensor, values: Optional[Tensor], ray_indices: Tensor, n_rays: int) -> Tensor:
    """[n_rays, D] sums of weights[:, None] * values per ray (D = 1, the weights themselves,
    without values)."""
    src = weights[:, None] if values is None else weights[:, None] * values
    out = torch.zeros((n_rays, src.shape[-1]), dtype=src.dtype, device=src.device)
    return out.index_add(0, ray_indices, src)


def _sigmas(conics: Tensor, deltas: Tensor) -> Tensor:
    dx, dy = deltas[:, 0], deltas[:, 1]
    return 0.5 * (conics[:, 0] * dx * dx + conics[:, 2] * dy * dy) + conics[:, 1] * dx * dy


def accumulate(
    means2d: Tensor,  # [C, N, 2]
    conics: Tensor,  # [C, N, 3]
    opacities: Tensor,  # [C, N]
    colors: Tensor,  # [C, N, channels]
    pix_vels: Tensor,  # [C, N, 2]
    rolling_shutter_time: Tensor,  # [C]
    gaussian_ids: Tensor,  # [M]
    pixel_ids: Tensor,  # [M]
    camera_ids: Tensor,  # [M]
    image_width: int,
    image_height: int,
) -> Tuple[Tensor, Tensor]:
    """Alpha compositing of the listed (Gaussian, pixel, camera) triples in plain torch.

    Returns (renders[C, image_height, image_width, channels],
    alphas[C, image_height, image_width, 1]).  Reference: gsplat/cuda/_torch_impl.py:610-706.
    """
    C = means2d.shape[0]
    channels = colors.shape[-1]
    col = pixel_ids % image_width
    row = pixel_ids // image_width
    # time offset of the pixel's row under a rolling shutter, -1/2 .. 1/2 of the readout time
    roll = rolling_shutter_time[camera_ids] * (row / (image_height - 1) - 0.5)
    centres = torch.stack([col, row], dim=-1) + 0.5
    pair = (camera_ids, gaussian_ids)
    deltas = means2d[pair] + roll[:, None] * pix_vels[pair] - centres
    alphas = torch.clamp_max(opacities[pair] * torch.exp(-_sigmas(conics[pair], deltas)), 0.999)

    rays = camera_ids * (image_height * image_width) + pixel_ids
    n_rays = C * image_height * image_width
    weights, _ = _weights_along_rays(alphas, rays)
    renders = _sum_along_rays(weights, colors[pair], rays, n_rays)
    accs = _sum_along_rays(weights, None, rays, n_rays)
    return (renders.reshape(C, image_height, image_width, channels),
            accs.reshape(C, image_height, image_width, 1))


def accumulate_lidar(
    means2d: Tensor,  # [C, N, 2]
    conics: Tensor,  # [C, N, 3]
    opacities: Tensor,  # [C, N]
    lidar_features: Tensor,  # [C, N, channels], last channel = range
    pix_vels: Tensor,  # [C, N, 3]
    depth_compensations: Tensor,  # [C, N, 2]
    raster_pts: Tensor,  # [C, image_height, image_width, 4] = azimuth, elevation, range, time
    gaussian_ids: Tensor,  # [M]
    pixel_ids: Tensor,  # [M]
    camera_ids: Tensor,  # [M]
    image_width: int,
    image_height: int,
    compute_alpha_sum_until_pts: bool,
    compute_alpha_sum_until_pts_threshold: float,
) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
    """Alpha compositing of the listed (Gaussian, point, lidar) triples in plain torch.  The
    rendered range channel is the Gaussian's range plus its depth compensation along the
    angular offset plus its range rate times the point's time.

    Returns (renders[C, H, W, channels], alphas[C, H, W, 1], alpha_sum_until_points[C, H, W, 1]
    or None: the sum of alphas of the Gaussians whose range lies more than the threshold in
    front of the point).  Reference: gsplat/cuda/_torch_impl.py:709-830.
    """
    C = means2d.shape[0]
    channels = lidar_features.shape[-1]
    col = pixel_ids % image_width
    row = pixel_ids // image_width
    pts = raster_pts[camera_ids, row, col]  # [M, 4]
    roll = pts[:, -1]
    pair = (camera_ids, gaussian_ids)
    vels = pix_vels[pair]
    # angular offsets folded into [-180, 180)
    deltas = torch.remainder(means2d[pair] + roll[:, None] * vels[:, :2] - pts[:, :2] + 180, 360) - 180
    deltas = torch.where(deltas < -180, deltas + 360, deltas)
    alphas = torch.clamp_max(opacities[pair] * torch.exp(-_sigmas(conics[pair], deltas)), 0.999)

    feats = lidar_features[pair]
    ranges = feats[:, -1] + (deltas * depth_compensations[pair]).sum(dim=-1) + vels[:, 2] * roll
    feats = torch.cat([feats[:, :-1], ranges[:, None]], dim=-1)

    rays = camera_ids * (image_height * image_width) + pixel_ids
    n_rays = C * image_height * image_width
    alpha_sum = None
    if compute_alpha_sum_until_pts:
        in_front = lidar_features[pair][:, -1] < pts[:, 2] - compute_alpha_sum_until_pts_threshold
        alpha_sum = _sum_along_rays(torch.where(in_front, alphas, torch.zeros_like(alphas)), None,
                                    rays, n_rays).reshape(C, image_height, image_width, 1)
    weights, _ = _weights_along_rays(alphas, rays)
    renders = _sum_along_rays(weights, feats, rays, n_rays)
    accs = _sum_along_rays(weights, None, rays, n_rays)
    return (renders.reshape(C, image_height, image_width, channels),
            accs.reshape(C, image_height, image_width, 1), alpha_sum)


def _composite_in_windows(shape, channels, n_isects, isect_offsets, tile_points, batch_per_iter, device,
                          list_window, composite_window, extra=False):
    """Shared driver of the list-based rasterizers: the tiles' lists are walked in windows of
    `batch_per_iter` batches of `tile_points` entries; `list_window(first, last, T)` emits the
    (Gaussian, pixel, sensor) triples of a window for pixels that arrive with transmittance T,
    `composite_window(triples)` composites them to (values, alphas[, extra]) as if the window
    stood alone, and the driver scales each window by the transmittance in front of it.  The
    optional third output (the lidar's alpha sum) is not scaled.  Returns (values [*shape,
    channels], alphas [*shape, 1], extra | None)."""
    values = torch.zeros((*shape, channels), device=device)
    alphas = torch.zeros((*shape, 1), device=device)
    extras = torch.zeros_like(alphas) if extra else None
    starts = isect_offsets.flatten()
    ends = torch.cat([starts[1:], starts.new_tensor([n_isects])])
    longest = int((ends - starts).max().item()) if ends.numel() else 0
    for first in range(0, -(-longest // tile_points), batch_per_iter):
        in_front = 1.0 - alphas[..., 0]
        triples = list_window(first, first + batch_per_iter, in_front)
        if len(triples[0]) == 0:
            break
        out = composite_window(triples)
        values = values + out[0] * in_front[..., None]
        alphas = alphas + out[1] * in_front[..., None]
        if extra:
            extras = extras + out[2]
    return values, alphas, extras


def _rasterize_to_pixels(
    means2d: Tensor,  # [C, N, 2]
    conics: Tensor,  # [C, N, 3]
    colors: Tensor,  # [C, N, channels]
    opacities: Tensor,  # [C, N]
    pix_vels: Tensor,  # [C, N, 2]
    image_width: int,
    image_height: int,
    tile_size: int,
    isect_offsets: Tensor,  # [C, tile_height, tile_width]
    flatten_ids: Tensor,  # [n_isects]
    rolling_shutter_time: Tensor,  # [C]
    backgrounds: Optional[Tensor] = None,  # [C, channels]
    batch_per_iter: int = 100,
):
    """`rasterize_to_pixels` through index lists and `accumulate`, `batch_per_iter` batches of
    each tile's list at a time; differentiable by autograd.  Returns (render_colors,
    render_alphas).  Reference: gsplat/cuda/_torch_impl.py:833-918.
    """
    from ._wrapper import rasterize_to_indices_in_range

    render_colors, render_alphas, _ = _composite_in_windows(
        (means2d.shape[0], image_height, image_width), colors.shape[-1], len(flatten_ids), isect_offsets,
        tile_size * tile_size, batch_per_iter, means2d.device,
        lambda first, last, T: rasterize_to_indices_in_range(
            first, last, T, means2d, conics, opacities, pix_vels, image_width, image_height, tile_size,
            isect_offsets, flatten_ids, rolling_shutter_time),
        lambda ids: accumulate(means2d, conics, opacities, colors, pix_vels, rolling_shutter_time, *ids,
                               image_width, image_height))
    if backgrounds is not None:
        render_colors = render_colors + backgrounds[:, None, None, :] * (1.0 - render_alphas)
    return render_colors, render_alphas


def _rasterize_to_points(
    means2d: Tensor,  # [C, N, 2]
    conics: Tensor,  # [C, N, 3]
    lidar_features: Tensor,  # [C, N, channels]
    opacities: Tensor,  # [C, N]
    pix_vels: Tensor,  # [C, N, 3]
    depth_compensations: Tensor,  # [C, N, 2]
    raster_pts: Tensor,  # [C, image_height, image_width, 4]
    image_width: int,
    image_height: int,
    tile_width: int,
    tile_height: int,
    isect_offsets: Tensor,  # [C, tile_grid_height, tile_grid_width]
    flatten_ids: Tensor,  # [n_isects]
    compute_alpha_sum_until_points: bool,
    compute_alpha_sum_until_points_threshold: float,
    batch_per_iter: int = 100,
):
    """`rasterize_to_points` through index lists and `accumulate_lidar`; differentiable by
    autograd.  Returns (render_lidar_features, render_alphas, alpha_sum_until_points | None).
    Reference: gsplat/cuda/_torch_impl.py:921-1022.
    """
    from ._wrapper import rasterize_to_indices_in_range_lidar

    return _composite_in_windows(
        (means2d.shape[0], image_height, image_width), lidar_features.shape[-1], len(flatten_ids),
        isect_offsets, tile_width * tile_height, batch_per_iter, means2d.device,
        lambda first, last, T: rasterize_to_indices_in_range_lidar(
            first, last, T, means2d, conics, opacities, pix_vels, raster_pts, image_width, image_height,
            tile_width, tile_height, isect_offsets, flatten_ids),
        lambda ids: accumulate_lidar(
            means2d, conics, opacities, lidar_features, pix_vels, depth_compensations, raster_pts, *ids,
            image_width, image_height, compute_alpha_sum_until_pts=compute_alpha_sum_until_points,
            compute_alpha_sum_until_pts_threshold=compute_alpha_sum_until_points_threshold),
        extra=compute_alpha_sum_until_points)
