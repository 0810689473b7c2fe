"""A stand-in for the HIP operator table that runs the CPU oracle (forward only).

Test infrastructure: it lets the CPU test-suite drive the host-side logic of
splatad_amd.rendering / splatad_amd.hip._wrapper (argument checks, packing, channel
chunking, render modes, meta dictionaries) without a GPU.  It is never installed outside a
test's monkeypatch.
"""
import numpy as np
import torch

import oracle


def _n(t):
    return None if t is None else t.detach().cpu().numpy()


def _t(a, dtype=None):
    if a is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(a))
    return t if dtype is None else t.to(dtype)


class OracleOps:
    def fully_fused_projection_fwd(self, means, covars, quats, scales, velocities, viewmats, Ks, W, H,
                                   lin, ang, rs, eps2d, near, far, radius_clip, calc_comp):
        out = oracle.projection_fwd(_n(means), _n(covars), _n(quats), _n(scales), _n(velocities),
                                    _n(viewmats), _n(Ks), W, H, _n(lin), _n(ang), _n(rs), eps2d, near, far,
                                    radius_clip, calc_comp, precision="f32")
        return tuple(_t(o) for o in out)

    def fully_fused_projection_packed_fwd(self, means, covars, quats, scales, velocities, viewmats, Ks,
                                          W, H, lin, ang, rs, eps2d, near, far, radius_clip, calc_comp,
                                          isect_grid=None, beside=None):
        radii, m2, d, con, comp, pv = self.fully_fused_projection_fwd(
            means, covars, quats, scales, velocities, viewmats, Ks, W, H, lin, ang, rs, eps2d, near, far,
            radius_clip, calc_comp)
        C = viewmats.shape[0]
        sel = torch.nonzero(radii[..., 0] > 0)
        cam, gid = sel[:, 0].contiguous(), sel[:, 1].contiguous()
        indptr = torch.zeros(C + 1, dtype=torch.int32)
        indptr[1:] = torch.cumsum(torch.bincount(cam, minlength=C), 0).int()
        pick = lambda t: None if t is None else t[cam, gid].contiguous()
        return indptr, cam, gid, pick(radii), pick(m2), pick(d), pick(con), pick(comp), pick(pv)

    def fully_fused_lidar_projection_fwd(self, means, covars, quats, scales, velocities, viewmats,
                                         min_el, max_el, min_az, max_az, lin, ang, rs, eps2d, near, far,
                                         radius_clip, calc_comp):
        out = oracle.lidar_projection_fwd(_n(means), _n(covars), _n(quats), _n(scales), _n(velocities),
                                          _n(viewmats), min_el, max_el, min_az, max_az, _n(lin), _n(ang),
                                          _n(rs), eps2d, near, far, radius_clip, calc_comp, precision="f32")
        return tuple(_t(o) for o in out)

    def compute_sh_fwd(self, degree, dirs, coeffs, masks):
        return _t(oracle.spherical_harmonics(degree, _n(dirs), _n(coeffs), _n(masks), precision="f32"))

    def view_colors_fwd(self, degree, means, viewmats, camera_ids, gaussian_ids, radii, coeffs, depths):
        # the chain of gsplat/rendering.py:325-351 on the oracle's spherical harmonics
        means, viewmats, radii, coeffs = _n(means), _n(viewmats), _n(radii), _n(coeffs)
        pos = np.linalg.inv(viewmats.astype(np.float64))[:, :3, 3]
        if camera_ids is not None:
            cam, gid = _n(camera_ids), _n(gaussian_ids)
            dirs = means[gid] - pos[cam]
            shs = coeffs[gid] if coeffs.ndim == 3 else coeffs[cam, gid]
        else:
            dirs = means[None] - pos[:, None]
            shs = np.broadcast_to(coeffs, (viewmats.shape[0],) + coeffs.shape[-3:]) if coeffs.ndim == 3 else coeffs
        cols = oracle.spherical_harmonics(degree, dirs.astype(np.float32), np.ascontiguousarray(shs),
                                          radii[..., 0] > 0, precision="f32")
        cols = np.maximum(cols + 0.5, 0.0).astype(np.float32)
        if depths is not None:
            cols = np.concatenate([cols, _n(depths)[..., None]], -1)
        return _t(cols)

    def isect_tiles(self, means2d, radii, depths, camera_ids, gaussian_ids, C, tile_size, tw, th, sort,
                    double_buffer, beside_work=None):
        if beside_work is not None:
            beside_work()
        out = oracle.isect_tiles(_n(means2d), _n(radii), _n(depths), tile_size, tw, th, sort, C,
                                 _n(camera_ids))
        return tuple(_t(o) for o in out)

    def isect_lidar_tiles(self, means2d, radii, depths, camera_ids, gaussian_ids, C, eb, res, min_az,
                          sort, double_buffer):
        out = oracle.isect_lidar_tiles(_n(means2d), _n(radii), _n(depths), _n(eb), res, min_az, sort, C,
                                       _n(camera_ids))
        return tuple(_t(o) for o in out)

    def isect_offset_encode(self, isect_ids, C, tw, th):
        return _t(oracle.isect_offset_encode(_n(isect_ids), C, tw, th))

    def rasterize_to_pixels_fwd(self, means2d, conics, colors, opacities, pix_vels, rs, backgrounds, W,
                                H, tile_size, offsets, flatten_ids):
        out = oracle.rasterize_to_pixels_fwd(_n(means2d), _n(conics), _n(colors), _n(opacities),
                                             _n(pix_vels), _n(rs), _n(backgrounds), W, H, tile_size,
                                             _n(offsets), _n(flatten_ids), precision="f32")
        return tuple(_t(o) for o in out)

    def rasterize_to_points_fwd(self, means2d, conics, colors, opacities, pix_vels, dcomp, backgrounds,
                                raster_pts, W, H, tw, th, asum, thr, offsets, flatten_ids, depth_idx,
                                range_channel=None):
        if range_channel is not None:  # the oracle follows the reference: one concatenated tensor
            colors = torch.cat([colors, range_channel[..., None]], dim=-1)
        out = oracle.rasterize_to_points_fwd(_n(means2d), _n(conics), _n(colors), _n(opacities),
                                             _n(pix_vels), _n(dcomp), _n(backgrounds), _n(raster_pts), W, H,
                                             tw, th, asum, thr, _n(offsets), _n(flatten_ids), depth_idx,
                                             precision="f32")
        return tuple(_t(o) for o in out)
