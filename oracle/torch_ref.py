"""Differentiable float64 restatement of the path in plain PyTorch -- TEST INFRASTRUCTURE ONLY.

Used as the gradient oracle: the HIP backward kernels are compared with torch.autograd
through these functions.  They restate the same forward rules as oracle/splatad_oracle.c
(which is pinned by closed forms and brute force, see tests/test_oracle_*.py) and are
themselves pinned by matching that C oracle's double-precision outputs to ~1e-10
(tests/test_oracle_torch_ref.py).  They follow what the reference's own torch restatement
does for its gradient tests (gsplat/cuda/_torch_impl.py:10-418, 610-1022): vectorised
projection, and per-tile dense compositing over the sorted intersection lists.

No culling happens here: callers mask with the radii produced by the implementation under
test, exactly like the reference's tests (tests/test_basic.py:360, 654).
"""
import math

import torch

RAD2DEG = 57.2957795131  # the constant of the reference (utils.cuh:10), not 180/pi to the last bit


def quat_scale_to_covar(quats, scales):
    q = quats / quats.norm(dim=-1, keepdim=True)
    w, x, y, z = q.unbind(-1)
    R = torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y),
        2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x),
        2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], dim=-1).reshape(-1, 3, 3)
    M = R * scales[:, None, :]
    return M @ M.transpose(-1, -2)


def covars6_to_mat(c):
    return torch.stack([c[:, 0], c[:, 1], c[:, 2], c[:, 1], c[:, 3], c[:, 4], c[:, 2], c[:, 4], c[:, 5]],
                       dim=-1).reshape(-1, 3, 3)


def _to_sensor(means, cov, velocities, viewmats):
    R = viewmats[:, :3, :3]
    t = viewmats[:, :3, 3]
    pc = torch.einsum("cij,nj->cni", R, means) + t[:, None, :]
    covc = torch.einsum("cij,njk,clk->cnil", R, cov, R)
    if velocities is None:
        velc = torch.zeros_like(pc)
    else:
        velc = torch.einsum("cij,nj->cni", R, velocities)
    return pc, covc, velc


def _blur_and_invert(cov2, eps2d):
    det_orig = cov2[..., 0, 0] * cov2[..., 1, 1] - cov2[..., 0, 1] * cov2[..., 1, 0]
    sxx = cov2[..., 0, 0] + eps2d
    syy = cov2[..., 1, 1] + eps2d
    sxy = 0.5 * (cov2[..., 0, 1] + cov2[..., 1, 0])
    det = sxx * syy - sxy * sxy
    comp = torch.sqrt(torch.clamp(det_orig / det, min=0.0))
    conics = torch.stack([syy / det, -sxy / det, sxx / det], dim=-1)
    return conics, comp


def projection_fwd(means, covars6, quats, scales, velocities, viewmats, Ks, width, height,
                   lin_vel, ang_vel, rs_time, eps2d=0.3):
    """Camera projection without culls. Returns means2d, depths, conics, compensations, pix_vels."""
    cov = covars6_to_mat(covars6) if covars6 is not None else quat_scale_to_covar(quats, scales)
    pc, covc, velc = _to_sensor(means, cov, velocities, viewmats)
    x, y, z = pc.unbind(-1)
    fx, fy = Ks[:, 0, 0, None], Ks[:, 1, 1, None]
    cx, cy = Ks[:, 0, 2, None], Ks[:, 1, 2, None]
    tan_fovx, tan_fovy = 0.5 * width / fx, 0.5 * height / fy
    lim_x_pos = (width - cx) / fx + 0.3 * tan_fovx
    lim_x_neg = cx / fx + 0.3 * tan_fovx
    lim_y_pos = (height - cy) / fy + 0.3 * tan_fovy
    lim_y_neg = cy / fy + 0.3 * tan_fovy
    tx = z * torch.minimum(lim_x_pos, torch.maximum(-lim_x_neg, x / z))
    ty = z * torch.minimum(lim_y_pos, torch.maximum(-lim_y_neg, y / z))
    O = torch.zeros_like(z)
    J = torch.stack([fx / z, O, -fx * tx / z ** 2, O, fy / z, -fy * ty / z ** 2], dim=-1).reshape(*z.shape, 2, 3)
    cov2 = J @ covc @ J.transpose(-1, -2)
    means2d = torch.stack([fx * x / z + cx, fy * y / z + cy], dim=-1)
    conics, comp = _blur_and_invert(cov2, eps2d)
    tv = lin_vel[:, None, :] + torch.cross(ang_vel[:, None, :].expand_as(pc), pc, dim=-1) - velc
    pix_vels = -(J @ tv[..., None])[..., 0] * (rs_time > 0)[:, None, None]
    return means2d, z, conics, comp, pix_vels


def lidar_projection_fwd(means, covars6, quats, scales, velocities, viewmats, lin_vel, ang_vel,
                         rs_time, eps2d=0.017):
    """Lidar projection without culls. Returns means2d, depths, conics, compensations,
    pix_vels [C,N,3], depth_compensations [C,N,2]."""
    cov = covars6_to_mat(covars6) if covars6 is not None else quat_scale_to_covar(quats, scales)
    pc, covc, velc = _to_sensor(means, cov, velocities, viewmats)
    x, y, z = pc.unbind(-1)
    rho2 = x * x + y * y
    r2 = rho2 + z * z
    r = torch.sqrt(r2)
    rho = torch.sqrt(rho2)
    O = torch.zeros_like(z)
    J = torch.stack([
        -y / rho2 * RAD2DEG, x / rho2 * RAD2DEG, O,
        -x * z / (r2 * rho) * RAD2DEG, -y * z / (r2 * rho) * RAD2DEG, rho / r2 * RAD2DEG,
        x / r, y / r, z / r], dim=-1).reshape(*z.shape, 3, 3)
    cs = J @ covc @ J.transpose(-1, -2)
    means2d = torch.stack([torch.atan2(y, x) * RAD2DEG, torch.asin(z / r) * RAD2DEG], dim=-1)
    a1, a2 = cs[..., 0, 0] + eps2d, cs[..., 0, 1]
    b1, b2 = cs[..., 1, 0], cs[..., 1, 1] + eps2d
    c1, c2 = cs[..., 2, 0], cs[..., 2, 1]
    D = a1 * b2 - a2 * b1
    dcomp = torch.stack([(b1 * c2 - b2 * c1) / D, (a2 * c1 - a1 * c2) / D], dim=-1)
    conics, comp = _blur_and_invert(cs[..., :2, :2], eps2d)
    tv = lin_vel[:, None, :] + torch.cross(ang_vel[:, None, :].expand_as(pc), pc, dim=-1) - velc
    pix_vels = -(J @ tv[..., None])[..., 0] * (rs_time > 0)[:, None, None]
    return means2d, r, conics, comp, pix_vels, dcomp


def sh_basis(degree, dirs):
    """Real SH basis values [..., (degree+1)^2] (sh.cu:13-93)."""
    d = dirs / dirs.norm(dim=-1, keepdim=True)
    x, y, z = d.unbind(-1)
    b = [torch.full_like(x, 0.2820947917738781)]
    if degree >= 1:
        b += [-0.48860251190292 * y, 0.48860251190292 * z, -0.48860251190292 * x]
    if degree >= 2:
        z2 = z * z
        c1, s1 = x * x - y * y, 2 * x * y
        b += [0.5462742152960395 * s1, -1.092548430592079 * z * y,
              0.9461746957575601 * z2 - 0.3153915652525201, -1.092548430592079 * z * x,
              0.5462742152960395 * c1]
    if degree >= 3:
        c2, s2 = x * c1 - y * s1, x * s1 + y * c1
        t = -2.285228997322329 * z2 + 0.4570457994644658
        b += [-0.5900435899266435 * s2, 1.445305721320277 * z * s1, t * y,
              z * (1.865881662950577 * z2 - 1.119528997770346), t * x,
              1.445305721320277 * z * c1, -0.5900435899266435 * c2]
    if degree >= 4:
        c3, s3 = x * c2 - y * s2, x * s2 + y * c2
        u = z * (-4.683325804901025 * z2 + 2.007139630671868)
        v = 3.31161143515146 * z2 - 0.47308734787878
        b += [0.6258357354491763 * s3, -1.770130769779931 * z * s2, v * s1, u * y,
              1.984313483298443 * z * b[12] - 1.006230589874905 * b[6], u * x, v * c1,
              -1.770130769779931 * z * c2, 0.6258357354491763 * c3]
    return torch.stack(b, dim=-1)


def spherical_harmonics(degree, dirs, coeffs):
    B = sh_basis(degree, dirs)
    return torch.einsum("...k,...kc->...c", B, coeffs[..., : B.shape[-1], :])


def _composite(alpha_raw, sigma):
    valid = (sigma >= 0) & (alpha_raw >= 1.0 / 255.0)
    a = torch.where(valid, alpha_raw, torch.zeros_like(alpha_raw))
    one_minus = 1.0 - a
    T_incl = torch.cumprod(one_minus, dim=1)
    T_excl = torch.cat([torch.ones_like(T_incl[:, :1]), T_incl[:, :-1]], dim=1)
    stop = valid & (T_incl <= 1e-4)
    alive = torch.cumsum(stop.to(torch.int64), dim=1) == 0
    w = a * T_excl * alive
    T_final = torch.prod(torch.where(alive, one_minus, torch.ones_like(one_minus)), dim=1)
    return w, T_final, alive & valid, a, T_excl, T_incl


def _angle_difference(a, b):
    d = torch.fmod(a - b + 180.0, 360.0) - 180.0
    return torch.where(d < -180.0, d + 360.0, d)


def rasterize_to_pixels(means2d, conics, colors, opacities, pix_vels, rs_time, backgrounds, width,
                        height, tile_size, offsets, flatten_ids, tiles=None, near=None):
    """Dense per-tile compositing; differentiable w.r.t. the float inputs.  [C,N,...] layout.
    With `tiles` (flat (camera, tile) indices) only those tiles are rendered, the rest stays 0.
    With `near` (a dict with "margin"), near["rows"] becomes a bool [C * N]: the Gaussians whose
    alpha lies within the relative margin of the 1/255 threshold at some pixel that is still
    compositing when it reaches them -- the pairs a float32 evaluation may decide differently --
    and the Gaussians composited at a pixel that has such a pair."""
    C, th, tw = offsets.shape
    D = colors.shape[-1]
    n_isects = flatten_ids.shape[0]
    m2, cn, col = means2d.reshape(-1, 2), conics.reshape(-1, 3), colors.reshape(-1, D)
    op, pv = opacities.reshape(-1), pix_vels.reshape(-1, 2)
    off = offsets.reshape(-1).tolist() + [n_isects]
    out = torch.zeros(C, height, width, D, dtype=means2d.dtype)
    alph = torch.zeros(C, height, width, 1, dtype=means2d.dtype)
    rows = []
    for c in range(C):
        for ty in range(th):
            for tx in range(tw):
                t = (c * th + ty) * tw + tx
                i0, j0 = ty * tile_size, tx * tile_size
                i1, j1 = min(i0 + tile_size, height), min(j0 + tile_size, width)
                if i1 <= i0 or j1 <= j0 or (tiles is not None and t not in tiles):
                    continue
                ii, jj = torch.meshgrid(torch.arange(i0, i1), torch.arange(j0, j1), indexing="ij")
                px = (jj.reshape(-1, 1) + 0.5).to(means2d.dtype)
                py = (ii.reshape(-1, 1) + 0.5).to(means2d.dtype)
                roll = rs_time[c] * ((py - 0.5) / (height - 1) - 0.5)
                g = flatten_ids[off[t]: off[t + 1]].long()
                if g.numel() == 0:
                    T_final = torch.ones(px.shape[0], dtype=means2d.dtype)
                    pix = torch.zeros(px.shape[0], D, dtype=means2d.dtype)
                else:
                    dx = m2[g, 0][None] + roll * pv[g, 0][None] - px
                    dy = m2[g, 1][None] + roll * pv[g, 1][None] - py
                    sigma = 0.5 * (cn[g, 0][None] * dx * dx + cn[g, 2][None] * dy * dy) + cn[g, 1][None] * dx * dy
                    alpha = torch.clamp(op[g][None] * torch.exp(-sigma), max=0.999)
                    w, T_final, _, _, _, _ = _composite(alpha, sigma)
                    pix = w @ col[g]
                    if near is not None:
                        with torch.no_grad():
                            near.setdefault("rows", torch.zeros(m2.shape[0], dtype=torch.bool))
                            raw = op[g][None] * torch.exp(-sigma)
                            _, _, _, a_, _, T_incl = _composite(alpha, sigma)
                            stop = (a_ > 0) & (T_incl <= 1e-4)
                            before = torch.cumsum(stop.to(torch.int64), dim=1) - stop.to(torch.int64)
                            close = ((raw * 255.0 - 1.0).abs() <= near["margin"]) & (before == 0)
                            # such a pair, decided the other way, changes its pixel for every
                            # Gaussian composited there: the transmittance of those behind it, the
                            # colour accumulated behind those in front of it, by alpha ~ 0.4 %
                            shared = close.any(1, keepdim=True) & (w > 0)
                            near["rows"][g[(close | shared).any(0)]] = True
                if backgrounds is not None:
                    pix = pix + T_final[:, None] * backgrounds[c][None]
                rows.append((c, i0, i1, j0, j1, pix, T_final))
    for c, i0, i1, j0, j1, pix, T_final in rows:
        out[c, i0:i1, j0:j1] = pix.reshape(i1 - i0, j1 - j0, D)
        alph[c, i0:i1, j0:j1, 0] = (1.0 - T_final).reshape(i1 - i0, j1 - j0)
    return out, alph


def rasterize_to_points(means2d, conics, colors, opacities, pix_vels, depth_comps, backgrounds,
                        raster_pts, tile_width, tile_height, compute_alpha_sum, threshold, offsets,
                        flatten_ids, depth_idx, tiles=None, near=None):
    """Dense per-tile compositing onto lidar points. Returns (colors, alphas, alpha_sum, median).
    With `tiles` (flat (sensor, tile) indices) only those tiles are rendered.  With `near` (a dict
    with "margin" and, for the alpha sum, "depth_margin" in metres), near["rows"] becomes a bool
    [C * N] as in rasterize_to_pixels: the Gaussians with an alpha within the relative margin of
    1/255 at a point still compositing, or a depth within depth_margin of the alpha sum's
    range - threshold cut there, and the Gaussians composited at a point that has such a pair."""
    C, gh, gw = offsets.shape
    H, W = raster_pts.shape[1:3]
    D = colors.shape[-1]
    n_isects = flatten_ids.shape[0]
    m2, cn, col = means2d.reshape(-1, 2), conics.reshape(-1, 3), colors.reshape(-1, D)
    op, pv, dc = opacities.reshape(-1), pix_vels.reshape(-1, 3), depth_comps.reshape(-1, 2)
    off = offsets.reshape(-1).tolist() + [n_isects]
    dt = means2d.dtype
    out = torch.zeros(C, H, W, D, dtype=dt)
    alph = torch.zeros(C, H, W, 1, dtype=dt)
    asum = torch.zeros(C, H, W, 1, dtype=dt)
    med = torch.zeros(C, H, W, 1, dtype=dt)
    pieces = []
    for c in range(C):
        for ty in range(gh):
            for tx in range(gw):
                t = (c * gh + ty) * gw + tx
                i0, j0 = ty * tile_height, tx * tile_width
                i1, j1 = min(i0 + tile_height, H), min(j0 + tile_width, W)
                if i1 <= i0 or j1 <= j0 or (tiles is not None and t not in tiles):
                    continue
                P = raster_pts[c, i0:i1, j0:j1].reshape(-1, 4)
                active = (P[:, 2] > 0).to(dt)
                g = flatten_ids[off[t]: off[t + 1]].long()
                if g.numel() == 0:
                    continue
                roll = P[:, 3:4]
                dx = _angle_difference(m2[g, 0][None] + roll * pv[g, 0][None], P[:, 0:1])
                dy = _angle_difference(m2[g, 1][None] + roll * pv[g, 1][None], P[:, 1:2])
                sigma = 0.5 * (cn[g, 0][None] * dx * dx + cn[g, 2][None] * dy * dy) + cn[g, 1][None] * dx * dy
                alpha = torch.clamp(op[g][None] * torch.exp(-sigma), max=0.999)
                w, T_final, used, a_eff, T_excl, T_incl = _composite(alpha, sigma)
                pix = w @ col[g]
                extra = dc[g, 0][None] * dx + dc[g, 1][None] * dy + pv[g, 2][None] * roll
                onehot = torch.zeros(D, dtype=dt)
                onehot[depth_idx] = 1.0
                pix = pix + (w * extra).sum(1, keepdim=True) * onehot[None]
                if backgrounds is not None:
                    pix = pix + T_final[:, None] * backgrounds[c][None]
                pix = pix * active[:, None]
                al = (1.0 - T_final) * active
                before = col[g, depth_idx][None] < (P[:, 2:3] - threshold)
                s = (a_eff * used * before).sum(1) * active if compute_alpha_sum else torch.zeros_like(al)
                if near is not None:
                    with torch.no_grad():
                        near.setdefault("rows", torch.zeros(m2.shape[0], dtype=torch.bool))
                        raw = op[g][None] * torch.exp(-sigma)
                        stop = (a_eff > 0) & (T_incl <= 1e-4)
                        earlier = torch.cumsum(stop.to(torch.int64), dim=1) - stop.to(torch.int64)
                        live = (earlier == 0) & (active[:, None] > 0)
                        close = ((raw * 255.0 - 1.0).abs() <= near["margin"]) & live
                        shared = close.any(1, keepdim=True) & (w > 0)
                        hit = close | shared
                        if compute_alpha_sum and near.get("depth_margin"):
                            cut = (col[g, depth_idx][None] - (P[:, 2:3] - threshold)).abs() <= near["depth_margin"]
                            hit = hit | (cut & used & live)
                        near["rows"][g[hit.any(0)]] = True
                cross = used & (T_excl > 0.5) & (T_incl <= 0.5)
                m = ((col[g, depth_idx][None] + extra) * cross).sum(1) * active
                pieces.append((c, i0, i1, j0, j1, pix, al, s, m))
    for c, i0, i1, j0, j1, pix, al, s, m in pieces:
        out[c, i0:i1, j0:j1] = pix.reshape(i1 - i0, j1 - j0, D)
        alph[c, i0:i1, j0:j1, 0] = al.reshape(i1 - i0, j1 - j0)
        asum[c, i0:i1, j0:j1, 0] = s.reshape(i1 - i0, j1 - j0)
        med[c, i0:i1, j0:j1, 0] = m.detach().reshape(i1 - i0, j1 - j0)
    return out, alph, (asum if compute_alpha_sum else None), med


# ---------------------------------------------------------------------------
# the unfused projection operators (gsplat/cuda/_torch_impl.py:10-200 of the reference
# holds the torch restatement its own tests compare against)
# ---------------------------------------------------------------------------
def _quat_to_rotmat(quats):
    q = quats / quats.norm(dim=-1, keepdim=True)
    w, x, y, z = q.unbind(-1)
    return torch.stack([
        1 - 2 * (y * y + z * z), 2 * (x * y - w * z), 2 * (x * z + w * y),
        2 * (x * y + w * z), 1 - 2 * (x * x + z * z), 2 * (y * z - w * x),
        2 * (x * z - w * y), 2 * (y * z + w * x), 1 - 2 * (x * x + y * y)], dim=-1).reshape(-1, 3, 3)


def quat_scale_to_covar_preci(quats, scales, compute_covar=True, compute_preci=True, triu=False):
    """covar = R S S R^T, preci = R S^-1 S^-1 R^T; `triu` returns (xx, xy, xz, yy, yz, zz)."""
    R = _quat_to_rotmat(quats)
    covars = precis = None
    if compute_covar:
        M = R * scales[:, None, :]
        covars = M @ M.transpose(-1, -2)
    if compute_preci:
        P = R * (1.0 / scales[:, None, :])
        precis = P @ P.transpose(-1, -2)
    if triu:
        pick = lambda m: None if m is None else torch.stack(
            [m[:, 0, 0], m[:, 0, 1], m[:, 0, 2], m[:, 1, 1], m[:, 1, 2], m[:, 2, 2]], dim=-1)
        covars, precis = pick(covars), pick(precis)
    return covars, precis


def world_to_cam(means, covars, viewmats):
    R = viewmats[:, :3, :3]
    t = viewmats[:, :3, 3]
    means_c = torch.einsum("cij,nj->cni", R, means) + t[:, None, :]
    covars_c = torch.einsum("cij,njk,clk->cnil", R, covars, R)
    return means_c, covars_c


def _persp_jacobian(means, Ks, width, height):
    x, y, z = means.unbind(-1)
    fx, fy = Ks[:, 0, 0, None], Ks[:, 1, 1, None]
    cx, cy = Ks[:, 0, 2, None], Ks[:, 1, 2, None]
    tan_fovx, tan_fovy = 0.5 * width / fx, 0.5 * height / fy
    lim_x_pos = (width - cx) / fx + 0.3 * tan_fovx
    lim_x_neg = cx / fx + 0.3 * tan_fovx
    lim_y_pos = (height - cy) / fy + 0.3 * tan_fovy
    lim_y_neg = cy / fy + 0.3 * tan_fovy
    tx = z * torch.minimum(lim_x_pos, torch.maximum(-lim_x_neg, x / z))
    ty = z * torch.minimum(lim_y_pos, torch.maximum(-lim_y_neg, y / z))
    O = torch.zeros_like(z)
    J = torch.stack([fx / z, O, -fx * tx / z ** 2, O, fy / z, -fy * ty / z ** 2], dim=-1).reshape(*z.shape, 2, 3)
    means2d = torch.stack([fx * x / z + cx, fy * y / z + cy], dim=-1)
    return J, means2d


def persp_proj(means, covars, Ks, width, height):
    J, means2d = _persp_jacobian(means, Ks, width, height)
    return means2d, J @ covars @ J.transpose(-1, -2)


def compute_pix_velocity(p_view, lin_vel, ang_vel, velocities, Ks, width, height):
    J, _ = _persp_jacobian(p_view, Ks, width, height)
    tv = lin_vel[:, None, :] + torch.cross(ang_vel[:, None, :].expand_as(p_view), p_view, dim=-1) - velocities
    return -(J @ tv[..., None])[..., 0]


def _lidar_jacobian(means):
    x, y, z = means.unbind(-1)
    rho2 = x * x + y * y
    r2 = rho2 + z * z
    r, rho = torch.sqrt(r2), torch.sqrt(rho2)
    O = torch.zeros_like(z)
    J = torch.stack([
        -y / rho2 * RAD2DEG, x / rho2 * RAD2DEG, O,
        -x * z / (r2 * rho) * RAD2DEG, -y * z / (r2 * rho) * RAD2DEG, rho / r2 * RAD2DEG,
        x / r, y / r, z / r], dim=-1).reshape(*z.shape, 3, 3)
    means2d = torch.stack([torch.atan2(y, x) * RAD2DEG, torch.asin(z / r) * RAD2DEG], dim=-1)
    return J, means2d


def lidar_proj(means, covars, eps2d):
    J, means2d = _lidar_jacobian(means)
    cs = J @ covars @ J.transpose(-1, -2)
    a1, a2 = cs[..., 0, 0] + eps2d, cs[..., 0, 1]
    b1, b2 = cs[..., 1, 0], cs[..., 1, 1] + eps2d
    c1, c2 = cs[..., 2, 0], cs[..., 2, 1]
    D = a1 * b2 - a2 * b1
    dcomp = torch.stack([(b1 * c2 - b2 * c1) / D, (a2 * c1 - a1 * c2) / D], dim=-1)
    return means2d, cs[..., :2, :2], dcomp


def compute_lidar_velocity(p_view, lin_vel, ang_vel, velocities):
    J, _ = _lidar_jacobian(p_view)
    tv = lin_vel[:, None, :] + torch.cross(ang_vel[:, None, :].expand_as(p_view), p_view, dim=-1) - velocities
    return -(J @ tv[..., None])[..., 0]
