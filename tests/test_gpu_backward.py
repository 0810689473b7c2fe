"""GPU parity of the backward kernels against float64 torch.autograd through the
restatement in oracle/torch_ref.py (pinned against the C oracle on the CPU).

Bar: 1e-3 relative.  "Relative" is taken per tensor against |reference| + its RMS, because
single gradient entries pass through zero; entries that are ill-conditioned in float32
(at most 0.5% of a tensor) get a looser 2e-2 bound.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref
from tests.gpu_util import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu

T64 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).double()


def assert_grad_close(got, ref, name, rtol=1e-3, frac=0.995, loose=2e-2, near_rows=None, near_loose=5e-2):
    """|got - ref| <= rtol (|ref| + rms) on at least `frac` of the entries and <= loose (|ref| + rms)
    on every entry.  With `near_rows` (bool per leading row: the Gaussians for which the float64
    comparator found an alpha >= 1/255 decision within rounding distance of its threshold, or
    that share a pixel with such a pair) that bar holds for every other row without exception,
    and the listed rows, whose gradient moves by the flipped pair's share, get `near_loose`."""
    got = np.asarray(got, np.float64)
    ref = np.asarray(ref, np.float64)
    assert got.shape == ref.shape, (name, got.shape, ref.shape)
    if ref.size == 0:
        return
    scale = math.sqrt(float((ref ** 2).mean())) + 1e-12
    rel = np.abs(got - ref) / (np.abs(ref) + scale)
    if near_rows is not None:
        near_rows = np.asarray(near_rows, bool).reshape(-1)
        assert near_rows.shape[0] == got.shape[0], (name, near_rows.shape, got.shape)
        if near_rows.any():
            worst_near = float(rel[near_rows].max())
            assert worst_near <= near_loose, f"{name}: worst rel {worst_near:.3e} on a row with a near-threshold pair"
        rel = rel[~near_rows]
        if rel.size == 0:
            return
    ok = (rel <= rtol).mean()
    worst = float(rel.max())
    assert ok >= frac and worst <= loose, f"{name}: {ok:.4f} within {rtol}, worst rel {worst:.3e} (rms {scale:.3e})"


def _gaussians(n, seed, spread=1.5, log_scale=-2.3):
    rng = np.random.default_rng(seed)
    means = (rng.uniform(-1, 1, (n, 3)) * spread).astype(np.float32)
    quats = rng.normal(size=(n, 4)).astype(np.float32)
    scales = np.exp(rng.normal(size=(n, 3)) * 0.4 + log_scale).astype(np.float32)
    vel = rng.normal(size=(n, 3)).astype(np.float32)
    return rng, means, quats, scales, vel


def _poses(rng, C, t=(0.1, -0.1, 3.0), rot=0.2):
    from scipy.spatial.transform import Rotation
    vms = []
    for _ in range(C):
        vm = np.eye(4)
        vm[:3, :3] = Rotation.from_rotvec(rng.normal(size=3) * rot).as_matrix()
        vm[:3, 3] = np.array(t) + rng.normal(size=3) * 0.05
        vms.append(vm)
    return np.array(vms, np.float32)


def _covars6(quats, scales):
    c = torch_ref.quat_scale_to_covar(T64(quats), T64(scales)).reshape(-1, 9)
    return c[:, [0, 1, 2, 4, 5, 8]].float().numpy()


@pytest.mark.parametrize("use_covars,use_vel,comp,packed,sparse", [
    (False, True, True, False, False), (False, False, False, False, False),
    (True, True, False, False, False), (False, True, True, True, False),
    (False, True, False, True, True), (True, False, True, True, True)])
def test_projection_camera_backward(use_covars, use_vel, comp, packed, sparse):
    from splatad_amd import fully_fused_projection
    C, N, W, H = 3, 4000, 96, 64
    rng, means, quats, scales, vel = _gaussians(N, 40)
    viewmats = _poses(rng, C)
    Ks = np.array([[[120.0, 0, 48.0], [0, 118.0, 32.0], [0, 0, 1]]] * C, np.float32)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array([0.02, 0.0, 0.03], np.float32)
    covars = _covars6(quats, scales) if use_covars else None

    def leaf(a):
        return None if a is None else to_dev(a).requires_grad_()
    g_means, g_cov, g_q, g_s = leaf(means), leaf(covars), leaf(None if use_covars else quats), leaf(None if use_covars else scales)
    g_vel, g_vm = leaf(vel if use_vel else None), leaf(viewmats)
    out = fully_fused_projection(g_means, g_cov, g_q, g_s, g_vel, g_vm, to_dev(Ks), W, H, to_dev(lin),
                                 to_dev(ang), to_dev(rs), eps2d=0.3, packed=packed, sparse_grad=sparse,
                                 calc_compensations=comp)
    if packed:
        cam_ids, gau_ids = to_np(out[0]), to_np(out[1])
        out = out[2:]
        sel = (cam_ids, gau_ids)
    else:
        valid = to_np(out[0])[..., 0] > 0
        sel = np.nonzero(valid)
    assert len(sel[0]) > 1000
    radii, means2d, depths, conics, comps, pix_vels = out

    # float64 reference on the same inputs; cotangents live on the selected (camera, gaussian) pairs
    r_means, r_vm = T64(means).requires_grad_(), T64(viewmats).requires_grad_()
    r_cov = T64(covars).requires_grad_() if use_covars else None
    r_q = None if use_covars else T64(quats).requires_grad_()
    r_s = None if use_covars else T64(scales).requires_grad_()
    r_vel = T64(vel).requires_grad_() if use_vel else None
    ref = torch_ref.projection_fwd(r_means, r_cov, r_q, r_s, r_vel, r_vm, T64(Ks), W, H, T64(lin), T64(ang),
                                   T64(rs), eps2d=0.3)
    rng2 = np.random.default_rng(1)
    loss_g, loss_r = 0.0, 0.0
    for got, want in ((means2d, ref[0]), (depths, ref[1]), (conics, ref[2]), (comps, ref[3]), (pix_vels, ref[4])):
        if got is None:
            continue
        w = rng2.normal(size=tuple(got.shape)).astype(np.float32)
        loss_g = loss_g + (got * to_dev(w)).sum()
        wsel = T64(w)
        want_sel = want[torch.from_numpy(sel[0]), torch.from_numpy(sel[1])] if packed else want
        if not packed:
            mask = torch.from_numpy(valid)
            wsel = wsel * (mask if want.dim() == 2 else mask[..., None])
        loss_r = loss_r + (want_sel * wsel).sum()
    inputs_g = [t for t in (g_means, g_cov, g_q, g_s, g_vel, g_vm) if t is not None]
    inputs_r = [t for t in (r_means, r_cov, r_q, r_s, r_vel, r_vm) if t is not None]
    names = [n for n, t in zip(("means", "covars", "quats", "scales", "velocities", "viewmats"),
                               (g_means, g_cov, g_q, g_s, g_vel, g_vm)) if t is not None]
    grads_g = torch.autograd.grad(loss_g, inputs_g)
    grads_r = torch.autograd.grad(loss_r, inputs_r)
    for n, a, b in zip(names, grads_g, grads_r):
        if a.is_sparse:
            assert sparse and n != "viewmats"
            a = a.to_dense()
        assert_grad_close(to_np(a), b.numpy(), n)


@pytest.mark.parametrize("use_covars,use_vel,comp", [(False, True, True), (True, False, False), (False, False, True)])
def test_projection_lidar_backward(use_covars, use_vel, comp):
    from splatad_amd import fully_fused_lidar_projection
    C, N = 2, 4000
    rng, means, quats, scales, vel = _gaussians(N, 41, spread=25.0, log_scale=-1.2)
    means[:, 2] *= 0.2
    viewmats = _poses(rng, C, t=(0.3, 0.2, 0.1), rot=0.1)
    lin = (rng.normal(size=(C, 3)) * 5).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.2).astype(np.float32)
    rs = np.array([0.1, 0.0], np.float32)
    covars = _covars6(quats, scales) if use_covars else None

    def leaf(a):
        return None if a is None else to_dev(a).requires_grad_()
    g_means, g_cov, g_q, g_s = leaf(means), leaf(covars), leaf(None if use_covars else quats), leaf(None if use_covars else scales)
    g_vel, g_vm = leaf(vel if use_vel else None), leaf(viewmats)
    out = fully_fused_lidar_projection(g_means, g_cov, g_q, g_s, g_vel, g_vm, to_dev(lin), to_dev(ang),
                                       to_dev(rs), -40.0, 40.0, -180.0, 180.0, eps2d=0.017, near_plane=2.0,
                                       calc_compensations=comp)
    valid = to_np(out[0])[..., 0] > 0
    assert valid.sum() > 1000
    r_means, r_vm = T64(means).requires_grad_(), T64(viewmats).requires_grad_()
    r_cov = T64(covars).requires_grad_() if use_covars else None
    r_q = None if use_covars else T64(quats).requires_grad_()
    r_s = None if use_covars else T64(scales).requires_grad_()
    r_vel = T64(vel).requires_grad_() if use_vel else None
    ref = torch_ref.lidar_projection_fwd(r_means, r_cov, r_q, r_s, r_vel, r_vm, T64(lin), T64(ang), T64(rs),
                                         eps2d=0.017)
    rng2 = np.random.default_rng(2)
    loss_g, loss_r = 0.0, 0.0
    mask = torch.from_numpy(valid)
    for got, want in zip(out[1:], ref):
        if got is None:
            continue
        w = rng2.normal(size=tuple(got.shape)).astype(np.float32)
        loss_g = loss_g + (got * to_dev(w)).sum()
        loss_r = loss_r + (want * T64(w) * (mask if want.dim() == 2 else mask[..., None])).sum()
    inputs_g = [t for t in (g_means, g_cov, g_q, g_s, g_vel, g_vm) if t is not None]
    inputs_r = [t for t in (r_means, r_cov, r_q, r_s, r_vel, r_vm) if t is not None]
    names = [n for n, t in zip(("means", "covars", "quats", "scales", "velocities", "viewmats"),
                               (g_means, g_cov, g_q, g_s, g_vel, g_vm)) if t is not None]
    grads_g = torch.autograd.grad(loss_g, inputs_g)
    grads_r = torch.autograd.grad(loss_r, inputs_r)
    for n, a, b in zip(names, grads_g, grads_r):
        assert_grad_close(to_np(a), b.numpy(), n)


def _raster_scene(seed, C, N, W, H, D):
    rng = np.random.default_rng(seed)
    means2d = np.stack([rng.uniform(-4, W + 4, (C, N)), rng.uniform(-4, H + 4, (C, N))], -1).astype(np.float32)
    s = rng.uniform(1.5, 7.0, (C, N, 2))
    conics = np.stack([1 / s[..., 0] ** 2, rng.uniform(-0.3, 0.3, (C, N)) / (s[..., 0] * s[..., 1]),
                       1 / s[..., 1] ** 2], -1).astype(np.float32)
    colors = rng.normal(size=(C, N, D)).astype(np.float32)
    opac = rng.uniform(0.05, 1.0, (C, N)).astype(np.float32)
    depths = rng.uniform(1, 10, (C, N)).astype(np.float32)
    pix_vels = (rng.normal(size=(C, N, 2)) * 20).astype(np.float32)
    radii = np.ceil(3 * s).astype(np.int32)
    bg = rng.uniform(size=(C, D)).astype(np.float32)
    return means2d, conics, colors, opac, depths, pix_vels, radii, bg


@pytest.mark.parametrize("D,ts,N", [(3, 16, 600), (4, 16, 3000), (1, 8, 500), (33, 16, 500), (40, 16, 400), (5, 4, 300),
                                    (5, 16, 500), (1, 16, 400), (8, 16, 300)])
def test_rasterize_to_pixels_backward(D, ts, N):
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_pixels
    C, W, H = 2, 72, 40
    means2d, conics, colors, opac, depths, pix_vels, radii, bg = _raster_scene(50 + D, C, N, W, H, D)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    rs = np.array([0.03, 0.0], np.float32)
    _, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    leaves_g = [to_dev(x).requires_grad_() for x in (means2d, conics, colors, opac, pix_vels, bg)]
    rc, ra = rasterize_to_pixels(leaves_g[0], leaves_g[1], leaves_g[2], leaves_g[3], leaves_g[4], W, H, ts,
                                 offs, flat, rolling_shutter_time=to_dev(rs), backgrounds=leaves_g[5])
    leaves_r = [T64(x).requires_grad_() for x in (means2d, conics, colors, opac, pix_vels, bg)]
    o_rc, o_ra = torch_ref.rasterize_to_pixels(leaves_r[0], leaves_r[1], leaves_r[2], leaves_r[3], leaves_r[4],
                                               T64(rs), leaves_r[5], W, H, ts, offs.cpu(), flat.cpu())
    np.testing.assert_allclose(to_np(rc), o_rc.detach().numpy(), atol=1e-4)
    rng = np.random.default_rng(0)
    wc = rng.normal(size=tuple(rc.shape)).astype(np.float32)
    wa = rng.normal(size=tuple(ra.shape)).astype(np.float32)
    grads_g = torch.autograd.grad((rc * to_dev(wc)).sum() + (ra * to_dev(wa)).sum(), leaves_g)
    grads_r = torch.autograd.grad((o_rc * T64(wc)).sum() + (o_ra * T64(wa)).sum(), leaves_r)
    for n, a, b in zip(("means2d", "conics", "colors", "opacities", "pix_vels", "backgrounds"), grads_g, grads_r):
        assert_grad_close(to_np(a), b.numpy(), f"{n} D={D}")


def test_rasterize_to_pixels_absgrad():
    # |d loss_p / d mean2d| summed over pixels, against per-pixel autograd on a tiny scene
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_pixels
    C, N, W, H, D, ts = 1, 40, 16, 16, 3, 16
    means2d, conics, colors, opac, depths, pix_vels, radii, _ = _raster_scene(7, C, N, W, H, D)
    rs = np.zeros(1, np.float32)
    _, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), ts, 1, 1)
    offs = isect_offset_encode(ids, C, 1, 1)
    m = to_dev(means2d).requires_grad_()
    rc, ra = rasterize_to_pixels(m, to_dev(conics), to_dev(colors), to_dev(opac), to_dev(pix_vels), W, H, ts,
                                 offs, flat, rolling_shutter_time=to_dev(rs), absgrad=True)
    rng = np.random.default_rng(0)
    wc = rng.normal(size=tuple(rc.shape)).astype(np.float32)
    (rc * to_dev(wc)).sum().backward()
    assert hasattr(m, "absgrad") and m.absgrad.shape == m.shape
    rm = T64(means2d).requires_grad_()
    o_rc, _ = torch_ref.rasterize_to_pixels(rm, T64(conics), T64(colors), T64(opac), T64(pix_vels), T64(rs), None,
                                            W, H, ts, offs.cpu(), flat.cpu())
    per_pixel = (o_rc * T64(wc)).sum(-1).reshape(-1)
    absref = torch.zeros_like(rm)
    for p in range(per_pixel.shape[0]):
        (g,) = torch.autograd.grad(per_pixel[p], rm, retain_graph=True)
        absref += g.abs()
    assert_grad_close(to_np(m.absgrad), absref.numpy(), "absgrad")
    assert_grad_close(to_np(m.grad), torch.autograd.grad(per_pixel.sum(), rm)[0].numpy(), "means2d")


@pytest.mark.parametrize("D,asum", [(5, True), (5, False), (33, True), (36, True), (2, True), (3, False)])
def test_rasterize_to_points_backward(D, asum):
    from splatad_amd import isect_lidar_tiles, isect_offset_encode, rasterize_to_points
    H, W, tw, th = 8, 128, 32, 4
    rng = np.random.default_rng(60 + D)
    N = 400
    az = -180.0 + (np.arange(W) + 0.5) * 360.0 / W
    el = np.linspace(-20, 20, H)
    rp = np.zeros((1, H, W, 4), np.float32)
    rp[0, :, :, 0] = az[None]; rp[0, :, :, 1] = el[:, None]
    rp[0, :, :, 2] = rng.uniform(5, 60, (H, W)); rp[0, :, :, 3] = rng.normal(size=(H, W)) * 0.05
    rp[0, 1, :4, 2] = 0
    means2d = np.stack([rng.uniform(-180, 180, N), rng.uniform(-25, 25, N)], -1)[None].astype(np.float32)
    s = rng.uniform(2.0, 12.0, (N, 2))
    conics = np.stack([1 / s[:, 0] ** 2, rng.uniform(-0.3, 0.3, N) / (s[:, 0] * s[:, 1]), 1 / s[:, 1] ** 2],
                      -1)[None].astype(np.float32)
    depths = rng.uniform(1, 70, (1, N)).astype(np.float32)
    feats = np.concatenate([rng.normal(size=(1, N, D - 1)).astype(np.float32), depths[..., None]], -1)
    opac = rng.uniform(0.05, 0.8, (1, N)).astype(np.float32)
    pv = (rng.normal(size=(1, N, 3)) * 20).astype(np.float32)
    dc = (rng.normal(size=(1, N, 2)) * 0.5).astype(np.float32)
    radii = (3 * s).astype(np.float32)[None]
    eb = np.array([-30.0, 0.0, 30.0], np.float32)
    res = 360.0 / W * tw
    _, ids, flat = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb), res, -180.0)
    offs = isect_offset_encode(ids, 1, W // tw, H // th)
    arrays = (means2d, conics, feats, opac, pv, dc)
    lg = [to_dev(x).requires_grad_() for x in arrays]
    rf, ra, rsum, med = rasterize_to_points(lg[0], lg[1], lg[2], lg[3], lg[4], lg[5], to_dev(rp), W, H, tw, th,
                                            offs, flat, asum, 0.3)
    lr = [T64(x).requires_grad_() for x in arrays]
    o = torch_ref.rasterize_to_points(lr[0], lr[1], lr[2], lr[3], lr[4], lr[5], None, T64(rp), tw, th, asum, 0.3,
                                      offs.cpu(), flat.cpu(), D - 1)
    np.testing.assert_allclose(to_np(rf), o[0].detach().numpy(), atol=2e-4, rtol=1e-4)
    rng2 = np.random.default_rng(0)
    wc = rng2.normal(size=tuple(rf.shape)).astype(np.float32)
    wa = rng2.normal(size=tuple(ra.shape)).astype(np.float32)
    ws = rng2.normal(size=tuple(ra.shape)).astype(np.float32)
    loss_g = (rf * to_dev(wc)).sum() + (ra * to_dev(wa)).sum()
    loss_r = (o[0] * T64(wc)).sum() + (o[1] * T64(wa)).sum()
    if asum:
        loss_g = loss_g + (rsum * to_dev(ws)).sum()
        loss_r = loss_r + (o[2] * T64(ws)).sum()
    grads_g = torch.autograd.grad(loss_g, lg)
    grads_r = torch.autograd.grad(loss_r, lr)
    names = ("means2d", "conics", "features", "opacities", "pix_vels", "depth_compensations")
    for n, a, b in zip(names, grads_g, grads_r):
        assert_grad_close(to_np(a), b.numpy(), f"{n} D={D}")
    # features and ranges handed over separately: the gradient of the last channel comes apart
    ls = [to_dev(x).requires_grad_() for x in (means2d, conics, np.ascontiguousarray(feats[..., :-1]), opac,
                                               pv, dc, depths)]
    sf, sa, ssum, _ = rasterize_to_points(ls[0], ls[1], ls[2], ls[3], ls[4], ls[5], to_dev(rp), W, H, tw, th,
                                          offs, flat, asum, 0.3, ranges=ls[6])
    assert torch.equal(sf, rf) and torch.equal(sa, ra)
    loss_s = (sf * to_dev(wc)).sum() + (sa * to_dev(wa)).sum()
    if asum:
        loss_s = loss_s + (ssum * to_dev(ws)).sum()
    grads_s = torch.autograd.grad(loss_s, ls)
    for n, a, b in zip(names, grads_s[:6], grads_r):
        want = b.numpy()[..., :-1] if n == "features" else b.numpy()
        assert_grad_close(to_np(a), want, f"split {n} D={D}")
    assert_grad_close(to_np(grads_s[6]), grads_r[2].numpy()[..., -1], f"split ranges D={D}")


@pytest.mark.parametrize("deg", [0, 1, 2, 3, 4])
def test_spherical_harmonics_backward(deg):
    from splatad_amd import spherical_harmonics
    rng = np.random.default_rng(deg)
    n, K = 3000, 25
    dirs = (rng.normal(size=(n, 3)) * 2).astype(np.float32)
    coeffs = rng.normal(size=(n, K, 3)).astype(np.float32)
    masks = rng.random(n) > 0.3
    w = rng.normal(size=(n, 3)).astype(np.float32)
    gd, gc = to_dev(dirs).requires_grad_(), to_dev(coeffs).requires_grad_()
    col = spherical_harmonics(deg, gd, gc, masks=to_dev(masks))
    v_d, v_c = torch.autograd.grad((col * to_dev(w)).sum(), (gd, gc), allow_unused=True)
    rd, rc = T64(dirs).requires_grad_(), T64(coeffs).requires_grad_()
    ref = torch_ref.spherical_harmonics(deg, rd, rc) * T64(masks.astype(np.float64))[:, None]
    r_d, r_c = torch.autograd.grad((ref * T64(w)).sum(), (rd, rc), allow_unused=True)
    assert_grad_close(to_np(v_c), r_c.numpy(), "coeffs", frac=0.999)
    if deg > 0:
        assert_grad_close(to_np(v_d), r_d.numpy(), "dirs", frac=0.999)
    else:
        assert float(v_d.abs().max()) == 0.0
