"""Pins of the differentiable torch restatement (oracle/torch_ref.py) used as gradient oracle:
its float64 forward values must agree with the C oracle's float64 build (itself pinned by
closed forms and brute force), and its gradients with central finite differences of the C
oracle for a few scalar losses (CPU only)."""
import math

import numpy as np
import torch

import oracle
from oracle import torch_ref

T = lambda a: torch.from_numpy(np.asarray(a)).double()


def _scene(n=400, C=2, seed=0):
    rng = np.random.default_rng(seed)
    means = (rng.uniform(-1, 1, (n, 3)) * 1.5).astype(np.float32)
    quats = rng.normal(size=(n, 4)).astype(np.float32)
    scales = np.exp(rng.normal(size=(n, 3)) * 0.4 - 2.3).astype(np.float32)
    vel = rng.normal(size=(n, 3)).astype(np.float32)
    vms = []
    from scipy.spatial.transform import Rotation
    for _ in range(C):
        vm = np.eye(4)
        vm[:3, :3] = Rotation.from_rotvec(rng.normal(size=3) * 0.2).as_matrix()
        vm[:3, 3] = [0.1, -0.1, 3.0]
        vms.append(vm)
    viewmats = np.array(vms, np.float32)
    Ks = np.array([[[120.0, 0, 48.0], [0, 118.0, 32.0], [0, 0, 1]]] * C, np.float32)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array([0.02, 0.0][:C], np.float32)
    return means, quats, scales, vel, viewmats, Ks, lin, ang, rs


def test_camera_projection_matches_c_oracle():
    means, quats, scales, vel, viewmats, Ks, lin, ang, rs = _scene()
    W, H = 96, 64
    ref = oracle.projection_fwd(means, None, quats, scales, vel, viewmats, Ks, W, H, lin, ang, rs,
                                calc_compensations=True, precision="f64")
    out = torch_ref.projection_fwd(T(means), None, T(quats), T(scales), T(vel), T(viewmats), T(Ks), W, H,
                                   T(lin), T(ang), T(rs))
    valid = ref[0][..., 0] > 0
    assert valid.sum() > 200
    for a, b in zip(out, ref[1:]):
        np.testing.assert_allclose(a.numpy()[valid], b[valid], rtol=1e-7, atol=1e-8)


def test_lidar_projection_matches_c_oracle():
    means, quats, scales, vel, viewmats, Ks, lin, ang, rs = _scene(seed=1)
    means = means * 10
    scales = scales * 4
    viewmats[:, :3, 3] = 0.3
    rs[:] = [0.1, 0.0]
    ref = oracle.lidar_projection_fwd(means, None, quats, scales, vel, viewmats, -60, 60, -180, 180, lin,
                                      ang, rs, eps2d=0.017, calc_compensations=True, precision="f64")
    out = torch_ref.lidar_projection_fwd(T(means), None, T(quats), T(scales), T(vel), T(viewmats), T(lin),
                                         T(ang), T(rs), eps2d=0.017)
    valid = ref[0][..., 0] > 0
    assert valid.sum() > 200
    for a, b in zip(out, ref[1:]):
        np.testing.assert_allclose(a.numpy()[valid], b[valid], rtol=1e-6, atol=1e-8)


def _raster_inputs(seed, C=1, N=300, W=40, H=24, D=3):
    rng = np.random.default_rng(seed)
    means2d = np.stack([rng.uniform(0, W, (C, N)), rng.uniform(0, H, (C, N))], -1).astype(np.float32)
    s = rng.uniform(1.5, 6.0, (C, N, 2))
    conics = np.stack([1 / s[..., 0] ** 2, rng.uniform(-0.3, 0.3, (C, N)) / (s[..., 0] * s[..., 1]),
                       1 / s[..., 1] ** 2], -1).astype(np.float32)
    colors = rng.normal(size=(C, N, D)).astype(np.float32)
    opac = rng.uniform(0.1, 1.0, (C, N)).astype(np.float32)
    depths = rng.uniform(1, 10, (C, N)).astype(np.float32)
    pix_vels = (rng.normal(size=(C, N, 2)) * 20).astype(np.float32)
    radii = np.ceil(3 * s).astype(np.int32)
    return means2d, conics, colors, opac, depths, pix_vels, radii


def test_rasterize_to_pixels_matches_c_oracle_and_finite_differences():
    C, N, W, H, D, ts = 1, 300, 40, 24, 3, 8
    means2d, conics, colors, opac, depths, pix_vels, radii = _raster_inputs(5, C, N, W, H, D)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    rs = np.array([0.03], np.float32)
    bg = np.array([[0.3, 0.6, 0.1]], np.float32)
    _, ids, flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    offs = oracle.isect_offset_encode(ids, C, tw, th)
    rc, ra, _ = oracle.rasterize_to_pixels_fwd(means2d, conics, colors, opac, pix_vels, rs, bg, W, H, ts,
                                               offs, flat, precision="f64")
    tm, tc, tcol, top, tpv = (T(x).requires_grad_() for x in (means2d, conics, colors, opac, pix_vels))
    o_rc, o_ra = torch_ref.rasterize_to_pixels(tm, tc, tcol, top, tpv, T(rs), T(bg), W, H, ts,
                                               torch.from_numpy(offs), torch.from_numpy(flat))
    np.testing.assert_allclose(o_rc.detach().numpy(), rc, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(o_ra.detach().numpy(), ra, rtol=1e-9, atol=1e-10)
    # gradient of a random linear functional vs central differences of the C oracle
    rng = np.random.default_rng(0)
    wc, wa = rng.normal(size=rc.shape), rng.normal(size=ra.shape)
    loss = (o_rc * T(wc)).sum() + (o_ra * T(wa)).sum()
    g_m, g_op, g_col = torch.autograd.grad(loss, (tm, top, tcol))

    def f(m2, op_, col_):
        a, b, _ = oracle.rasterize_to_pixels_fwd(m2, conics, col_, op_, pix_vels, rs, bg, W, H, ts, offs,
                                                 flat, precision="f64")
        return (a * wc).sum() + (b * wa).sum()

    # inputs are float32 in the C interface: use a step that float32 represents exactly enough
    for n_chk in range(6):
        g = int(rng.integers(0, N))
        h = 2.0 ** -9
        mp, mm = means2d.copy(), means2d.copy()
        mp[0, g, 0] += h; mm[0, g, 0] -= h
        fd = (f(mp, opac, colors) - f(mm, opac, colors)) / (float(mp[0, g, 0]) - float(mm[0, g, 0]))
        assert abs(fd - g_m[0, g, 0].item()) <= 2e-3 * max(1.0, abs(fd)), (g, fd, g_m[0, g, 0].item())
        cp, cm = colors.copy(), colors.copy()
        cp[0, g, 1] += h; cm[0, g, 1] -= h
        fd = (f(means2d, opac, cp) - f(means2d, opac, cm)) / (float(cp[0, g, 1]) - float(cm[0, g, 1]))
        assert abs(fd - g_col[0, g, 1].item()) <= 1e-6 * max(1.0, abs(fd))


def test_rasterize_to_points_matches_c_oracle():
    H, W, tw, th, D = 8, 64, 16, 4, 4
    rng = np.random.default_rng(3)
    N = 150
    az = -180.0 + (np.arange(W) + 0.5) * 360.0 / W
    el = np.linspace(-20, 20, H)
    rp = np.zeros((1, H, W, 4), np.float32)
    rp[0, :, :, 0] = az[None]; rp[0, :, :, 1] = el[:, None]
    rp[0, :, :, 2] = rng.uniform(5, 60, (H, W)); rp[0, :, :, 3] = rng.normal(size=(H, W)) * 0.05
    rp[0, 1, :4, 2] = 0
    means2d = np.stack([rng.uniform(-180, 180, N), rng.uniform(-25, 25, N)], -1)[None].astype(np.float32)
    s = rng.uniform(3.0, 20.0, (N, 2))
    conics = np.stack([1 / s[:, 0] ** 2, rng.uniform(-0.3, 0.3, N) / (s[:, 0] * s[:, 1]), 1 / s[:, 1] ** 2],
                      -1)[None].astype(np.float32)
    depths = rng.uniform(1, 70, (1, N)).astype(np.float32)
    feats = np.concatenate([rng.normal(size=(1, N, D - 1)).astype(np.float32), depths[..., None]], -1)
    opac = rng.uniform(0.05, 0.7, (1, N)).astype(np.float32)
    pv = (rng.normal(size=(1, N, 3)) * 20).astype(np.float32)
    dc = (rng.normal(size=(1, N, 2)) * 0.5).astype(np.float32)
    radii = (3 * s).astype(np.float32)[None]
    eb = np.array([-30.0, 0.0, 30.0], np.float32)
    res = 360.0 / W * tw
    _, ids, flat = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, -180.0)
    offs = oracle.isect_offset_encode(ids, 1, W // tw, H // th)
    ref = oracle.rasterize_to_points_fwd(means2d, conics, feats, opac, pv, dc, None, rp, W, H, tw, th,
                                         True, 0.3, offs, flat, D - 1, precision="f64")
    out = torch_ref.rasterize_to_points(T(means2d), T(conics), T(feats), T(opac), T(pv), T(dc), None, T(rp),
                                        tw, th, True, 0.3, torch.from_numpy(offs), torch.from_numpy(flat), D - 1)
    np.testing.assert_allclose(out[0].numpy(), ref[0], rtol=1e-8, atol=1e-9)
    np.testing.assert_allclose(out[1].numpy(), ref[1], rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(out[2].numpy(), ref[3], rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(out[3].numpy(), ref[4], rtol=1e-8, atol=1e-9)


def test_sh_matches_c_oracle():
    rng = np.random.default_rng(2)
    dirs = rng.normal(size=(200, 3)).astype(np.float32)
    coeffs = rng.normal(size=(200, 25, 3)).astype(np.float32)
    for deg in range(5):
        a = torch_ref.spherical_harmonics(deg, T(dirs), T(coeffs)).numpy()
        np.testing.assert_allclose(a, oracle.spherical_harmonics(deg, dirs, coeffs, precision="f64"),
                                   rtol=1e-10, atol=1e-12)
