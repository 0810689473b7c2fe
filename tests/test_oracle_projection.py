"""Pins for the oracle's projection functions (CPU only).

Each check is chosen so that a plausible mistake in oracle/splatad_oracle.c
(dropped term, wrong sign or index, transposed operand) fails it; none of them
re-types the oracle's own formula:
  * rotation matrices against scipy.spatial.transform.Rotation,
  * projection Jacobians against central finite differences of the point map,
  * pixel / spherical velocities against finite differences in time of the
    projected position of a moving point,
  * depth compensation against numpy.linalg.inv of the eps-augmented 3x3,
  * closed-form special cases (on-axis Gaussian, point on the +x axis,
    identity quaternion) and the cull rules by construction.
"""
import math

import numpy as np
import pytest
from scipy.spatial.transform import Rotation

import oracle

RAD2DEG = 180.0 / math.pi


def _rand_scene(n, seed, spread=1.0):
    rng = np.random.default_rng(seed)
    means = (rng.uniform(-1, 1, (n, 3)) * spread).astype(np.float32)
    quats = rng.normal(size=(n, 4)).astype(np.float32)
    scales = np.exp(rng.normal(size=(n, 3)) * 0.3 - 2.5).astype(np.float32)
    vel = rng.normal(size=(n, 3)).astype(np.float32)
    return rng, means, quats, scales, vel


def _covar_from_scipy(quats, scales):
    # scipy is scalar-last; the reference is (w, x, y, z)
    R = Rotation.from_quat(quats[:, [1, 2, 3, 0]].astype(np.float64)).as_matrix()
    S2 = scales.astype(np.float64) ** 2
    return np.einsum("nij,nj,nkj->nik", R, S2, R), R


def _cam(rng, C):
    vms, Ks = [], []
    for _ in range(C):
        R = Rotation.from_rotvec(rng.normal(size=3) * 0.2).as_matrix()
        vm = np.eye(4)
        vm[:3, :3] = R
        vm[:3, 3] = [rng.normal() * 0.1, rng.normal() * 0.1, 4.0]
        vms.append(vm)
        Ks.append([[310.0, 0, 158.0], [0, 295.0, 123.0], [0, 0, 1]])
    return np.array(vms, np.float32), np.array(Ks, np.float32)


def _pinhole(p, K):
    return np.array([K[0, 0] * p[0] / p[2] + K[0, 2], K[1, 1] * p[1] / p[2] + K[1, 2]])


def _fd_jac(f, p, h=1e-6):
    cols = []
    for k in range(3):
        d = np.zeros(3)
        d[k] = h
        cols.append((f(p + d) - f(p - d)) / (2 * h))
    return np.stack(cols, axis=-1)


@pytest.mark.parametrize("use_covars", [False, True])
def test_camera_projection_against_finite_differences(use_covars):
    C, N, W, H = 2, 300, 320, 240
    rng, means, quats, scales, vel = _rand_scene(N, 1)
    viewmats, Ks = _cam(rng, C)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array([0.02, 0.0], np.float32)
    cov, _ = _covar_from_scipy(quats, scales)
    covars6 = cov.reshape(N, 9)[:, [0, 1, 2, 4, 5, 8]].astype(np.float32)
    eps2d = 0.3
    out = oracle.projection_fwd(means, covars6 if use_covars else None,
                                None if use_covars else quats, None if use_covars else scales,
                                vel, viewmats, Ks, W, H, lin, ang, rs, eps2d=eps2d,
                                calc_compensations=True, precision="f64")
    radii, means2d, depths, conics, comps, pix_vels = out
    n_valid = 0
    for c in range(C):
        R = viewmats[c, :3, :3].astype(np.float64)
        t = viewmats[c, :3, 3].astype(np.float64)
        K = Ks[c].astype(np.float64)
        for g in range(N):
            if radii[c, g, 0] <= 0:
                continue
            n_valid += 1
            covw = cov[g] if not use_covars else np.array(
                [[covars6[g, 0], covars6[g, 1], covars6[g, 2]],
                 [covars6[g, 1], covars6[g, 3], covars6[g, 4]],
                 [covars6[g, 2], covars6[g, 4], covars6[g, 5]]], np.float64)
            pc = R @ means[g].astype(np.float64) + t
            J = _fd_jac(lambda p: _pinhole(p, K), pc)
            cov2 = J @ (R @ covw @ R.T) @ J.T
            det0 = np.linalg.det(cov2)
            cov2b = cov2 + eps2d * np.eye(2)
            con = np.linalg.inv(cov2b)
            np.testing.assert_allclose(means2d[c, g], _pinhole(pc, K), rtol=1e-9, atol=1e-9)
            np.testing.assert_allclose(depths[c, g], pc[2], rtol=1e-12)
            np.testing.assert_allclose(conics[c, g], [con[0, 0], con[0, 1], con[1, 1]],
                                       rtol=1e-5, atol=1e-7)
            np.testing.assert_allclose(comps[c, g], math.sqrt(max(0, det0 / np.linalg.det(cov2b))),
                                       rtol=1e-5, atol=1e-7)
            ext = 3 * np.sqrt(np.diag(cov2b))
            if rs[c] > 0:
                # image-plane velocity of the point as seen from the moving sensor
                vrel = lin[c].astype(np.float64) + np.cross(ang[c].astype(np.float64), pc) \
                    - R @ vel[g].astype(np.float64)
                h = 1e-6
                pv = (_pinhole(pc - vrel * h, K) - _pinhole(pc + vrel * h, K)) / (2 * h)
                np.testing.assert_allclose(pix_vels[c, g], pv, rtol=1e-5, atol=1e-6)
                ext = ext + np.abs(pv) * 0.5 * rs[c]
            else:
                assert (pix_vels[c, g] == 0).all()
            assert abs(radii[c, g, 0] - int(ext[0])) <= 1 and abs(radii[c, g, 1] - int(ext[1])) <= 1
    assert n_valid > 100


def test_camera_on_axis_closed_form_and_unnormalised_quat():
    # identity view, Gaussian on the optical axis: mu2 = (cx, cy), Sigma2 = (f/z)^2 Sigma_xy + eps
    z, f, cx, cy = 5.0, 300.0, 160.0, 120.0
    means = np.array([[0, 0, z]], np.float32)
    scales = np.array([[0.1, 0.2, 0.3]], np.float32)
    K = np.array([[[f, 0, cx], [0, f, cy], [0, 0, 1]]], np.float32)
    vm = np.eye(4, dtype=np.float32)[None]
    zero = np.zeros((1, 3), np.float32)
    for q in ([1, 0, 0, 0], [3.0, 0, 0, 0]):
        quats = np.array([q], np.float32)
        radii, m2, d, con, _, pv = oracle.projection_fwd(
            means, None, quats, scales, None, vm, K, 320, 240, zero, zero,
            np.zeros(1, np.float32), eps2d=0.3, precision="f64")
        sx = (f / z * 0.1) ** 2 + 0.3
        sy = (f / z * 0.2) ** 2 + 0.3
        np.testing.assert_allclose(m2[0, 0], [cx, cy], atol=1e-9)
        np.testing.assert_allclose(con[0, 0], [1 / sx, 0, 1 / sy], rtol=1e-6, atol=1e-12)
        assert d[0, 0] == z
        assert radii[0, 0].tolist() == [int(3 * math.sqrt(sx)), int(3 * math.sqrt(sy))]
    # rotating by 90 deg about z swaps the x/y extents
    c = math.sqrt(0.5)
    radii2, *_ = oracle.projection_fwd(means, None, np.array([[c, 0, 0, c]], np.float32), scales,
                                       None, vm, K, 320, 240, zero, zero, np.zeros(1, np.float32),
                                       precision="f64")
    assert radii2[0, 0].tolist() == [int(3 * math.sqrt(sy)), int(3 * math.sqrt(sx))]


def test_camera_rolling_shutter_notebook_scene():
    # 20 Gaussians at z=10, y in [-5,5], f=500, 500x500; pure sideways ego motion
    # gives pix_vel = (-f v_x / z, 0) and no vertical component.
    n, f, z, vx = 20, 500.0, 10.0, 3.0
    means = np.stack([np.zeros(n), np.linspace(-5, 5, n), np.full(n, z)], -1).astype(np.float32)
    quats = np.tile(np.array([[1, 0, 0, 0]], np.float32), (n, 1))
    scales = np.full((n, 3), 0.05, np.float32)
    K = np.array([[[f, 0, 250], [0, f, 250], [0, 0, 1]]], np.float32)
    vm = np.eye(4, dtype=np.float32)[None]
    lin = np.array([[vx, 0, 0]], np.float32)
    rs = np.array([0.1], np.float32)
    radii, m2, d, con, _, pv = oracle.projection_fwd(
        means, None, quats, scales, None, vm, K, 500, 500, lin, np.zeros((1, 3), np.float32), rs,
        precision="f64")
    assert (radii[0, :, 0] > 0).all()
    np.testing.assert_allclose(pv[0, :, 0], -f * vx / z, rtol=1e-12)
    np.testing.assert_allclose(pv[0, :, 1], 0, atol=1e-12)
    sx = (f / z * 0.05) ** 2 + 0.3
    assert (radii[0, :, 0] == int(3 * math.sqrt(sx) + f * vx / z * 0.05)).all()


def test_camera_cull_rules():
    K = np.array([[[300, 0, 160], [0, 300, 120], [0, 0, 1]]], np.float32)
    vm = np.eye(4, dtype=np.float32)[None]
    zero = np.zeros((1, 3), np.float32)
    quats = np.tile(np.array([[1, 0, 0, 0]], np.float32), (6, 1))
    scales = np.full((6, 3), 0.01, np.float32)
    means = np.array([
        [0, 0, 0.005],    # in front of near plane -> culled
        [0, 0, 200.0],    # beyond far plane (far=100) -> culled
        [0, 0, -1.0],     # behind -> culled
        [50, 0, 1.0],     # far outside the image -> culled
        [0, 0, 1.0],      # visible
        [0, 0, 50.0],     # tiny, removed by radius_clip
    ], np.float32)
    radii, m2, d, con, _, pv = oracle.projection_fwd(
        means, None, quats, scales, None, vm, K, 320, 240, zero, zero, np.zeros(1, np.float32),
        near_plane=0.01, far_plane=100.0, radius_clip=2.0, precision="f32")
    assert (radii[0, :, 0] > 0).tolist() == [False, False, False, False, True, False]
    # culled rows are zero-filled
    assert (m2[0, 0] == 0).all() and (con[0, 3] == 0).all() and d[0, 1] == 0


def _spherical(p):
    r = np.linalg.norm(p)
    return np.array([math.atan2(p[1], p[0]) * RAD2DEG, math.asin(p[2] / r) * RAD2DEG, r])


@pytest.mark.parametrize("use_covars", [False, True])
def test_lidar_projection_against_finite_differences(use_covars):
    C, N = 2, 300
    rng, means, quats, scales, vel = _rand_scene(N, 2, spread=20.0)
    means[:, 2] *= 0.2
    scales *= 3
    vms = []
    for _ in range(C):
        vm = np.eye(4)
        vm[:3, :3] = Rotation.from_rotvec(rng.normal(size=3) * 0.1).as_matrix()
        vm[:3, 3] = rng.normal(size=3)
        vms.append(vm)
    viewmats = np.array(vms, np.float32)
    lin = (rng.normal(size=(C, 3)) * 5).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array([0.1, 0.0], np.float32)
    cov, _ = _covar_from_scipy(quats, scales)
    covars6 = cov.reshape(N, 9)[:, [0, 1, 2, 4, 5, 8]].astype(np.float32)
    eps2d = 0.017
    out = oracle.lidar_projection_fwd(
        means, covars6 if use_covars else None, None if use_covars else quats,
        None if use_covars else scales, vel, viewmats, -45.0, 45.0, -180.0, 180.0, lin, ang, rs,
        eps2d=eps2d, calc_compensations=True, precision="f64")
    radii, means2d, depths, conics, comps, pix_vels, dcomps = out
    n_valid = 0
    for c in range(C):
        R = viewmats[c, :3, :3].astype(np.float64)
        t = viewmats[c, :3, 3].astype(np.float64)
        for g in range(N):
            if radii[c, g, 0] <= 0:
                continue
            n_valid += 1
            covw = cov[g] if not use_covars else np.array(
                [[covars6[g, 0], covars6[g, 1], covars6[g, 2]],
                 [covars6[g, 1], covars6[g, 3], covars6[g, 4]],
                 [covars6[g, 2], covars6[g, 4], covars6[g, 5]]], np.float64)
            pc = R @ means[g].astype(np.float64) + t
            sph = _spherical(pc)
            J = _fd_jac(_spherical, pc, h=1e-5)
            cs = J @ (R @ covw @ R.T) @ J.T
            cov2b = cs[:2, :2] + eps2d * np.eye(2)
            con = np.linalg.inv(cov2b)
            np.testing.assert_allclose(means2d[c, g], sph[:2], rtol=1e-9, atol=1e-9)
            np.testing.assert_allclose(depths[c, g], sph[2], rtol=1e-12)
            np.testing.assert_allclose(conics[c, g], [con[0, 0], con[0, 1], con[1, 1]],
                                       rtol=2e-5, atol=1e-6)
            np.testing.assert_allclose(
                comps[c, g], math.sqrt(max(0, np.linalg.det(cs[:2, :2]) / np.linalg.det(cov2b))),
                rtol=2e-5, atol=1e-6)
            # depth compensation == Lambda[2, :2] / Lambda[2, 2] of the eps-augmented covariance
            lam = np.linalg.inv(cs + np.diag([eps2d, eps2d, 0.0]))
            np.testing.assert_allclose(dcomps[c, g], lam[2, :2] / lam[2, 2], rtol=2e-4, atol=1e-7)
            ext = 3 * np.sqrt(np.diag(cov2b))
            if rs[c] > 0:
                vrel = lin[c].astype(np.float64) + np.cross(ang[c].astype(np.float64), pc) \
                    - R @ vel[g].astype(np.float64)
                h = 1e-6
                pv = (_spherical(pc - vrel * h) - _spherical(pc + vrel * h)) / (2 * h)
                np.testing.assert_allclose(pix_vels[c, g], pv, rtol=1e-5, atol=1e-6)
                ext = ext + np.abs(pv[:2]) * 0.5 * rs[c]
            else:
                assert (pix_vels[c, g] == 0).all()
            np.testing.assert_allclose(radii[c, g], ext, rtol=2e-5)
    assert n_valid > 100


def test_lidar_point_on_x_axis_closed_form():
    # az = el = 0 and J = [[0, k/x, 0], [0, 0, k/x], [1, 0, 0]], k = 180/pi
    x = 20.0
    means = np.array([[x, 0, 0]], np.float32)
    quats = np.array([[1, 0, 0, 0]], np.float32)
    scales = np.array([[0.5, 0.2, 0.1]], np.float32)
    vm = np.eye(4, dtype=np.float32)[None]
    zero = np.zeros((1, 3), np.float32)
    radii, m2, d, con, _, pv, dc = oracle.lidar_projection_fwd(
        means, None, quats, scales, None, vm, -45, 45, -180, 180, zero, zero,
        np.zeros(1, np.float32), eps2d=0.017, precision="f64")
    k = RAD2DEG / x
    s_az = (k * 0.2) ** 2 + 0.017
    s_el = (k * 0.1) ** 2 + 0.017
    np.testing.assert_allclose(m2[0, 0], [0, 0], atol=1e-12)
    np.testing.assert_allclose(d[0, 0], x)
    np.testing.assert_allclose(con[0, 0], [1 / s_az, 0, 1 / s_el], rtol=1e-6, atol=1e-12)
    np.testing.assert_allclose(radii[0, 0], [3 * math.sqrt(s_az), 3 * math.sqrt(s_el)], rtol=1e-6)
    np.testing.assert_allclose(dc[0, 0], [0, 0], atol=1e-12)  # axis-aligned: no range/angle coupling


def test_lidar_cull_rules():
    vm = np.eye(4, dtype=np.float32)[None]
    zero = np.zeros((1, 3), np.float32)
    quats = np.tile(np.array([[1, 0, 0, 0]], np.float32), (5, 1))
    scales = np.full((5, 3), 0.05, np.float32)
    means = np.array([
        [0.001, 0, 0],     # closer than near -> culled
        [500.0, 0, 0],     # beyond far=100 -> culled
        [10, 0, 30.0],     # elevation ~71.6 deg, above max_elevation=45 -> culled
        [10, 0, 0],        # visible
        [-10, 1, 0],       # azimuth ~174 deg, outside [-90, 90] -> culled
    ], np.float32)
    radii, *_ = oracle.lidar_projection_fwd(
        means, None, quats, scales, None, vm, -45, 45, -90, 90, zero, zero,
        np.zeros(1, np.float32), near_plane=0.01, far_plane=100.0, precision="f32")
    assert (radii[0, :, 0] > 0).tolist() == [False, False, False, True, False]


def test_f32_and_f64_builds_agree():
    C, N = 1, 2000
    rng, means, quats, scales, vel = _rand_scene(N, 3)
    viewmats, Ks = _cam(rng, C)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array([0.02], np.float32)
    a = oracle.projection_fwd(means, None, quats, scales, vel, viewmats, Ks, 320, 240, lin, ang,
                              rs, calc_compensations=True, precision="f32")
    b = oracle.projection_fwd(means, None, quats, scales, vel, viewmats, Ks, 320, 240, lin, ang,
                              rs, calc_compensations=True, precision="f64")
    valid = (a[0][..., 0] > 0) & (b[0][..., 0] > 0)
    assert valid.sum() > 500
    assert (np.abs(a[0] - b[0])[valid] <= 1).all()
    for x, y in zip(a[1:], b[1:]):
        np.testing.assert_allclose(x[valid], y[valid], rtol=2e-4, atol=2e-4)


def test_camera_fov_clamp_property():
    # Beyond the field-of-view limit the Jacobian is evaluated at the clamped ray
    # (utils.cuh:198-208): the projected covariance of a Gaussian at x/z = 3 equals that
    # of the same Gaussian moved to x/z = lim_x_pos, while the projected mean does not clamp.
    W, H, f, cx, cy, z = 320, 240, 300.0, 160.0, 120.0, 2.0
    lim = (W - cx) / f + 0.3 * (0.5 * W / f)
    K = np.array([[[f, 0, cx], [0, f, cy], [0, 0, 1]]], np.float32)
    vm = np.eye(4, dtype=np.float32)[None]
    zero = np.zeros((1, 3), np.float32)
    quats = np.array([[0.9, 0.1, 0.3, -0.2]] * 2, np.float32)
    scales = np.array([[3.0, 2.5, 2.0]] * 2, np.float32)   # big enough to still reach the image
    means = np.array([[3.0 * z, 0.1, z], [lim * z, 0.1, z]], np.float64).astype(np.float32)
    radii, m2, d, con, _, _ = oracle.projection_fwd(
        means, None, quats, scales, None, vm, K, W, H, zero, zero, np.zeros(1, np.float32),
        precision="f64")
    assert (radii[0, :, 0] > 0).all()
    np.testing.assert_allclose(con[0, 0], con[0, 1], rtol=1e-5)
    np.testing.assert_allclose(m2[0, 0, 0], f * 3.0 + cx, rtol=1e-6)
