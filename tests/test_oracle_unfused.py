"""Pins of the float64 torch restatements of the unfused projection operators
(oracle/torch_ref.py): library routines (scipy rotations, numpy inverses), finite differences
of the point maps, and composition into the fused projections that the C oracle pins."""
import numpy as np
import torch
from scipy.spatial.transform import Rotation

from oracle import torch_ref as T

torch.manual_seed(0)
F64 = dict(dtype=torch.float64)


def _gaussians(n):
    g = torch.Generator().manual_seed(3)
    means = torch.randn(n, 3, generator=g, **F64) * 2.0
    quats = torch.randn(n, 4, generator=g, **F64)
    scales = torch.rand(n, 3, generator=g, **F64) * 0.5 + 0.05
    return means, quats, scales


def _viewmats(C):
    rot = Rotation.from_euler("xyz", np.random.default_rng(1).uniform(-0.3, 0.3, (C, 3))).as_matrix()
    vm = torch.eye(4, **F64).repeat(C, 1, 1)
    vm[:, :3, :3] = torch.from_numpy(rot)
    vm[:, :3, 3] = torch.tensor([0.1, -0.2, 6.0], **F64)
    return vm


def test_quat_scale_to_covar_preci_against_scipy_and_inverse():
    _, quats, scales = _gaussians(50)
    covars, precis = T.quat_scale_to_covar_preci(quats, scales)
    q = quats.numpy()
    R = Rotation.from_quat(np.stack([q[:, 1], q[:, 2], q[:, 3], q[:, 0]], -1)).as_matrix()  # scipy: xyzw
    want = R @ (np.eye(3) * (scales.numpy() ** 2)[:, None, :]) @ R.transpose(0, 2, 1)
    np.testing.assert_allclose(covars.numpy(), want, atol=1e-12)
    np.testing.assert_allclose(precis.numpy(), np.linalg.inv(want), rtol=1e-9, atol=1e-9)
    c6, p6 = T.quat_scale_to_covar_preci(quats, scales, triu=True)
    iu = np.triu_indices(3)
    np.testing.assert_allclose(c6.numpy(), want[:, iu[0], iu[1]], atol=1e-12)
    assert T.quat_scale_to_covar_preci(quats, scales, compute_preci=False)[1] is None


def test_world_to_cam_against_numpy():
    means, quats, scales = _gaussians(20)
    covars, _ = T.quat_scale_to_covar_preci(quats, scales)
    vm = _viewmats(3)
    mc, cc = T.world_to_cam(means, covars, vm)
    for c in range(3):
        R, t = vm[c, :3, :3].numpy(), vm[c, :3, 3].numpy()
        np.testing.assert_allclose(mc[c].numpy(), means.numpy() @ R.T + t, atol=1e-12)
        np.testing.assert_allclose(cc[c].numpy(), R @ covars.numpy() @ R.T, atol=1e-12)


def _finite_difference(fn, p, h=1e-6):
    cols = []
    for k in range(3):
        d = torch.zeros(3, **F64); d[k] = h
        cols.append((fn(p + d) - fn(p - d)) / (2 * h))
    return torch.stack(cols, dim=-1)


def test_projection_jacobians_match_finite_differences():
    Ks = torch.tensor([[[300.0, 0, 160.0], [0, 310.0, 120.0], [0, 0, 1.0]]], **F64)
    p = torch.tensor([[[0.4, -0.3, 5.0], [-1.0, 0.8, 3.0]]], **F64)     # inside the field of view
    cov = torch.eye(3, **F64).expand(1, 2, 3, 3) * 0.01
    J = _finite_difference(lambda q: T.persp_proj(q, cov, Ks, 320, 240)[0], p)
    _, cov2 = T.persp_proj(p, cov, Ks, 320, 240)
    np.testing.assert_allclose(cov2.numpy(), (J @ cov @ J.transpose(-1, -2)).numpy(), rtol=1e-6, atol=1e-8)
    # pixel velocity of a static point under pure sensor translation v is -J v
    lin = torch.tensor([[1.0, -2.0, 0.5]], **F64)
    zero = torch.zeros_like(lin)
    pv = T.compute_pix_velocity(p, lin, zero, torch.zeros_like(p), Ks, 320, 240)
    np.testing.assert_allclose(pv.numpy(), -(J @ lin[0]).numpy(), rtol=1e-6, atol=1e-8)
    # lidar: (azimuth, elevation) in degrees
    Jl = _finite_difference(lambda q: T.lidar_proj(q, cov, 0.017)[0], p)
    _, cov2l, _ = T.lidar_proj(p, cov, 0.017)
    np.testing.assert_allclose(cov2l.numpy(), (Jl @ cov @ Jl.transpose(-1, -2)).numpy(), rtol=1e-6, atol=1e-8)
    lv = T.compute_lidar_velocity(p, lin, zero, torch.zeros_like(p))
    np.testing.assert_allclose(lv[..., :2].numpy(), -(Jl @ lin[0]).numpy(), rtol=1e-6, atol=1e-8)
    # third component: range rate, -v . p / |p|
    np.testing.assert_allclose(lv[..., 2].numpy(), -(p @ lin[0] / p.norm(dim=-1)).numpy(), rtol=1e-9)
    # angular part: omega x p
    ang = torch.tensor([[0.1, 0.2, -0.3]], **F64)
    pa = T.compute_pix_velocity(p, zero, ang, torch.zeros_like(p), Ks, 320, 240)
    want = -(J @ torch.cross(ang.expand(2, 3), p[0], dim=-1)[..., None])[..., 0]
    np.testing.assert_allclose(pa.numpy(), want.numpy(), rtol=1e-6, atol=1e-8)


def test_unfused_ops_compose_to_the_fused_projections():
    means, quats, scales = _gaussians(40)
    vm = _viewmats(2)
    Ks = torch.tensor([[300.0, 0, 160.0], [0, 300.0, 120.0], [0, 0, 1.0]], **F64).repeat(2, 1, 1)
    lin = torch.tensor([[1.0, 0.5, 0.2], [-0.3, 0.1, 2.0]], **F64)
    ang = torch.tensor([[0.05, -0.1, 0.02], [0.0, 0.2, 0.1]], **F64)
    rs = torch.tensor([0.03, 0.05], **F64)
    vel = torch.randn(40, 3, **F64)
    covars, _ = T.quat_scale_to_covar_preci(quats, scales)
    mc, cc = T.world_to_cam(means, covars, vm)
    vel_c = torch.einsum("cij,nj->cni", vm[:, :3, :3], vel)
    # camera
    m2, cov2 = T.persp_proj(mc, cc, Ks, 320, 240)
    conics, _ = T._blur_and_invert(cov2, 0.3)
    pv = T.compute_pix_velocity(mc, lin, ang, vel_c, Ks, 320, 240)
    f = T.projection_fwd(means, None, quats, scales, vel, vm, Ks, 320, 240, lin, ang, rs, eps2d=0.3)
    for got, want in ((m2, f[0]), (mc[..., 2], f[1]), (conics, f[2]), (pv, f[4])):
        np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-9, atol=1e-11)
    # lidar
    m2, cov2, dc = T.lidar_proj(mc, cc, 0.017)
    conics, _ = T._blur_and_invert(cov2, 0.017)
    lv = T.compute_lidar_velocity(mc, lin, ang, vel_c)
    f = T.lidar_projection_fwd(means, None, quats, scales, vel, vm, lin, ang, rs, eps2d=0.017)
    for got, want in ((m2, f[0]), (conics, f[2]), (lv, f[4]), (dc, f[5])):
        np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=1e-9, atol=1e-11)
