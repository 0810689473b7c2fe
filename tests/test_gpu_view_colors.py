"""GPU parity of the fused view-dependent colour operator.

The operator stands for a chain of tensor operations of the reference's pipeline
(gsplat/rendering.py:325-351): inverse view matrices -> directions -> masks ->
spherical_harmonics -> max(c + 1/2, 0) -> depth channel.  It is checked against the CPU oracle
evaluated on directions from numpy.linalg.inv (values, 1e-4) and against that chain built from
torch operations and the separately tested `spherical_harmonics` operator (gradients, 1e-3).
"""
import numpy as np
import pytest
import torch

import oracle
from tests.gpu_util import DEV, assert_close, to_dev, to_np
from tests.test_gpu_backward import assert_grad_close

pytestmark = pytest.mark.gpu


def _scene(C, N, K, seed, per_sensor):
    rng = np.random.default_rng(seed)
    means = rng.normal(size=(N, 3)).astype(np.float32) * 3
    viewmats = np.tile(np.eye(4, dtype=np.float32), (C, 1, 1))
    for c in range(C):
        q, _ = np.linalg.qr(rng.normal(size=(3, 3)))
        viewmats[c, :3, :3] = q * np.sign(np.linalg.det(q))
        viewmats[c, :3, 3] = rng.normal(size=3) * 2
    viewmats[0, :3, :3] *= 1.3  # not a rigid motion: the general inverse is needed
    coeffs = rng.normal(size=((C, N, K, 3) if per_sensor else (N, K, 3))).astype(np.float32) * 0.5
    radii = rng.integers(0, 3, size=(C, N, 2)).astype(np.int32)
    depths = rng.uniform(1, 9, (C, N)).astype(np.float32)
    return means, viewmats, coeffs, radii, depths


def _chain(degree, means, viewmats, coeffs, radii, depths, camera_ids=None, gaussian_ids=None):
    from splatad_amd import spherical_harmonics
    C = viewmats.shape[0]
    camtoworlds = torch.inverse(viewmats)
    masks = radii[..., 0] > 0
    if camera_ids is not None:
        dirs = means[gaussian_ids] - camtoworlds[camera_ids, :3, 3]
        shs = coeffs[gaussian_ids] if coeffs.dim() == 3 else coeffs[camera_ids, gaussian_ids]
    else:
        dirs = means[None] - camtoworlds[:, None, :3, 3]
        shs = coeffs.expand(C, -1, -1, -1) if coeffs.dim() == 3 else coeffs
    colors = torch.clamp_min(spherical_harmonics(degree, dirs, shs, masks=masks) + 0.5, 0.0)
    return colors if depths is None else torch.cat([colors, depths[..., None]], -1)


@pytest.mark.parametrize("C,degree,K,per_sensor,with_depth",
                         [(1, 3, 16, False, True), (3, 3, 16, False, True), (2, 4, 25, True, False),
                          (2, 0, 4, False, False), (3, 2, 16, True, True)])
def test_view_colors_unpacked(C, degree, K, per_sensor, with_depth):
    from splatad_amd.hip._wrapper import view_dependent_colors
    N = 3000
    means, viewmats, coeffs, radii, depths = _scene(C, N, K, 10 + C + degree, per_sensor)
    leaves = [to_dev(a).requires_grad_() for a in (means, coeffs, depths)]
    ref_leaves = [to_dev(a).requires_grad_() for a in (means, coeffs, depths)]
    vm, rd = to_dev(viewmats), to_dev(radii)
    out = view_dependent_colors(degree, leaves[0], vm, leaves[1], rd, leaves[2] if with_depth else None)
    ref = _chain(degree, ref_leaves[0], vm, ref_leaves[1], rd, ref_leaves[2] if with_depth else None)
    assert out.shape == (C, N, 4 if with_depth else 3)
    # oracle: float64 SH on directions from numpy's inverse
    pos = np.linalg.inv(viewmats.astype(np.float64))[:, :3, 3]
    dirs = means[None].astype(np.float64) - pos[:, None]
    shs = coeffs if per_sensor else np.broadcast_to(coeffs, (C,) + coeffs.shape)
    o = oracle.spherical_harmonics(degree, dirs.astype(np.float32), np.ascontiguousarray(shs),
                                   radii[..., 0] > 0, precision="f64")
    want = np.maximum(o + 0.5, 0.0)
    if with_depth:
        want = np.concatenate([want, depths[..., None]], -1)
    assert_close(to_np(out), want, atol=1e-4, name="colours")
    assert (to_np(out)[radii[..., 0] <= 0][:, :3] == 0.5).all()
    rng = np.random.default_rng(0)
    w = to_dev(rng.normal(size=tuple(out.shape)).astype(np.float32))
    n_leaf = 3 if with_depth else 2
    g = torch.autograd.grad((out * w).sum(), leaves[:n_leaf])
    g_ref = torch.autograd.grad((ref * w).sum(), ref_leaves[:n_leaf])
    for name, a, b in zip(("means", "coeffs", "depths"), g, g_ref):
        assert_grad_close(to_np(a), to_np(b), name)


@pytest.mark.parametrize("per_sensor", [False, True])
def test_view_colors_packed(per_sensor):
    from splatad_amd.hip._wrapper import view_dependent_colors
    C, N, K, degree = 3, 2000, 16, 3
    means, viewmats, coeffs, radii, depths = _scene(C, N, K, 33, per_sensor)
    cam, gid = np.nonzero(radii[..., 0] > 0)
    keep = np.random.default_rng(1).uniform(size=cam.shape[0]) < 0.7
    cam, gid = cam[keep], gid[keep]
    rd, dp = radii[cam, gid], depths[cam, gid]
    rd[::17, 0] = 0  # packed rows are normally all visible; inactive ones must still give 1/2
    cam_t, gid_t, rd_t, vm = to_dev(cam), to_dev(gid), to_dev(rd), to_dev(viewmats)
    leaves = [to_dev(a).requires_grad_() for a in (means, coeffs, dp)]
    ref_leaves = [to_dev(a).requires_grad_() for a in (means, coeffs, dp)]
    out = view_dependent_colors(degree, leaves[0], vm, leaves[1], rd_t, leaves[2], cam_t, gid_t)
    ref = _chain(degree, ref_leaves[0], vm, ref_leaves[1], rd_t, ref_leaves[2], cam_t, gid_t)
    assert out.shape == (cam.shape[0], 4)
    assert_close(to_np(out), to_np(ref), atol=1e-4, name="colours")
    w = to_dev(np.random.default_rng(2).normal(size=tuple(out.shape)).astype(np.float32))
    g = torch.autograd.grad((out * w).sum(), leaves)
    g_ref = torch.autograd.grad((ref * w).sum(), ref_leaves)
    for name, a, b in zip(("means", "coeffs", "depths"), g, g_ref):
        assert_grad_close(to_np(a), to_np(b), name)


@pytest.mark.parametrize("C,degree,K,packed", [(1, 3, 16, False), (2, 2, 16, False), (2, 3, 16, True)])
def test_view_colors_gradients_where_stretches_of_rows_take_none(C, degree, K, packed):
    """Rows that no pixel composited have a zero colour gradient; a workgroup (256 rows) that
    holds only such rows writes its zeros on a path of its own.  The cotangent here is zero on
    stretches longer than a workgroup, beside stretches that are not; also with fewer bases in
    use than the coefficient rows hold (degree 2 of 16)."""
    from splatad_amd.hip._wrapper import view_dependent_colors
    N = 3000
    means, viewmats, coeffs, radii, depths = _scene(C, N, K, 71 + degree, False)
    radii[...] = np.maximum(radii, 1)
    vm = to_dev(viewmats)
    if packed:
        cam, gid = np.nonzero(radii[..., 0] > 0)
        rd, dp = radii[cam, gid], depths[cam, gid]
        ids = (to_dev(cam), to_dev(gid))
    else:
        rd, dp, ids = radii, depths, ()
    rd_t = to_dev(rd)
    leaves = [to_dev(a).requires_grad_() for a in (means, coeffs, dp)]
    ref_leaves = [to_dev(a).requires_grad_() for a in (means, coeffs, dp)]
    out = view_dependent_colors(degree, leaves[0], vm, leaves[1], rd_t, leaves[2], *ids)
    ref = _chain(degree, ref_leaves[0], vm, ref_leaves[1], rd_t, ref_leaves[2], *ids)
    w = np.random.default_rng(5).normal(size=tuple(out.shape)).astype(np.float32)
    flat = w.reshape(-1, w.shape[-1])
    flat[:700, :3] = 0
    flat[1500:2300, :3] = 0
    flat[2600:, :3] = 0  # the last, partial workgroup
    w = to_dev(w)
    g = torch.autograd.grad((out * w).sum(), leaves)
    g_ref = torch.autograd.grad((ref * w).sum(), ref_leaves)
    for name, a, b in zip(("means", "coeffs", "depths"), g, g_ref):
        assert_grad_close(to_np(a), to_np(b), name)
    if not packed and C == 1:  # rows without a gradient get exact zeros
        assert (to_np(g[1])[:700] == 0).all() and (to_np(g[1])[1500:2300] == 0).all()
        assert (to_np(g[0])[:700] == 0).all()
