"""GPU parity of the unfused projection operators (forward values and gradients) against
the float64 torch restatement in oracle/torch_ref.py, the way the reference's own tests
compare them with its torch implementation (tests/test_basic.py:97-352)."""
import numpy as np
import pytest
import torch

from oracle import torch_ref as T
from tests.gpu_util import DEV, to_np
from tests.test_gpu_backward import assert_grad_close

pytestmark = pytest.mark.gpu


def _scene(C=3, N=4000, seed=0):
    from scipy.spatial.transform import Rotation
    rng = np.random.default_rng(seed)
    d = {}
    d["means"] = rng.uniform(-1.5, 1.5, (N, 3))
    d["quats"] = rng.normal(size=(N, 4))
    d["scales"] = np.exp(rng.normal(size=(N, 3)) * 0.4 - 2.0)
    vm = np.tile(np.eye(4), (C, 1, 1))
    for c in range(C):
        vm[c, :3, :3] = Rotation.from_rotvec(rng.normal(size=3) * 0.2).as_matrix()
        vm[c, :3, 3] = np.array([0.1, -0.1, 4.0]) + rng.normal(size=3) * 0.1
    d["viewmats"] = vm
    d["Ks"] = np.tile(np.array([[300.0, 0, 160.0], [0, 290.0, 120.0], [0, 0, 1.0]]), (C, 1, 1))
    d["lin_vel"] = rng.normal(size=(C, 3)) * 3
    d["ang_vel"] = rng.normal(size=(C, 3)) * 0.2
    d["vel_view"] = rng.normal(size=(C, N, 3))
    return {k: torch.from_numpy(v).double() for k, v in d.items()}


def _pair(t, grad=True):
    """(float32 GPU leaf, float64 CPU leaf) of one tensor"""
    g = t.float().to(DEV).requires_grad_(grad)
    r = t.clone().requires_grad_(grad)
    return g, r


def _check(outs_gpu, outs_ref, leaves_gpu, leaves_ref, names, seed=0, atol=1e-4, rtol=1e-4):
    gen = torch.Generator().manual_seed(seed)
    loss_g, loss_r = 0.0, 0.0
    for og, orf, n in zip(outs_gpu, outs_ref, names):
        ref = orf.detach().numpy()
        # float32 results: the absolute floor scales with the size of the tensor's entries
        floor = atol * max(1.0, float(np.sqrt((ref ** 2).mean())))
        np.testing.assert_allclose(to_np(og), ref, atol=floor, rtol=rtol, err_msg=n)
        w = torch.randn(orf.shape, generator=gen, dtype=torch.float64)
        loss_g = loss_g + (og * w.float().to(DEV)).sum()
        loss_r = loss_r + (orf * w).sum()
    loss_g.backward()
    loss_r.backward()
    for lg, lr in zip(leaves_gpu, leaves_ref):
        assert lg.grad is not None
        assert_grad_close(to_np(lg.grad), lr.grad.numpy(), "gradient")


@pytest.mark.parametrize("triu", [False, True])
@pytest.mark.parametrize("which", ["both", "covar", "preci"])
def test_quat_scale_to_covar_preci(triu, which):
    from splatad_amd import quat_scale_to_covar_preci
    s = _scene()
    qg, qr = _pair(s["quats"]); sg, sr = _pair(s["scales"])
    cc, cp = which != "preci", which != "covar"
    og = quat_scale_to_covar_preci(qg, sg, compute_covar=cc, compute_preci=cp, triu=triu)
    orf = T.quat_scale_to_covar_preci(qr, sr, compute_covar=cc, compute_preci=cp, triu=triu)
    assert (og[0] is None) == (not cc) and (og[1] is None) == (not cp)
    keep = [i for i in (0, 1) if og[i] is not None]
    # precisions reach 1 / 0.03^2: relative tolerance
    _check([og[i] for i in keep], [orf[i] for i in keep], [qg, sg], [qr, sr],
           ["covars", "precis"], atol=1e-5, rtol=1e-4)


def test_world_to_cam():
    from splatad_amd import world_to_cam
    s = _scene()
    cov = T.quat_scale_to_covar_preci(s["quats"], s["scales"])[0].detach()
    mg, mr = _pair(s["means"]); cg, cr = _pair(cov); vg, vr = _pair(s["viewmats"])
    _check(world_to_cam(mg, cg, vg), T.world_to_cam(mr, cr, vr), [mg, cg, vg], [mr, cr, vr],
           ["means_c", "covars_c"])
    # gradients only where asked for
    mg2 = s["means"].float().to(DEV)
    cg2, _ = _pair(cov)
    out = world_to_cam(mg2, cg2, s["viewmats"].float().to(DEV))
    out[1].sum().backward()
    assert cg2.grad is not None


def _sensor_frame(s):
    cov = T.quat_scale_to_covar_preci(s["quats"], s["scales"])[0]
    mc, cc = T.world_to_cam(s["means"], cov, s["viewmats"])
    return mc.detach(), cc.detach()


def test_persp_proj_and_pix_velocity():
    from splatad_amd import compute_pix_velocity, persp_proj
    s = _scene()
    mc, cc = _sensor_frame(s)
    mc[:, :200, 0] *= 4.0        # some points outside the field of view: clamped Jacobian
    mg, mr = _pair(mc); cg, cr = _pair(cc)
    Kg = s["Ks"].float().to(DEV)
    _check(persp_proj(mg, cg, Kg, 320, 240), T.persp_proj(mr, cr, s["Ks"], 320, 240), [mg, cg], [mr, cr],
           ["means2d", "covars2d"], atol=2e-3, rtol=1e-4)
    pg, pr = _pair(mc); vg, vr = _pair(s["vel_view"])
    out_g = compute_pix_velocity(pg, s["lin_vel"].float().to(DEV), s["ang_vel"].float().to(DEV), vg, Kg, 320, 240)
    out_r = T.compute_pix_velocity(pr, s["lin_vel"], s["ang_vel"], vr, s["Ks"], 320, 240)
    _check([out_g], [out_r], [pg, vg], [pr, vr], ["pix_vel"], atol=2e-3, rtol=1e-4)


def test_lidar_proj_and_lidar_velocity():
    from splatad_amd import compute_lidar_velocity, lidar_proj
    s = _scene()
    mc, cc = _sensor_frame(s)
    mg, mr = _pair(mc); cg, cr = _pair(cc)
    _check(lidar_proj(mg, cg, 0.017), T.lidar_proj(mr, cr, 0.017), [mg, cg], [mr, cr],
           ["means2d", "covars2d", "depth_compensations"], atol=1e-3, rtol=1e-3)
    pg, pr = _pair(mc); vg, vr = _pair(s["vel_view"])
    out_g = compute_lidar_velocity(pg, s["lin_vel"].float().to(DEV), s["ang_vel"].float().to(DEV), vg)
    out_r = T.compute_lidar_velocity(pr, s["lin_vel"], s["ang_vel"], vr)
    _check([out_g], [out_r], [pg, vg], [pr, vr], ["lidar_vel"], atol=1e-3, rtol=1e-4)


def test_unfused_ops_handle_empty_inputs():
    from splatad_amd import persp_proj, quat_scale_to_covar_preci, world_to_cam
    z = lambda *shape: torch.zeros(shape, device=DEV)
    c, p = quat_scale_to_covar_preci(z(0, 4), z(0, 3))
    assert c.shape == (0, 3, 3) and p.shape == (0, 3, 3)
    mc, cc = world_to_cam(z(0, 3), z(0, 3, 3), torch.eye(4, device=DEV)[None])
    assert mc.shape == (1, 0, 3) and cc.shape == (1, 0, 3, 3)
    m2, c2 = persp_proj(mc, cc, torch.eye(3, device=DEV)[None], 10, 10)
    assert m2.shape == (1, 0, 2) and c2.shape == (1, 0, 2, 2)
