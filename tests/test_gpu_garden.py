"""The reference's own operator tests on its own fixture, with the CPU oracle as comparator.

Data: tests/golden/garden_subset.npz, cut from the reference's assets/test_garden.npz by
tests/golden/make_garden_subset.py (every third point of the [-2, 2]^3 crop its loader keeps,
gsplat/_helper.py:9-36; the three real 648x420 cameras unchanged).  The reference draws scales,
rotations and opacities from the GPU's generator without a seed (gsplat/_helper.py:51-53), so
those are drawn here from seeded CPU generators with the same distributions, and so are the
sensor velocities and lidar parameters of its test fixture (tests/test_basic.py:20-55).

Recipes and tolerances follow tests/test_basic.py: test_projection (:284-396),
test_lidar_projection with the scene scaled by 100 and the camera-to-lidar axis swap (:564-694),
test_isect on projected data (:697-723 is exact), test_rasterize_to_pixels with 3 / 32 / 64
channels (:891-1010), test_rasterize_to_points (:1013-1197).  Where the reference compares its
CUDA kernels with its float32 torch code, these compare the HIP kernels with the float64 oracle
under the same rtol / atol.
"""
import math
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref
from tests.gpu_util import (DEV, assert_matches_oracle_decisions, render_variants, to_dev, to_np)
from tests.test_gpu_forward import points_oracle

pytestmark = pytest.mark.gpu

T64 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).double()
GARDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "garden_subset.npz")


def ref_close(got, want, rtol, atol, name, flips=0, near_rows=None):
    """torch.testing.assert_close of the reference's tests: |got - want| <= atol + rtol |want|
    on every element.  The reference composites its torch comparison over the index lists its
    CUDA kernels emit, so both sides of its rasterizer tests share every alpha >= 1/255
    decision; the float64 comparator here decides for itself, and a (pixel, Gaussian) pair it
    keeps where float32 drops it moves the gradient row of that Gaussian (all its channels).
    `flips` such rows (or two in 100 000, whichever is more) may exceed the tolerance, by a
    bounded amount.  With `near_rows` (the comparator's own list of the Gaussians that have a
    pair within 1e-4 relative of the threshold at a pixel still compositing, or are composited
    at a pixel with such a pair: the transmittance in front of them or the colour accumulated
    behind them hinges on it there, by 0.4 %) the rows are not counted but attributed: a row
    outside that list must meet the tolerance, no exception."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, (name, got.shape, want.shape)
    if got.size == 0:
        return
    tol = atol + rtol * np.abs(want)
    err = np.abs(got - want)
    over = err > tol
    if over.ndim > 2:
        over = over.any(-1)  # [C, N, k] -> rows: a flipped pair moves every channel of its Gaussian
    if near_rows is not None:
        near_rows = np.asarray(near_rows, bool).reshape(over.shape)
        stray = over & ~near_rows
        assert not stray.any(), (
            f"{name}: {int(stray.sum())} rows off with no decision near the threshold "
            f"(first {np.argwhere(stray)[0].tolist()}); {int(near_rows.sum())} rows have one")
        flips = int(near_rows.sum())
    else:
        flips = max(flips, int(2e-5 * over.size)) if flips else 0
    # a flipped pair moves an entry by that pair's own share, alpha ~ 1/255 of the largest
    # shares in the tensor
    assert over.sum() <= flips and (err <= 20 * tol + 0.05 * np.abs(want).max()).all(), (
        f"{name}: {int(over.sum())}/{over.size} rows off (allowed {flips}), worst excess {(err - tol).max():.3e}")


@pytest.fixture(scope="module")
def garden():
    data = np.load(GARDEN)  # allow_pickle=False
    g = torch.Generator().manual_seed(42)
    means = torch.from_numpy(data["means3d"]).float()
    N, C = means.shape[0], data["viewmats"].shape[0]
    rnd = lambda *sh: torch.rand(*sh, generator=g)
    rndn = lambda *sh: torch.randn(*sh, generator=g)
    quats = rndn(N, 4)
    return dict(
        means=means, colors=torch.from_numpy(data["colors"] / 255.0).float(),
        scales=rnd(N, 3) * 0.02, quats=quats / quats.norm(dim=-1, keepdim=True), opacities=rnd(N),
        viewmats=torch.from_numpy(data["viewmats"]).float(), Ks=torch.from_numpy(data["Ks"]).float(),
        width=int(data["width"]), height=int(data["height"]),
        min_azimuth=-180.0, max_azimuth=180.0, min_elevation=-45 - 1e-2, max_elevation=45 + 1e-2,
        velocities=rndn(N, 3) * 0.1, linear_velocity=rndn(C, 3) * 0.5, angular_velocity=rndn(C, 3) * 0.1,
        rolling_shutter_time=torch.ones(C) * 0.01, n_elev_channels=32, tile_height=4, tile_width=64,
        azim_resolution=0.2)


def _grads(loss, leaves):
    return [to_np(t) if t.is_cuda else t.numpy() for t in torch.autograd.grad(loss, leaves)]


@pytest.mark.parametrize("calc_compensations", [False, True])
@pytest.mark.parametrize("use_velocities", [False, True])
def test_garden_projection(garden, calc_compensations, use_velocities):
    from splatad_amd import fully_fused_projection
    t = garden
    W, H = t["width"], t["height"]
    vel = t["velocities"] if use_velocities else None
    leaves = [to_dev(t[k].numpy()).requires_grad_() for k in ("viewmats", "quats", "scales", "means")]
    vm, q, s, m = leaves
    radii, means2d, depths, conics, comps, pix_vels = fully_fused_projection(
        m, None, q, s, None if vel is None else to_dev(vel.numpy()), vm, to_dev(t["Ks"].numpy()), W, H,
        to_dev(t["linear_velocity"].numpy()), to_dev(t["angular_velocity"].numpy()),
        to_dev(t["rolling_shutter_time"].numpy()), calc_compensations=calc_compensations)
    npy = lambda k: t[k].numpy()
    o = oracle.projection_fwd(npy("means"), None, npy("quats"), npy("scales"), None if vel is None else vel.numpy(),
                              npy("viewmats"), npy("Ks"), W, H, npy("linear_velocity"), npy("angular_velocity"),
                              npy("rolling_shutter_time"), calc_compensations=calc_compensations, precision="f64")
    valid = (to_np(radii)[..., 0] > 0) & (o[0][..., 0] > 0)
    assert valid.sum() > 20000 and ((to_np(radii)[..., 0] > 0) == (o[0][..., 0] > 0)).mean() > 0.999
    ref_close(to_np(radii)[valid], o[0][valid], 0, 1, "radii")
    ref_close(to_np(means2d)[valid], o[1][valid], 1e-4, 1e-4, "means2d")
    ref_close(to_np(depths)[valid], o[2][valid], 1e-4, 1e-4, "depths")
    ref_close(to_np(conics)[valid], o[3][valid], 1e-4, 1e-4, "conics")
    if calc_compensations:
        ref_close(to_np(comps)[valid], o[4][valid], 1e-4, 1e-3, "compensations")
    ref_close(to_np(pix_vels)[valid], o[5][valid], 1e-4, 1e-4, "pix_vels")

    # backward: random cotangents on the valid rows, float64 autograd as the comparator
    g = torch.Generator().manual_seed(1)
    vmask = torch.from_numpy(valid)
    rleaves = [T64(t[k].numpy()).requires_grad_() for k in ("viewmats", "quats", "scales", "means")]
    r = torch_ref.projection_fwd(rleaves[3], None, rleaves[1], rleaves[2], None if vel is None else T64(vel.numpy()),
                                 rleaves[0], T64(npy("Ks")), W, H, T64(npy("linear_velocity")),
                                 T64(npy("angular_velocity")), T64(npy("rolling_shutter_time")))
    loss_g, loss_r = 0.0, 0.0
    pairs = [(means2d, r[0]), (depths, r[1]), (conics, r[2]), (pix_vels, r[4])]
    if calc_compensations:
        pairs.append((comps, r[3]))
    for got, want in pairs:
        w = torch.randn(tuple(got.shape), generator=g) * (vmask if got.dim() == 2 else vmask[..., None])
        loss_g = loss_g + (got * to_dev(w.numpy())).sum()
        loss_r = loss_r + (want * w.double()).sum()
    gv, gq, gs, gm = _grads(loss_g, leaves)
    rv, rq, rs_, rm = _grads(loss_r, rleaves)
    ref_close(gv, rv, 1e-3, 1e-3 * max(1.0, np.abs(rv).max() * 1e-3), "v_viewmats")
    ref_close(gq, rq, 2e-1, 1e-2, "v_quats")
    ref_close(gs, rs_, 1e-1, 2e-1, "v_scales")
    ref_close(gm, rm, 1e-2, 6e-2, "v_means")


def _lidar_pose_and_scene(t, rescale=100.0):
    """tests/test_basic.py:573-590: the cameras become lidars through an axis swap (x right, y
    down, z forward -> x forward, y left, z up comes out of rot), the scene grows by 100."""
    world2cam = t["viewmats"].double()
    lidar2cam = torch.eye(4, dtype=torch.float64).expand(len(world2cam), -1, -1).clone()
    lidar2cam[:, :3, :3] = torch.tensor([[1.0, 0, 0], [0, 0, -1], [0, 1, 0]], dtype=torch.float64)
    world2lidar = lidar2cam.inverse() @ world2cam
    lidar2world = world2lidar.inverse()
    lidar2world[:, :3, 3] *= rescale
    return lidar2world.inverse().float(), t["scales"] * rescale, t["means"] * rescale


@pytest.mark.parametrize("calc_compensations", [False, True])
@pytest.mark.parametrize("use_velocities", [True, False])
def test_garden_lidar_projection(garden, calc_compensations, use_velocities):
    from splatad_amd import fully_fused_lidar_projection
    t = garden
    viewmats, scales, means = _lidar_pose_and_scene(t)
    vel = t["velocities"] if use_velocities else None
    leaves = [to_dev(a.numpy()).requires_grad_() for a in (viewmats, t["quats"], scales, means)]
    vm, q, s, m = leaves
    lim = (t["min_elevation"], t["max_elevation"], t["min_azimuth"], t["max_azimuth"])
    out = fully_fused_lidar_projection(
        m, None, q, s, None if vel is None else to_dev(vel.numpy()), vm, to_dev(t["linear_velocity"].numpy()),
        to_dev(t["angular_velocity"].numpy()), to_dev(t["rolling_shutter_time"].numpy()), *lim,
        calc_compensations=calc_compensations)
    radii, means2d, depths, conics, comps, pix_vels, dcomp = out
    o = oracle.lidar_projection_fwd(means.numpy(), None, t["quats"].numpy(), scales.numpy(),
                                    None if vel is None else vel.numpy(), viewmats.numpy(), *lim,
                                    t["linear_velocity"].numpy(), t["angular_velocity"].numpy(),
                                    t["rolling_shutter_time"].numpy(), calc_compensations=calc_compensations,
                                    precision="f64")
    valid = (to_np(radii)[..., 0] > 0) & (o[0][..., 0] > 0)
    assert valid.sum() > 20000 and ((to_np(radii)[..., 0] > 0) == (o[0][..., 0] > 0)).mean() > 0.999
    ref_close(to_np(radii)[valid], o[0][valid], 1e-4, 1e-4, "radii")
    ref_close(to_np(means2d)[valid], o[1][valid], 1e-4, 1e-4, "means2d")
    ref_close(to_np(depths)[valid], o[2][valid], 1e-4, 1e-4, "depths")
    ref_close(to_np(conics)[valid], o[3][valid], 1e-3, 1e-3, "conics")
    if calc_compensations:
        ref_close(to_np(comps)[valid], o[4][valid], 1e-3, 2e-3, "compensations")
    ref_close(to_np(pix_vels)[valid], o[5][valid], 2e-4, 1e-4, "pix_vels")
    ref_close(to_np(dcomp)[valid], o[6][valid], 1e-1, 1e-2, "depth_compensations")

    g = torch.Generator().manual_seed(2)
    vmask = torch.from_numpy(valid)
    rleaves = [T64(a.numpy()).requires_grad_() for a in (viewmats, t["quats"], scales, means)]
    r = torch_ref.lidar_projection_fwd(rleaves[3], None, rleaves[1], rleaves[2],
                                       None if vel is None else T64(vel.numpy()), rleaves[0],
                                       T64(t["linear_velocity"].numpy()), T64(t["angular_velocity"].numpy()),
                                       T64(t["rolling_shutter_time"].numpy()), eps2d=0.01)
    loss_g, loss_r = 0.0, 0.0
    pairs = [(means2d, r[0]), (depths, r[1]), (conics, r[2]), (pix_vels, r[4]), (dcomp, r[5])]
    if calc_compensations:
        pairs.append((comps, r[3]))
    for got, want in pairs:
        w = torch.randn(tuple(got.shape), generator=g) * (vmask if got.dim() == 2 else vmask[..., None])
        loss_g = loss_g + (got * to_dev(w.numpy())).sum()
        loss_r = loss_r + (want * w.double()).sum()
    gv, gq, gs, gm = _grads(loss_g, leaves)
    rv, rq, rs_, rm = _grads(loss_r, rleaves)
    ref_close(gv, rv, 1e-2, 1e-3 * max(1.0, np.abs(rv).max() * 1e-3), "v_viewmats")
    ref_close(gq, rq, 2e-1, 1e-1, "v_quats")
    ref_close(gs, rs_, 2e-1, 5e-1, "v_scales")
    ref_close(gm, rm, 1e-2, 6e-2, "v_means")


def _project_cameras(t, scale=1.0):
    from splatad_amd import fully_fused_projection, quat_scale_to_covar_preci
    covars, _ = quat_scale_to_covar_preci(to_dev(t["quats"].numpy()), to_dev((t["scales"] * scale).numpy()),
                                          compute_preci=False, triu=True)
    return fully_fused_projection(
        to_dev(t["means"].numpy()), covars, None, None, to_dev(t["velocities"].numpy()),
        to_dev(t["viewmats"].numpy()), to_dev(t["Ks"].numpy()), t["width"], t["height"],
        to_dev(t["linear_velocity"].numpy()), to_dev(t["angular_velocity"].numpy()),
        to_dev(t["rolling_shutter_time"].numpy()))


def test_garden_isect_on_projected_scene(garden):
    """Tile lists of the three real cameras: exact, as tests/test_basic.py:720-723 demands."""
    from splatad_amd import isect_offset_encode, isect_tiles
    t = garden
    radii, means2d, depths, _, _, _ = _project_cameras(t)
    for ts in (16, 4):
        tw, th = math.ceil(t["width"] / ts), math.ceil(t["height"] / ts)
        got = isect_tiles(means2d, radii, depths, ts, tw, th)
        want = oracle.isect_tiles(to_np(means2d), to_np(radii), to_np(depths), ts, tw, th)
        for a, b in zip(got, want):
            np.testing.assert_array_equal(to_np(a), b)
        np.testing.assert_array_equal(to_np(isect_offset_encode(got[1], 3, tw, th)),
                                      oracle.isect_offset_encode(want[1], 3, tw, th))
        assert want[1].shape[0] > 30000


@pytest.mark.parametrize("channels", [3, 32, 64])
def test_garden_rasterize_to_pixels(garden, channels):
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_pixels
    t = garden
    C, W, H = 3, t["width"], t["height"]
    # the 64-channel case of the reference shrinks the Gaussians tenfold and uses 4x4 tiles; one
    # camera of it keeps the float64 per-tile autograd comparator within a minute
    if channels == 64:
        t = dict(t, viewmats=t["viewmats"][:1], Ks=t["Ks"][:1], linear_velocity=t["linear_velocity"][:1],
                 angular_velocity=t["angular_velocity"][:1], rolling_shutter_time=t["rolling_shutter_time"][:1])
        C = 1
    radii, means2d, depths, conics, _, pix_vels = _project_cameras(t, scale=0.1)
    g = torch.Generator().manual_seed(42)
    N = t["means"].shape[0]
    colors = torch.randn(C, N, channels, generator=g)
    backgrounds = torch.rand(C, channels, generator=g)
    opac = t["opacities"].repeat(C, 1)
    ts = 16 if channels <= 32 else 4
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    _, ids, flat = isect_tiles(means2d, radii, depths, ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    rs = to_dev(t["rolling_shutter_time"].numpy())
    leaves = [x.detach().clone().requires_grad_() for x in
              (means2d, conics, to_dev(colors.numpy()), to_dev(opac.numpy()), pix_vels, to_dev(backgrounds.numpy()))]
    rc, ra = rasterize_to_pixels(leaves[0], leaves[1], leaves[2], leaves[3], leaves[4], W, H, ts, offs, flat,
                                 rolling_shutter_time=rs, backgrounds=leaves[5])
    base = [to_np(x) for x in leaves]

    def render():
        o = oracle.rasterize_to_pixels_fwd(base[0], base[1], base[2], base[3], base[4], to_np(rs), base[5], W, H,
                                           ts, to_np(offs), to_np(flat), precision="f64")
        return dict(colors=o[0], alphas=o[1])

    assert_matches_oracle_decisions(dict(colors=to_np(rc), alphas=to_np(ra)), render_variants(render),
                                    dict(colors=(1e-4, 1e-4), alphas=(1e-4, 1e-4)), name=f"garden {channels} ch")
    assert float(ra.detach().max()) > 0.5
    gen = torch.Generator().manual_seed(7)
    v_c, v_a = torch.randn(tuple(rc.shape), generator=gen), torch.randn(tuple(ra.shape), generator=gen)
    tiles = None
    if ts == 4:
        # 17 000 tiles of 4x4 pixels: the float64 per-tile comparator takes a sample of 2000, the
        # cotangents are zero on the other tiles
        tiles = set(torch.randperm(C * tw * th, generator=gen)[:2000].tolist())
        mask = torch.zeros(C, th * ts, tw * ts, 1)
        for t_ in tiles:
            c_, r_ = divmod(t_, tw * th)
            mask[c_, (r_ // tw) * ts:(r_ // tw + 1) * ts, (r_ % tw) * ts:(r_ % tw + 1) * ts] = 1.0
        v_c, v_a = v_c * mask[:, :H, :W], v_a * mask[:, :H, :W]
    got = _grads((rc * to_dev(v_c.numpy())).sum() + (ra * to_dev(v_a.numpy())).sum(), leaves)
    rl = [T64(x).requires_grad_() for x in base]
    near = {"margin": 1e-4}  # float32 alpha (a polynomial in tile coordinates) is good to a few 1e-5 relative
    r_rc, r_ra = torch_ref.rasterize_to_pixels(rl[0], rl[1], rl[2], rl[3], rl[4], T64(to_np(rs)), rl[5], W, H, ts,
                                               offs.cpu(), flat.cpu(), tiles=tiles, near=near)
    near_rows = near["rows"].numpy().reshape(C, -1)
    # a plausibility bound on the list itself: a window of 2e-4 around the threshold (a few
    # dozen pairs) and the Gaussians that share those pixels
    assert near_rows.sum() <= max(100, 3e-2 * near_rows.size), int(near_rows.sum())
    want = _grads((r_rc * v_c.double()).sum() + (r_ra * v_a.double()).sum(), rl)
    tol = dict(v_means2d=5e-3, v_conics=1e-3, v_colors=1e-3, v_opacities=2e-3, v_pix_vels=1e-3, v_backgrounds=1e-3)
    for (name, e), a, b in zip(tol.items(), got, want):
        # v_backgrounds sums a cotangent over every pixel of an image: its atol scales with the
        # float32 rounding of that sum
        atol = e * max(1.0, np.abs(b).max() * 1e-2) if name == "v_backgrounds" else e
        ref_close(a, b, e, atol, name, flips=3, near_rows=None if name == "v_backgrounds" else near_rows)


@pytest.mark.parametrize("compute_alpha_sum_until_points", [False, True])
@pytest.mark.parametrize("use_depth_compensations", [False, True])
def test_garden_rasterize_to_points(garden, compute_alpha_sum_until_points, use_depth_compensations):
    from splatad_amd import (fully_fused_lidar_projection, isect_lidar_tiles, isect_offset_encode,
                             quat_scale_to_covar_preci, rasterize_to_points)
    t = garden
    C = 3
    g = torch.Generator().manual_seed(42)
    lim = (t["min_elevation"], t["max_elevation"], t["min_azimuth"], t["max_azimuth"])
    tile_h, tile_w, n_ch, az_res = t["tile_height"], t["tile_width"], t["n_elev_channels"], t["azim_resolution"]
    elev = torch.linspace(lim[0], lim[1], n_ch)
    n_elev_tiles = n_ch // tile_h
    eb = torch.linspace(lim[0] - 1e-2, lim[1] + 1e-2, n_elev_tiles + 1)
    H, W = n_ch, math.ceil(360 / az_res)
    az = torch.linspace(lim[2] + az_res / 2, lim[3] - az_res / 2, W)
    tile_az_res = az_res * tile_w
    n_az_tiles = math.ceil(360 / tile_az_res)
    ae = torch.stack(torch.meshgrid(elev, az, indexing="ij"), dim=-1)[..., [1, 0]]
    ranges = torch.rand(H, W, 1, generator=g) * 10
    keep = torch.rand(H, W, generator=g) > 0.1
    pts = torch.cat([ae, ranges], -1)[None].repeat(C, 1, 1, 1)
    pts = pts + torch.randn(pts.shape, generator=g) * 0.01 * keep[None, ..., None]
    pts = torch.cat([pts, 0.01 * torch.randn(pts[..., :1].shape, generator=g)], -1).contiguous()
    N = t["means"].shape[0]
    feats = torch.randn(C, N, 5, generator=g) * float(ranges.max()) * 1.5
    feats[..., -1] = torch.rand(C, N, generator=g) * float(ranges.max()) * 1.5
    covars, _ = quat_scale_to_covar_preci(to_dev(t["quats"].numpy()), to_dev(t["scales"].numpy()),
                                          compute_preci=False, triu=True)
    rs = to_dev(t["rolling_shutter_time"].numpy())
    radii, means2d, depths, conics, _, pix_vels, dcomp = fully_fused_lidar_projection(
        to_dev(t["means"].numpy()), covars, None, None, to_dev(t["velocities"].numpy()),
        to_dev(t["viewmats"].numpy()), to_dev(t["linear_velocity"].numpy()), to_dev(t["angular_velocity"].numpy()),
        rs, *lim, eps2d=0.0)
    _, ids, flat = isect_lidar_tiles(means2d, radii, depths, to_dev(eb.numpy()), tile_az_res, lim[2])
    o_isect = oracle.isect_lidar_tiles(to_np(means2d), to_np(radii), to_np(depths), eb.numpy(), tile_az_res, lim[2])
    np.testing.assert_array_equal(to_np(ids), o_isect[1])
    np.testing.assert_array_equal(to_np(flat), o_isect[2])
    offs = isect_offset_encode(ids, C, n_az_tiles, n_elev_tiles)
    dcomp = dcomp * float(use_depth_compensations)
    opac = to_dev(t["opacities"].repeat(C, 1).numpy())
    pts_d = to_dev(pts.numpy())
    leaves = [x.detach().clone().requires_grad_() for x in
              (means2d, conics, to_dev(feats.numpy()), opac, pix_vels, dcomp)]
    rf, ra, asum, med = rasterize_to_points(*leaves, pts_d, W, H, tile_w, tile_h, offs, flat,
                                            compute_alpha_sum_until_points=compute_alpha_sum_until_points,
                                            compute_alpha_sum_until_points_threshold=0.5)
    variants = render_variants(lambda: points_oracle(
        *[x.detach() for x in leaves], None, pts_d, W, H, tile_w, tile_h, compute_alpha_sum_until_points, 0.5,
        offs, flat, 4), lidar=True)
    got = dict(features=to_np(rf), alphas=to_np(ra))
    tols = dict(features=(2e-2, 1e-2), alphas=(1e-3, 1e-3))
    if compute_alpha_sum_until_points:
        got["alpha_sum"] = to_np(asum)
        tols["alpha_sum"] = (1e-3, 1e-3)
    assert_matches_oracle_decisions(got, variants, tols, name="garden points")
    assert float(ra.detach().max()) > 0.5
    gen = torch.Generator().manual_seed(9)
    v_f, v_a = torch.randn(tuple(rf.shape), generator=gen), torch.randn(tuple(ra.shape), generator=gen)
    v_s = torch.randn(tuple(ra.shape), generator=gen)
    loss = (rf * to_dev(v_f.numpy())).sum() + (ra * to_dev(v_a.numpy())).sum()
    if compute_alpha_sum_until_points:
        loss = loss + (asum * to_dev(v_s.numpy())).sum()
    g_got = _grads(loss, leaves)
    rl = [T64(to_np(x)).requires_grad_() for x in leaves]
    r = torch_ref.rasterize_to_points(*rl, None, T64(pts.numpy()), tile_w, tile_h, compute_alpha_sum_until_points,
                                      0.5, offs.cpu(), flat.cpu(), 4)
    r_loss = (r[0] * v_f.double()).sum() + (r[1] * v_a.double()).sum()
    if compute_alpha_sum_until_points:
        r_loss = r_loss + (r[2] * v_s.double()).sum()
    g_want = _grads(r_loss, rl)
    for name, a, b in zip(("v_means2d", "v_conics", "v_features", "v_opacities", "v_pix_vels", "v_depth_comp"),
                          g_got, g_want):
        ref_close(a, b, 5e-2, 5e-2, name, flips=3)
