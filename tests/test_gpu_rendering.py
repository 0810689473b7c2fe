"""End-to-end GPU parity of rasterization() / lidar_rasterization() against the CPU oracle,
plus size-independent properties at the full benchmark sizes."""
import math

import numpy as np
import pytest
import torch

import oracle
from oracle import torch_ref
from splatad_amd import workloads
from tests.gpu_util import (DEV, assert_close, assert_matches_oracle_decisions, render_variants, to_dev,
                            to_np)
from tests.oracle_backend import OracleOps
from tests.test_gpu_forward import points_oracle

pytestmark = pytest.mark.gpu

T64 = lambda a: torch.from_numpy(np.ascontiguousarray(a)).double()


def _cam_scene(n=10000, rolling=True):
    s = workloads.camera_small(n=n)
    if rolling:
        s["linear_velocity"] = torch.tensor([[1.0, 0.5, 0.2]])
        s["angular_velocity"] = torch.tensor([[0.0, 0.1, 0.05]])
        s["rolling_shutter_time"] = torch.tensor([0.03])
    return s


def _render(s, dev_scene=None, **kw):
    from splatad_amd import rasterization
    d = dev_scene or workloads.to_device(s, DEV)
    return rasterization(d["means"], d["quats"], d["scales"], d["opacities"], d["colors"], d["velocities"],
                         d["viewmats"], d["Ks"], d["width"], d["height"], d["linear_velocity"],
                         d["angular_velocity"], d["rolling_shutter_time"], near_plane=d["near_plane"],
                         far_plane=d["far_plane"], eps2d=d["eps2d"], tile_size=d["tile_size"], **kw)


def _camera_stages_against_oracle(s, meta, rc, ra, C, packed=False, sh_degree=None, name="",
                                  max_attributed=1.5e-2):
    """Every stage behind the projection against the oracle on the GPU's own inputs to that
    stage: tile counts, sorted keys, flatten ids and offsets bit-exact; the render within 1e-4
    of the float64 oracle's composite of the same lists (depth channel: 1e-4 relative too),
    decided as tests.gpu_util.assert_matches_oracle_decisions describes."""
    m2, radii, depths = to_np(meta["means2d"]), to_np(meta["radii"]), to_np(meta["depths"])
    cam_ids = to_np(meta["camera_ids"]) if packed else None
    tw, th, ts = meta["tile_width"], meta["tile_height"], meta["tile_size"]
    o_tpg, o_ids, o_flat = oracle.isect_tiles(m2, radii, depths, ts, tw, th, n_cameras=C, camera_ids=cam_ids)
    np.testing.assert_array_equal(to_np(meta["tiles_per_gauss"]), o_tpg)
    np.testing.assert_array_equal(to_np(meta["isect_ids"]), o_ids)
    np.testing.assert_array_equal(to_np(meta["flatten_ids"]), o_flat)
    o_offs = oracle.isect_offset_encode(o_ids, C, tw, th)
    np.testing.assert_array_equal(to_np(meta["isect_offsets"]), o_offs)
    coeffs = s["colors"].numpy()
    if sh_degree is None:
        cols = coeffs[to_np(meta["gaussian_ids"])] if packed else np.broadcast_to(coeffs[None], (C,) + coeffs.shape)
    else:
        # colours: SH of the view directions, + 0.5, clamped (rendering.py:325-347)
        cam2world = np.linalg.inv(s["viewmats"].numpy().astype(np.float64))
        means = s["means"].numpy().astype(np.float64)
        if packed:
            gid = to_np(meta["gaussian_ids"])
            dirs = means[gid] - cam2world[cam_ids, :3, 3]
            sh = oracle.spherical_harmonics(sh_degree, dirs, coeffs[gid], None, "f64")
        else:
            dirs = means[None] - cam2world[:, None, :3, 3]
            sh = oracle.spherical_harmonics(sh_degree, dirs, np.broadcast_to(coeffs[None], (C,) + coeffs.shape),
                                            radii[..., 0] > 0, "f64")
        cols = np.maximum(sh + 0.5, 0.0)
    cols = np.concatenate([cols, depths[..., None]], -1).astype(np.float32)
    rs = s["rolling_shutter_time"]
    rs = np.zeros((C,), np.float32) if rs is None else rs.numpy()
    conics, opac, pv = to_np(meta["conics"]), to_np(meta["opacities"]), to_np(meta["pix_vels"])

    def render():
        o = oracle.rasterize_to_pixels_fwd(m2, conics, cols, opac, pv, rs, None, s["width"], s["height"], ts,
                                           o_offs, o_flat, precision="f64")
        return dict(render=o[0], alpha=o[1])

    return assert_matches_oracle_decisions(dict(render=to_np(rc), alpha=to_np(ra)), render_variants(render),
                                           dict(render=(1e-4, 1e-4), alpha=(1e-4, 0.0)), name=name,
                                           max_attributed=max_attributed)


@pytest.mark.parametrize("packed", [False, True])
def test_camera_small_config_against_oracle_pipeline(packed, monkeypatch):
    """10k Gaussians, 320x240 (the CPU-runnable benchmark configuration)."""
    s = _cam_scene()
    rc, ra, meta = _render(s, packed=packed, render_mode="RGB+D")
    # (1) every stage against the oracle on the GPU's own inputs to that stage
    _camera_stages_against_oracle(s, meta, rc, ra, 1, packed=packed, name="config 0")
    # (2) the whole call against the whole oracle pipeline (float32 oracle projection may cull
    # or truncate a boundary Gaussian differently: allow that on a sliver of the pixels)
    from splatad_amd import rasterization
    from splatad_amd.hip import _backend
    monkeypatch.setattr(_backend, "_C", OracleOps())
    e_rc, e_ra, e_meta = rasterization(s["means"], s["quats"], s["scales"], s["opacities"], s["colors"], None,
                                       s["viewmats"], s["Ks"], s["width"], s["height"], s["linear_velocity"],
                                       s["angular_velocity"], s["rolling_shutter_time"], packed=packed,
                                       render_mode="RGB+D")
    # (a Gaussian kept by one projection and culled by the other changes a pixel by at most
    # its alpha times its colour or depth, depths reach 5 here)
    assert_close(to_np(rc), e_rc.numpy(), atol=1e-4, rtol=1e-4, frac=0.999, outlier_bound=5.0,
                 name="render vs full oracle")
    assert_close(to_np(ra), e_ra.numpy(), atol=1e-4, frac=0.999, outlier_bound=1.0, name="alpha vs full oracle")
    assert abs(e_meta["flatten_ids"].shape[0] - meta["flatten_ids"].shape[0]) <= 20


def test_camera_render_modes_backgrounds_sh_and_determinism():
    s = workloads.camera_driving(n=20000, width=320, height=180, with_velocities=True)
    d = workloads.to_device(s, DEV)
    bg = torch.rand(1, 3, device=DEV)
    outs = {}
    for mode in ("RGB", "D", "ED", "RGB+D", "RGB+ED"):
        rc, ra, meta = _render(s, d, sh_degree=3, packed=False, render_mode=mode, backgrounds=bg)
        outs[mode] = (rc, ra)
        X = {"RGB": 3, "RGB+D": 4, "RGB+ED": 4, "D": 1, "ED": 1}[mode]
        assert rc.shape == (1, 180, 320, X)
    torch.testing.assert_close(outs["RGB+D"][0][..., :3], outs["RGB"][0], rtol=0, atol=1e-6)
    torch.testing.assert_close(outs["RGB+D"][0][..., 3:], outs["D"][0], rtol=0, atol=1e-5)
    ed = outs["D"][0] / outs["D"][1].clamp(min=1e-10)
    torch.testing.assert_close(outs["ED"][0], ed, rtol=1e-6, atol=1e-6)
    # bitwise reproducible
    again = _render(s, d, sh_degree=3, packed=False, render_mode="RGB+D", backgrounds=bg)
    assert torch.equal(again[0], outs["RGB+D"][0]) and torch.equal(again[1], outs["RGB+D"][1])
    # SH colours against the oracle
    cam2world = np.linalg.inv(s["viewmats"].numpy())
    dirs = s["means"].numpy()[None] - cam2world[:, None, :3, 3]
    _, _, meta = _render(s, d, sh_degree=3, packed=False)
    sh = oracle.spherical_harmonics(3, dirs, s["colors"].numpy()[None], to_np(meta["radii"])[..., 0] > 0, "f64")
    # packed and unpacked agree
    p = _render(s, d, sh_degree=3, packed=True, render_mode="RGB+D", backgrounds=bg)
    torch.testing.assert_close(p[0], outs["RGB+D"][0], rtol=0, atol=1e-5)
    # channel chunking agrees with one pass
    feat = torch.rand(20000, 40, device=DEV)
    from splatad_amd import rasterization
    a = rasterization(d["means"], d["quats"], d["scales"], d["opacities"], feat, None, d["viewmats"], d["Ks"],
                      320, 180, packed=False, channel_chunk=64)
    b = rasterization(d["means"], d["quats"], d["scales"], d["opacities"], feat, None, d["viewmats"], d["Ks"],
                      320, 180, packed=False, channel_chunk=16)
    torch.testing.assert_close(a[0], b[0], rtol=0, atol=1e-5)
    assert sh.shape == (1, 20000, 3)


@pytest.mark.parametrize("packed", [False, True])
def test_surround_cameras_small_against_oracle(packed):
    """Three yawed cameras over one set of Gaussians: every stage of the multi-camera call
    against the oracle on the GPU's own inputs to that stage."""
    C = 3
    s = workloads.camera_driving(n=20000, width=320, height=180, n_cameras=C, with_velocities=True)
    rc, ra, meta = _render(s, sh_degree=3, packed=packed, render_mode="RGB+D")
    assert rc.shape == (C, 180, 320, 4)
    _camera_stages_against_oracle(s, meta, rc, ra, C, packed=packed, sh_degree=3, name="surround")
    assert all(float(ra[c].max()) > 0.5 for c in range(C))  # every camera sees the scene


def _lidar(n=20000, D=8, **kw):
    l = workloads.lidar_sweep(n=n, n_beams=32, n_azimuth=512, feature_dim=D, tile_width=64, tile_height=4,
                              with_velocities=True, **kw)
    l["scales"] = l["scales"] * 2.0
    return l


def _lidar_render(d, **kw):
    from splatad_amd import lidar_rasterization
    return lidar_rasterization(
        d["means"], d["quats"], d["scales"], d["opacities"], d["lidar_features"], d["velocities"],
        d["viewmats"], d["raster_pts"], d["tile_elevation_boundaries"], d["linear_velocity"],
        d["angular_velocity"], d["rolling_shutter_time"], min_azimuth=d["min_azimuth"],
        max_azimuth=d["max_azimuth"], min_elevation=d["min_elevation"], max_elevation=d["max_elevation"],
        n_elevation_channels=d["n_elevation_channels"], azimuth_resolution=d["azimuth_resolution"],
        tile_width=d["tile_width"], tile_height=d["tile_height"], eps2d=d["eps2d"], **kw)


def _lidar_stages_against_oracle(l, d, meta, rf, ra, asum, name="", threshold=0.2, use_depth_compensation=True,
                                 max_attributed=1.5e-2):
    """The stages behind the lidar projection against the oracle on the GPU's own inputs: tile
    counts, sorted keys, flatten ids and offsets bit-exact; features, range, alpha, alpha sum
    and median depth against the float64 oracle's composite of the same lists."""
    from splatad_amd import fully_fused_lidar_projection
    tw, th = l["tile_width"], l["tile_height"]
    H, W = l["raster_pts"].shape[1:3]
    C = l["viewmats"].shape[0]
    res = np.float32(l["azimuth_resolution"] * tw)
    o = oracle.isect_lidar_tiles(to_np(meta["means2d"]), to_np(meta["radii"]), to_np(meta["depths"]),
                                 l["tile_elevation_boundaries"].numpy(), float(res), l["min_azimuth"])
    np.testing.assert_array_equal(to_np(meta["tiles_per_gauss"]), o[0])
    np.testing.assert_array_equal(to_np(meta["isect_ids"]), o[1])
    np.testing.assert_array_equal(to_np(meta["flatten_ids"]), o[2])
    gw, gh = meta["tile_grid_width"], meta["tile_grid_height"]
    o_offs = oracle.isect_offset_encode(o[1], C, gw, gh)
    np.testing.assert_array_equal(to_np(meta["isect_offsets"]), o_offs)
    dcomp = fully_fused_lidar_projection(  # the one projection output the meta does not carry
        d["means"], None, d["quats"], d["scales"], d["velocities"], d["viewmats"], d["linear_velocity"],
        d["angular_velocity"], d["rolling_shutter_time"], min_elevation=d["min_elevation"],
        max_elevation=d["max_elevation"], min_azimuth=d["min_azimuth"], max_azimuth=d["max_azimuth"],
        eps2d=d["eps2d"])[-1]
    if not use_depth_compensation:
        dcomp = dcomp * 0
    feats = torch.cat([d["lidar_features"].expand(C, -1, -1), meta["depths"][..., None]], -1)
    D = feats.shape[-1]
    variants = render_variants(lambda: points_oracle(
        meta["means2d"], meta["conics"], feats, meta["opacities"], meta["pix_vels"], dcomp, None,
        d["raster_pts"], W, H, tw, th, True, threshold, o_offs, o[2], D - 1), lidar=True)
    got = dict(features=to_np(rf), alphas=to_np(ra), alpha_sum=to_np(asum), median=to_np(meta["median_depths"]))
    tols = dict(features=(2e-4, 1e-4), alphas=(1e-4, 0.0), alpha_sum=(1e-4, 1e-4), median=(1e-3, 1e-4))
    return assert_matches_oracle_decisions(got, variants, tols, name=name, max_attributed=max_attributed)


def test_lidar_end_to_end_against_oracle(monkeypatch):
    l = _lidar()
    d = workloads.to_device(l, DEV)
    rf, ra, asum, meta = _lidar_render(d)
    assert rf.shape == (1, 32, 512, 9)
    _lidar_stages_against_oracle(l, d, meta, rf, ra, asum, name="lidar small")
    from splatad_amd import lidar_rasterization
    from splatad_amd.hip import _backend
    monkeypatch.setattr(_backend, "_C", OracleOps())
    e = lidar_rasterization(
        l["means"], l["quats"], l["scales"], l["opacities"], l["lidar_features"], l["velocities"],
        l["viewmats"], l["raster_pts"], l["tile_elevation_boundaries"], l["linear_velocity"],
        l["angular_velocity"], l["rolling_shutter_time"], min_azimuth=-180.0, max_azimuth=180.0,
        min_elevation=-26.0, max_elevation=16.0, n_elevation_channels=32,
        azimuth_resolution=l["azimuth_resolution"], tile_width=64, tile_height=4, eps2d=0.017)
    # the whole call against the whole float32 oracle pipeline: a Gaussian kept by one projection
    # and culled by the other moves a point by at most its alpha times its feature or range
    assert_close(to_np(rf), e[0].numpy(), atol=3e-4, rtol=1e-4, frac=0.999, outlier_bound=60.0, name="features")
    assert_close(to_np(ra), e[1].numpy(), atol=1e-4, frac=0.999, outlier_bound=1.0, name="alphas")
    assert_close(to_np(asum), e[2].numpy(), atol=1e-4, rtol=1e-4, frac=0.999, outlier_bound=1.0, name="alpha sum")
    assert_close(to_np(meta["median_depths"]), e[3]["median_depths"].numpy(), atol=1e-3, rtol=1e-4, frac=0.995,
                 outlier_bound=60.0, name="median")
    assert float(ra.max()) > 0.5


def test_camera_pipeline_gradients_end_to_end():
    """loss -> rasterize -> SH -> projection, against float64 autograd on the same tile lists."""
    s = workloads.camera_driving(n=3000, width=96, height=64, with_velocities=True, sh_degree=2)
    s["colors"] = s["colors"][:, :9]
    s["means"][:, 2] = s["means"][:, 2] * 0.2 + 3.0     # keep the scene close enough to cover pixels
    s["means"][:, :2] *= 0.1
    s["scales"] = s["scales"] * 0.5
    d = workloads.to_device(s, DEV)
    names = ("means", "quats", "scales", "opacities", "colors", "velocities")
    for k in names:
        d[k] = d[k].clone().requires_grad_()
    rc, ra, meta = _render(s, d, sh_degree=2, packed=False, render_mode="RGB+D")
    rng = np.random.default_rng(0)
    wc = rng.normal(size=tuple(rc.shape)).astype(np.float32)
    wa = rng.normal(size=tuple(ra.shape)).astype(np.float32)
    grads = torch.autograd.grad((rc * to_dev(wc)).sum() + (ra * to_dev(wa)).sum(), [d[k] for k in names])
    # float64 pipeline with the GPU's culling decisions and tile lists
    r = {k: T64(s[k].numpy()).requires_grad_() for k in names}
    m2, depths, conics, _, pv = torch_ref.projection_fwd(
        r["means"], None, r["quats"], r["scales"], r["velocities"], T64(s["viewmats"].numpy()),
        T64(s["Ks"].numpy()), 96, 64, T64(s["linear_velocity"].numpy()), T64(s["angular_velocity"].numpy()),
        T64(s["rolling_shutter_time"].numpy()), eps2d=0.3)
    c2w = torch.inverse(T64(s["viewmats"].numpy()))
    dirs = r["means"][None] - c2w[:, None, :3, 3]
    cols = torch.clamp_min(torch_ref.spherical_harmonics(2, dirs, r["colors"][None]) + 0.5, 0.0)
    cols = torch.cat([cols, depths[..., None]], -1)
    o_rc, o_ra = torch_ref.rasterize_to_pixels(m2, conics, cols, r["opacities"][None], pv,
                                               T64(s["rolling_shutter_time"].numpy()), None, 96, 64, 16,
                                               meta["isect_offsets"].cpu(), meta["flatten_ids"].cpu())
    assert_close(to_np(rc), o_rc.detach().numpy(), atol=2e-4, rtol=1e-4, name="render")
    ref = torch.autograd.grad((o_rc * T64(wc)).sum() + (o_ra * T64(wa)).sum(), [r[k] for k in names])
    from tests.test_gpu_backward import assert_grad_close
    for k, a, b in zip(names, grads, ref):
        assert_grad_close(to_np(a), b.numpy(), k)
    # the densification hook: absgrad lands on meta["means2d"], which is a non-leaf of the graph
    rc, ra, meta = _render(s, d, sh_degree=2, packed=True, absgrad=True)
    meta["means2d"].retain_grad()
    rc.sum().backward()
    assert meta["means2d"].grad is not None and meta["means2d"].absgrad.shape == meta["means2d"].shape
    assert (meta["means2d"].absgrad >= meta["means2d"].grad.abs() - 1e-6).all()


def test_lidar_pipeline_gradients_end_to_end():
    l = _lidar(n=3000, D=4)
    d = workloads.to_device(l, DEV)
    names = ("means", "quats", "scales", "opacities", "lidar_features", "velocities")
    for k in names:
        d[k] = d[k].clone().requires_grad_()
    rf, ra, asum, meta = _lidar_render(d)
    rng = np.random.default_rng(0)
    wc = rng.normal(size=tuple(rf.shape)).astype(np.float32)
    wa = rng.normal(size=tuple(ra.shape)).astype(np.float32)
    ws = rng.normal(size=tuple(ra.shape)).astype(np.float32)
    loss = (rf * to_dev(wc)).sum() + (ra * to_dev(wa)).sum() + (asum * to_dev(ws)).sum()
    grads = torch.autograd.grad(loss, [d[k] for k in names])
    r = {k: T64(l[k].numpy()).requires_grad_() for k in names}
    m2, depths, conics, _, pv, dc = torch_ref.lidar_projection_fwd(
        r["means"], None, r["quats"], r["scales"], r["velocities"], T64(l["viewmats"].numpy()),
        T64(l["linear_velocity"].numpy()), T64(l["angular_velocity"].numpy()),
        T64(l["rolling_shutter_time"].numpy()), eps2d=0.017)
    feats = torch.cat([r["lidar_features"], depths[..., None]], -1)
    o = torch_ref.rasterize_to_points(m2, conics, feats, r["opacities"][None], pv, dc, None,
                                      T64(l["raster_pts"].numpy()), 64, 4, True, 0.2,
                                      meta["isect_offsets"].cpu(), meta["flatten_ids"].cpu(), 4)
    assert_close(to_np(rf), o[0].detach().numpy(), atol=3e-4, rtol=1e-4, name="features")
    ref = torch.autograd.grad((o[0] * T64(wc)).sum() + (o[1] * T64(wa)).sum() + (o[2] * T64(ws)).sum(),
                              [r[k] for k in names])
    from tests.test_gpu_backward import assert_grad_close
    for k, a, b in zip(names, grads, ref):
        assert_grad_close(to_np(a), b.numpy(), k)


def _check_isect_invariants(meta, C, n_tiles):
    ids = meta["isect_ids"]
    assert int(meta["tiles_per_gauss"].sum()) == ids.shape[0] == meta["flatten_ids"].shape[0]
    assert bool((ids[1:] >= ids[:-1]).all())
    offs = meta["isect_offsets"].reshape(-1).long()
    assert bool((offs[1:] >= offs[:-1]).all()) and int(offs[-1]) <= ids.shape[0]
    tb = int(n_tiles).bit_length()
    hi = ids >> 32
    lin = (hi >> tb) * n_tiles + (hi & ((1 << tb) - 1))
    counts = torch.bincount(lin, minlength=C * n_tiles)
    ends = torch.cat([offs[1:], torch.tensor([ids.shape[0]], device=offs.device)])
    assert torch.equal(ends - offs, counts)


def test_full_size_driving_camera_properties():
    """1M Gaussians, 1920x1080, SH degree 3, rolling shutter: properties that need no oracle."""
    s = workloads.camera_driving()
    d = workloads.to_device(s, DEV)
    rc, ra, meta = _render(s, d, sh_degree=3, packed=False, render_mode="RGB+D")
    assert rc.shape == (1, 1080, 1920, 4) and torch.isfinite(rc).all()
    assert float(ra.min()) >= 0.0 and float(ra.max()) <= 1.0 - 1e-4 + 1e-6
    _check_isect_invariants(meta, 1, meta["tile_width"] * meta["tile_height"])
    # compositing is linear in the colours: render(a) + render(b) == render(a + b)
    from splatad_amd import rasterize_to_pixels
    N = s["means"].shape[0]
    ca, cb = torch.rand(1, N, 3, device=DEV), torch.rand(1, N, 3, device=DEV)
    args = (meta["opacities"], meta["pix_vels"], 1920, 1080, 16, meta["isect_offsets"], meta["flatten_ids"])
    kw = dict(rolling_shutter_time=d["rolling_shutter_time"])
    ra_, _ = rasterize_to_pixels(meta["means2d"], meta["conics"], ca, *args, **kw)
    rb_, _ = rasterize_to_pixels(meta["means2d"], meta["conics"], cb, *args, **kw)
    rab, alpha_ab = rasterize_to_pixels(meta["means2d"], meta["conics"], ca + cb, *args, **kw)
    torch.testing.assert_close(ra_ + rb_, rab, rtol=1e-5, atol=2e-5)
    # with all colours equal to one the image is the accumulated alpha
    ones, a1 = rasterize_to_pixels(meta["means2d"], meta["conics"], torch.ones(1, N, 1, device=DEV), *args, **kw)
    torch.testing.assert_close(ones, a1, rtol=1e-5, atol=1e-5)
    # packed and unpacked agree
    p = _render(s, d, sh_degree=3, packed=True, render_mode="RGB+D")
    torch.testing.assert_close(p[0], rc, rtol=1e-5, atol=1e-4)
    assert p[2]["camera_ids"].shape[0] == int((meta["radii"][..., 0] > 0).sum())


def test_full_size_lidar_sweep_properties():
    """1M Gaussians, 128 x 2048 lidar sweep with 32 features."""
    l = workloads.lidar_sweep()
    d = workloads.to_device(l, DEV)
    rf, ra, asum, meta = _lidar_render(d, channel_chunk=33)
    assert rf.shape == (1, 128, 2048, 33) and torch.isfinite(rf).all()
    assert float(ra.min()) >= 0.0 and float(ra.max()) <= 1.0
    assert float(asum.min()) >= 0.0
    _check_isect_invariants(meta, 1, meta["tile_grid_width"] * meta["tile_grid_height"])
    # two chunks (31 features + range, 1 feature + range) reproduce the single pass
    rf2, ra2, asum2, meta2 = _lidar_render(d, channel_chunk=32)
    torch.testing.assert_close(rf2, rf, rtol=1e-5, atol=1e-4)
    torch.testing.assert_close(ra2, ra, rtol=0, atol=1e-6)
    assert meta2["median_depths"].shape[-1] == 2
    # expected range lies between the nearest and the farthest Gaussian range where opaque
    opaque = ra[..., 0] > 0.99
    rng_ch = rf[..., -1][opaque]
    assert float(rng_ch.min()) > 0.0 and float(rng_ch.max()) < 60.0
    # the reference's chunk loop spelled out (rendering.py:733-771): concatenated chunks of 31
    # features + range, the range kept from the last chunk only
    from splatad_amd import fully_fused_lidar_projection, rasterize_to_points
    dcomp = fully_fused_lidar_projection(  # the one projection output the meta does not carry
        d["means"], None, d["quats"], d["scales"], d["velocities"], d["viewmats"], d["linear_velocity"],
        d["angular_velocity"], d["rolling_shutter_time"], min_elevation=d["min_elevation"],
        max_elevation=d["max_elevation"], min_azimuth=d["min_azimuth"], max_azimuth=d["max_azimuth"],
        eps2d=d["eps2d"])[-1]
    feats_out = []
    for i in range(2):
        chunk = torch.cat([d["lidar_features"][..., i * 31:(i + 1) * 31], meta["depths"][..., None]], -1)
        out = rasterize_to_points(meta["means2d"], meta["conics"], chunk, meta["opacities"], meta["pix_vels"],
                                  dcomp, d["raster_pts"], 2048, 128, d["tile_width"],
                                  d["tile_height"], meta["isect_offsets"], meta["flatten_ids"], True, 0.3)
        feats_out.append(out[0] if i == 1 else out[0][..., :-1])
        torch.testing.assert_close(out[1], ra2, rtol=0, atol=1e-6)
    torch.testing.assert_close(torch.cat(feats_out, -1), rf2, rtol=1e-5, atol=1e-4)


def test_full_size_surround_rig_properties():
    """2M Gaussians, six 1920x1080 cameras around the sensor in one call, and a lidar sweep
    over the same number of Gaussians: each camera's image equals the image of a call with that
    camera alone, and the lists keep their invariants with camera bits in the keys."""
    C = 6
    s = workloads.camera_driving(n=2_000_000, n_cameras=C)
    d = workloads.to_device(s, DEV)
    rc, ra, meta = _render(s, d, sh_degree=3, packed=False, render_mode="RGB+D")
    assert rc.shape == (C, 1080, 1920, 4) and torch.isfinite(rc).all()
    _check_isect_invariants(meta, C, meta["tile_width"] * meta["tile_height"])
    for c in (0, 3, 5):
        one = dict(d)
        for k in ("viewmats", "Ks", "linear_velocity", "angular_velocity", "rolling_shutter_time"):
            one[k] = d[k][c:c + 1].contiguous()
        rc1, ra1, meta1 = _render(s, one, sh_degree=3, packed=False, render_mode="RGB+D")
        assert torch.equal(rc1[0], rc[c]) and torch.equal(ra1[0], ra[c])
        assert float(ra1.max()) > 0.5
    del rc, ra, meta
    l = workloads.lidar_sweep(n=2_000_000)
    rf, la, asum, lmeta = _lidar_render(workloads.to_device(l, DEV), channel_chunk=33)
    assert rf.shape == (1, 128, 2048, 33) and torch.isfinite(rf).all()
    _check_isect_invariants(lmeta, 1, lmeta["tile_grid_width"] * lmeta["tile_grid_height"])


def test_camera_antialiased_packed_sparse_grad_end_to_end():
    """rasterize_mode="antialiased" (opacities scaled by the blur compensation, rendering.py:286-287),
    packed=True with sparse_grad=True (COO gradients, _wrapper.py:2256-2296), end to end on the
    HIP path: compensated opacities and every later stage against the oracle; the sparse gradients
    equal the dense ones of the same call."""
    s = workloads.camera_driving(n=20000, width=320, height=180, with_velocities=True)
    d = workloads.to_device(s, DEV)
    rc, ra, meta = _render(s, d, sh_degree=3, packed=True, render_mode="RGB+D", rasterize_mode="antialiased")
    npy = lambda k: s[k].numpy()
    o = oracle.projection_fwd(npy("means"), None, npy("quats"), npy("scales"), npy("velocities"), npy("viewmats"),
                              npy("Ks"), 320, 180, npy("linear_velocity"), npy("angular_velocity"),
                              npy("rolling_shutter_time"), eps2d=0.3, calc_compensations=True, precision="f64")
    gid = to_np(meta["gaussian_ids"])
    assert_close(to_np(meta["opacities"]), npy("opacities")[gid] * o[4][0][gid], atol=1e-4, rtol=1e-4,
                 name="compensated opacities")
    plain = _render(s, d, sh_degree=3, packed=True, render_mode="RGB+D")
    assert float((plain[2]["opacities"] - meta["opacities"]).abs().max()) > 1e-3  # the mode does something
    _camera_stages_against_oracle(s, meta, rc, ra, 1, packed=True, sh_degree=3, name="antialiased")
    # sparse gradients
    names = ("means", "quats", "scales")
    rng = np.random.default_rng(3)
    w = to_dev(rng.normal(size=tuple(rc.shape)).astype(np.float32))
    grads = {}
    for sparse in (False, True):
        p = dict(d)
        for k in names:
            p[k] = d[k].clone().requires_grad_()
        out = _render(s, p, sh_degree=3, packed=True, render_mode="RGB+D", rasterize_mode="antialiased",
                      sparse_grad=sparse)
        grads[sparse] = torch.autograd.grad((out[0] * w).sum(), [p[k] for k in names])
    from tests.test_gpu_backward import assert_grad_close
    for k, dense, sp in zip(names, grads[False], grads[True]):
        # the means also reach the image through the view directions of the colours, whose
        # gradient is dense; rotations and scales only through the projection
        assert not dense.is_sparse and (sp.is_sparse or k == "means")
        assert_grad_close(to_np(sp.to_dense() if sp.is_sparse else sp), to_np(dense), k)


def test_lidar_without_depth_compensation_end_to_end():
    """use_depth_compensation=False (rendering.py:704-705) on the HIP path against the oracle."""
    l = _lidar()
    d = workloads.to_device(l, DEV)
    rf, ra, asum, meta = _lidar_render(d, use_depth_compensation=False)
    _lidar_stages_against_oracle(l, d, meta, rf, ra, asum, name="no depth compensation",
                                 use_depth_compensation=False)
    with_dc = _lidar_render(d)
    assert float((with_dc[0][..., -1] - rf[..., -1]).abs().max()) > 1e-3  # the switch does something
    assert torch.equal(with_dc[0][..., :-1], rf[..., :-1])


@pytest.mark.parametrize("opts", [
    dict(sh_degree=3, render_mode="RGB"), dict(sh_degree=0, render_mode="RGB+ED"),
    dict(sh_degree=None, render_mode="RGB+D"), dict(sh_degree=2, render_mode="D"),
    dict(sh_degree=3, render_mode="RGB+D", rasterize_mode="antialiased", radius_clip=2.0),
    dict(sh_degree=1, render_mode="ED", tile_size=8), dict(sh_degree=3, render_mode="RGB", per_sensor=True)])
def test_surround_packed_equals_unpacked_for_every_option(opts):
    """What the packed call makes beside the sort (rows, opacities, colours) feeds the same
    compositing kernel as the unpacked call's tensors: the renders are equal bit for bit, with
    gradients switched off and with them switched on (where the opacities come from a gather
    that autograd sees)."""
    from splatad_amd import rasterization
    opts = dict(opts)
    s = workloads.camera_driving(n=20000, width=320, height=180, n_cameras=3, with_velocities=True)
    d = workloads.to_device(s, DEV)
    C, N = d["viewmats"].shape[0], d["means"].shape[0]
    colors = d["colors"]
    if opts.get("sh_degree") is None:
        colors = torch.rand((N, 3), device=DEV, generator=torch.Generator(device=DEV).manual_seed(5))
    elif opts.pop("per_sensor", False):
        colors = colors[None].expand(C, -1, -1, -1).contiguous() * torch.linspace(0.5, 1.5, C, device=DEV).view(C, 1, 1, 1)
    opts.pop("per_sensor", None)
    bg = torch.rand((C, 3 if "RGB" in opts["render_mode"] else 1), device=DEV,
                    generator=torch.Generator(device=DEV).manual_seed(6))
    if opts["render_mode"] in ("D", "ED"):
        bg = None
    kw = dict(near_plane=d["near_plane"], far_plane=d["far_plane"], eps2d=d["eps2d"],
              tile_size=opts.pop("tile_size", d["tile_size"]), backgrounds=bg, **opts)
    args = (d["means"], d["quats"], d["scales"], d["opacities"], colors, d["velocities"], d["viewmats"], d["Ks"],
            d["width"], d["height"], d["linear_velocity"], d["angular_velocity"], d["rolling_shutter_time"])
    with torch.no_grad():
        dense = rasterization(*args, packed=False, **kw)
        packed = rasterization(*args, packed=True, **kw)
    assert torch.equal(dense[0], packed[0]) and torch.equal(dense[1], packed[1])
    assert float(dense[1].max()) > 0.5  # something was rendered
    sel = dense[2]["radii"][..., 0] > 0
    assert torch.equal(dense[2]["opacities"].expand(C, N)[sel], packed[2]["opacities"])
    # gradients on: the same images again
    leaves = [t.clone().requires_grad_() for t in (d["means"], d["opacities"])]
    packed_grad = rasterization(leaves[0], d["quats"], d["scales"], leaves[1], *args[4:], packed=True, **kw)
    assert torch.equal(packed_grad[0].detach(), dense[0]) and torch.equal(packed_grad[1].detach(), dense[1])


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("sh", [False, True])
def test_helper_stream_switch_renders_the_same(packed, sh, monkeypatch):
    """rendering.HELPER_STREAM (off by default) moves the colour kernel, the packed rows and their
    opacities to a helper stream beside the tile intersection: same images and gradients."""
    import splatad_amd.rendering as rendering
    s = workloads.camera_driving(n=20000, width=320, height=180, n_cameras=2, sh_degree=3 if sh else None)
    d = workloads.to_device(s, DEV)
    kw = dict(near_plane=d["near_plane"], far_plane=d["far_plane"], eps2d=d["eps2d"], tile_size=16,
              sh_degree=3 if sh else None, render_mode="RGB+D", packed=packed)
    rest = (d["velocities"], d["viewmats"], d["Ks"], d["width"], d["height"], d["linear_velocity"],
            d["angular_velocity"], d["rolling_shutter_time"])
    out = {}
    for helper in (False, True):
        monkeypatch.setattr(rendering, "HELPER_STREAM", helper)
        leaves = [d[k].clone().requires_grad_() for k in ("means", "opacities", "colors")]
        rc, ra, _ = rendering.rasterization(leaves[0], d["quats"], d["scales"], leaves[1], leaves[2], *rest, **kw)
        (rc.sum() + 2.0 * ra.sum()).backward()
        torch.cuda.synchronize()
        out[helper] = (rc.detach(), ra.detach(), [t.grad for t in leaves])
    assert torch.equal(out[False][0], out[True][0]) and torch.equal(out[False][1], out[True][1])
    # (the backward kernels add with float atomics, so two runs differ in the last bits anyway)
    for a, b in zip(out[False][2], out[True][2]):
        torch.testing.assert_close(a, b, rtol=1e-3, atol=1e-3 * float(a.abs().max()))


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("case", ["behind", "between_tiles"])
def test_camera_frames_without_rows_or_without_intersections(packed, case):
    """Nothing in front of the camera (no packed rows at all), and Gaussians that are kept by the
    projection but meet no tile (pushed outside the image after it): empty lists, a render of
    the background, no alpha; the packed path's helper-stream work has nothing to write."""
    from splatad_amd import rasterization
    s = _cam_scene(n=2000)
    d = workloads.to_device(s, DEV)
    if case == "behind":
        d["means"] = d["means"].clone()
        d["means"][:, 2] = -torch.abs(d["means"][:, 2]) - 100.0  # behind every near plane
    bg = torch.tensor([[0.25, 0.5, 0.75]], device=DEV)
    kw = dict(near_plane=d["near_plane"], far_plane=d["far_plane"], eps2d=d["eps2d"], tile_size=d["tile_size"],
              packed=packed, sh_degree=s["sh_degree"], backgrounds=bg, render_mode="RGB")
    W, H = d["width"], d["height"]
    if case == "between_tiles":
        # a sliver of an image: the few Gaussians the projection keeps are culled again by ...
        # nothing here; instead ask for an image that no Gaussian of the scene reaches
        Ks = d["Ks"].clone()
        Ks[:, 0, 2] += 1.0e6  # principal point far to the right: all means project outside
        d = dict(d, Ks=Ks)
    for _ in range(2):
        rc, ra, meta = rasterization(d["means"], d["quats"], d["scales"], d["opacities"], d["colors"],
                                     d["velocities"], d["viewmats"], d["Ks"], W, H, d["linear_velocity"],
                                     d["angular_velocity"], d["rolling_shutter_time"], **kw)
        torch.cuda.synchronize()
        assert meta["isect_ids"].numel() == 0 and meta["flatten_ids"].numel() == 0
        assert int(meta["tiles_per_gauss"].sum().item()) == 0
        assert int(meta["isect_offsets"].abs().sum().item()) == 0
        if packed:
            assert meta["camera_ids"].numel() == meta["radii"].shape[0] == meta["means2d"].shape[0]
        assert torch.equal(ra, torch.zeros_like(ra))
        assert torch.allclose(rc, bg.view(1, 1, 1, 3).expand_as(rc))


def test_two_host_threads_on_two_streams():
    """The boundary is callable from several host threads, each on a stream of its own: two
    threads render cameras (packed and unpacked: both counting calls) and lidar sweeps at the
    same time, several times over; every result equals the single-threaded one bit for bit."""
    import threading
    s = workloads.camera_driving(n=60000, width=640, height=360, with_velocities=True)
    d = workloads.to_device(s, DEV)
    l = _lidar(n=40000)
    dl = workloads.to_device(l, DEV)
    jobs = {"packed": lambda: _render(s, d, sh_degree=3, packed=True, render_mode="RGB+D")[:2],
            "unpacked": lambda: _render(s, d, sh_degree=3, packed=False, render_mode="RGB+D")[:2],
            "lidar": lambda: _lidar_render(dl)[:3]}
    with torch.no_grad():
        want = {k: f() for k, f in jobs.items()}
    torch.cuda.synchronize()
    errors = []

    def worker(order, rounds):
        try:
            stream = torch.cuda.Stream(device=DEV)
            stream.wait_stream(torch.cuda.default_stream(DEV))
            with torch.no_grad(), torch.cuda.stream(stream):
                for r in range(rounds):
                    for k in order:
                        got = jobs[k]()
                        stream.synchronize()
                        for a, b in zip(got, want[k]):
                            if not torch.equal(a, b):
                                errors.append(f"{k} round {r}: result differs from the single-threaded one")
        except Exception as e:  # noqa: BLE001 -- reported to the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(o, 4)) for o in
               (("packed", "lidar", "unpacked"), ("lidar", "unpacked", "packed"))]
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors


def test_packed_multi_camera_backward_is_reproducible_within_rounding():
    """packed=True with several cameras sums a Gaussian's gradients over the cameras that see it
    with float atomics (gathers by index_select, SH coefficient gradients added in the kernel):
    two runs may differ in the order of those sums, by rounding only."""
    from splatad_amd import rasterization
    s = workloads.camera_driving(n=30000, width=320, height=180, n_cameras=3)
    d = workloads.to_device(s, DEV)
    runs = []
    for _ in range(2):
        leaves = [d[k].clone().requires_grad_() for k in ("means", "quats", "scales", "opacities", "colors")]
        rc, ra, _ = rasterization(*leaves, d["velocities"], d["viewmats"], d["Ks"], d["width"], d["height"],
                                  d["linear_velocity"], d["angular_velocity"], d["rolling_shutter_time"],
                                  near_plane=d["near_plane"], far_plane=d["far_plane"], eps2d=d["eps2d"],
                                  sh_degree=3, render_mode="RGB+D", packed=True)
        (rc * rc).sum().backward()
        torch.cuda.synchronize()
        runs.append((rc.detach(), [t.grad for t in leaves]))
    assert torch.equal(runs[0][0], runs[1][0])  # the forward pass is bitwise repeatable
    for name, a, b in zip(("means", "quats", "scales", "opacities", "colors"), runs[0][1], runs[1][1]):
        scale = float(a.abs().max())
        assert scale > 0
        # a few units in the last place of the largest summands
        assert float((a - b).abs().max()) <= 2e-5 * scale, (name, float((a - b).abs().max()), scale)
