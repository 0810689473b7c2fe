"""GPU parity of the forward operators against the CPU oracle (same seeded inputs).

Bars: tile intersection lists, sort order and offsets bit-exact; projected and rendered
floats within 1e-4 (absolute, plus 1e-4 relative where values reach hundreds of pixels);
radii exact up to the truncation of a float that differs in its last bits (|diff| <= 1 on
<0.1% of rows).
"""
import math

import numpy as np
import pytest
import torch

import oracle
from tests.gpu_util import (DEV, assert_close, assert_matches_oracle_decisions, render_variants, to_dev,
                            to_np)

# Rendered values are compared with tests.gpu_util.assert_matches_oracle_decisions: 1e-4 on
# every pixel whose float64 oracle value does not hinge on a decision (alpha >= 1/255,
# transmittance <= 1e-4, ...) within a few float32 rounding errors of its threshold; the
# pixels that do hinge on one must equal the oracle's render for one of the two outcomes.

pytestmark = pytest.mark.gpu


def _gaussians(n, seed, spread=2.0, log_scale=-3.0):
    rng = np.random.default_rng(seed)
    means = (rng.uniform(-1, 1, (n, 3)) * spread).astype(np.float32)
    quats = rng.normal(size=(n, 4)).astype(np.float32)
    scales = np.exp(rng.normal(size=(n, 3)) * 0.5 + log_scale).astype(np.float32)
    vel = rng.normal(size=(n, 3)).astype(np.float32)
    return rng, means, quats, scales, vel


def _cameras(rng, C, W, H, f=300.0):
    from scipy.spatial.transform import Rotation
    vms, Ks = [], []
    for _ in range(C):
        vm = np.eye(4)
        vm[:3, :3] = Rotation.from_rotvec(rng.normal(size=3) * 0.3).as_matrix()
        vm[:3, 3] = [rng.normal() * 0.2, rng.normal() * 0.2, 3.0]
        vms.append(vm)
        Ks.append([[f, 0, W / 2 + 1.5], [0, f * 0.97, H / 2 - 2.0], [0, 0, 1]])
    return np.array(vms, np.float32), np.array(Ks, np.float32)


def _covars6(quats, scales):
    from scipy.spatial.transform import Rotation
    R = Rotation.from_quat(quats[:, [1, 2, 3, 0]].astype(np.float64)).as_matrix()
    cov = np.einsum("nij,nj,nkj->nik", R, scales.astype(np.float64) ** 2, R)
    return cov.reshape(-1, 9)[:, [0, 1, 2, 4, 5, 8]].astype(np.float32)


def _check_projection(out, ref32, ref64, lidar=False):
    radii = to_np(out[0])
    valid = (radii[..., 0] > 0) & (ref32[0][..., 0] > 0) & (ref64[0][..., 0] > 0)
    # the same Gaussians survive the culls (boundary cases may flip with the last float bit)
    agree = ((radii[..., 0] > 0) == (ref32[0][..., 0] > 0)).mean()
    assert agree > 0.999, agree
    assert valid.sum() > 100
    if lidar:
        assert_close(radii[valid], ref64[0][valid], atol=1e-4, rtol=1e-4, name="radii")
    else:
        d = np.abs(radii[valid].astype(np.int64) - ref32[0][valid])
        assert d.max() <= 1 and (d > 0).mean() < 1e-3, (d.max(), (d > 0).mean())
    names = ["means2d", "depths", "conics", "compensations", "pix_vels", "depth_compensations"]
    for k, name in enumerate(names[: len(out) - 1], start=1):
        if out[k] is None:
            assert ref64[k] is None
            continue
        got = to_np(out[k])
        assert_close(got[valid], ref64[k][valid], atol=1e-4, rtol=1e-4, name=name)
        assert (got[radii[..., 0] <= 0] == 0).all(), f"{name}: culled rows must be zero"


@pytest.mark.parametrize("use_covars", [False, True])
@pytest.mark.parametrize("use_vel", [False, True])
@pytest.mark.parametrize("comp", [False, True])
def test_projection_camera(use_covars, use_vel, comp):
    from splatad_amd import fully_fused_projection
    C, N, W, H = 3, 20000, 320, 240
    rng, means, quats, scales, vel = _gaussians(N, 10)
    viewmats, Ks = _cameras(rng, C, W, H)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array([0.03, 0.0, 0.01], np.float32)
    covars = _covars6(quats, scales) if use_covars else None
    kw = dict(eps2d=0.3, near_plane=0.5, far_plane=4.5, radius_clip=0.5, calc_compensations=comp)
    args = (means, covars, None if use_covars else quats, None if use_covars else scales,
            vel if use_vel else None, viewmats, Ks, W, H, lin, ang, rs)
    ref32 = oracle.projection_fwd(*args, precision="f32", **kw)
    ref64 = oracle.projection_fwd(*args, precision="f64", **kw)
    t = [to_dev(a) if isinstance(a, np.ndarray) else a for a in args]
    out = fully_fused_projection(*t, packed=False, **kw)
    _check_projection(out, ref32, ref64)

    # packed == compacted unpacked, in (camera, gaussian) order
    pk = fully_fused_projection(*t, packed=True, **kw)
    cam, gid = to_np(pk[0]), to_np(pk[1])
    radii = to_np(out[0])
    sel = np.argwhere(radii[..., 0] > 0)
    np.testing.assert_array_equal(cam, sel[:, 0])
    np.testing.assert_array_equal(gid, sel[:, 1])
    assert pk[0].dtype == torch.int64 and pk[1].dtype == torch.int64
    for a, b in zip(pk[2:], out):
        if b is None:
            assert a is None
        else:
            np.testing.assert_array_equal(to_np(a), to_np(b)[sel[:, 0], sel[:, 1]])


@pytest.mark.parametrize("C,N,W,H,ts", [(3, 20000, 320, 240, 16), (1, 5000, 200, 120, 8), (2, 300, 64, 48, 16)])
def test_packed_projection_counts_the_intersections_of_its_rows(C, N, W, H, ts):
    """isect_grid: the packed projection returns rows that carry the lists of their tile
    intersections; isect_tiles on those tensors hands them out without a count of its own and
    they are the same lists; writing to the tensors, or another grid, makes it count again."""
    from splatad_amd import fully_fused_projection, isect_tiles
    rng, means, quats, scales, vel = _gaussians(N, 17)
    viewmats, Ks = _cameras(rng, C, W, H)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.linspace(0.0, 0.03, C).astype(np.float32)
    t = [to_dev(a) if isinstance(a, np.ndarray) else a
         for a in (means, None, quats, scales, vel, viewmats, Ks, W, H, lin, ang, rs)]
    kw = dict(eps2d=0.3, near_plane=0.5, far_plane=4.5, radius_clip=0.0, packed=True)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    plain = fully_fused_projection(*t, **kw)

    def lists(rows, ts=ts, tw=tw, th=th):
        cam, gid, radii, means2d, depths = rows[:5]
        return isect_tiles(means2d, radii, depths, ts, tw, th, packed=True, n_cameras=C,
                           camera_ids=cam, gaussian_ids=gid)

    def oracle_lists(rows, ts=ts, tw=tw, th=th):
        cam, gid, radii, means2d, depths = rows[:5]
        return oracle.isect_tiles(to_np(means2d), to_np(radii), to_np(depths), ts, tw, th, n_cameras=C,
                                  camera_ids=to_np(cam))

    want = lists(plain)  # counts by itself
    hinted = fully_fused_projection(*t, isect_grid=(ts, tw, th), **kw)
    for a, b in zip(plain, hinted):
        assert (a is None and b is None) or torch.equal(a, b)
    grid, made = hinted[2]._splatad_isect_count[:2]
    assert grid == (ts, tw, th)
    assert int(want[0].sum().item()) == made[1].numel() == want[1].numel()
    got = lists(hinted)  # what the projection made
    assert not hasattr(hinted[2], "_splatad_isect_count")  # good for one call
    for a, b in zip(want, got):
        assert torch.equal(a, b)
    for a, b in zip(got, oracle_lists(hinted)):
        np.testing.assert_array_equal(to_np(a), b)
    for a, b in zip(want, lists(hinted)):  # a second call counts by itself
        assert torch.equal(a, b)
    # another grid: the count does not apply
    hinted = fully_fused_projection(*t, isect_grid=(ts, tw, th), **kw)
    g2 = dict(ts=2 * ts, tw=math.ceil(W / (2 * ts)), th=math.ceil(H / (2 * ts)))
    for a, b in zip(lists(hinted, **g2), oracle_lists(hinted, **g2)):
        np.testing.assert_array_equal(to_np(a), b)
    # rows written to after the projection: counted again
    hinted = fully_fused_projection(*t, isect_grid=(ts, tw, th), **kw)
    hinted[2][: hinted[2].shape[0] // 2] = 0
    changed = lists(hinted)
    assert changed[1].numel() < want[1].numel()
    for a, b in zip(changed, oracle_lists(hinted)):
        np.testing.assert_array_equal(to_np(a), b)


@pytest.mark.parametrize("C,N,W,H,ts,comp,degree,per_sensor,with_depth",
                         [(3, 20000, 320, 240, 16, False, 3, False, True),
                          (2, 6000, 200, 120, 8, True, 2, True, False),
                          (1, 400, 64, 48, 16, True, 0, False, True)])
def test_packed_projection_makes_what_was_asked_for_beside_the_sort(C, N, W, H, ts, comp, degree, per_sensor,
                                                                  with_depth):
    """beside=: the packed rows, their opacities and their colours are written on the helper
    stream; after the join they equal, bit for bit, the plain projection's rows, the gather
    opacities[gaussian_ids] (* compensations) and view_dependent_colors on those rows."""
    from splatad_amd import fully_fused_projection, isect_tiles
    from splatad_amd.hip._wrapper import view_dependent_colors
    from splatad_amd._helper_stream import HelperStream as _Beside
    rng, means, quats, scales, vel = _gaussians(N, 23)
    viewmats, Ks = _cameras(rng, C, W, H)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.linspace(0.0, 0.03, C).astype(np.float32)
    K = (degree + 1) ** 2 + 2
    coeffs = to_dev(rng.normal(size=((C, N, K, 3) if per_sensor else (N, K, 3))).astype(np.float32) * 0.5)
    opacities = to_dev(rng.uniform(0.05, 1.0, N).astype(np.float32))
    t = [to_dev(a) if isinstance(a, np.ndarray) else a
         for a in (means, None, quats, scales, vel, viewmats, Ks, W, H, lin, ang, rs)]
    kw = dict(eps2d=0.3, near_plane=0.5, far_plane=4.5, radius_clip=0.0, packed=True, calc_compensations=comp)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    plain = fully_fused_projection(*t, **kw)
    cam, gid, radii, means2d, depths, conics, comps, pix_vels = plain
    want_lists = isect_tiles(means2d, radii, depths, ts, tw, th, packed=True, n_cameras=C,
                             camera_ids=cam, gaussian_ids=gid)
    want_colors = view_dependent_colors(degree, t[0], t[5], coeffs, radii, depths if with_depth else None, cam, gid)
    want_opacities = opacities[gid] * comps if comp else opacities[gid]
    for _ in range(2):  # the second call meets the first one's memory on the helper stream
        beside = _Beside(torch.device(DEV))
        assert beside.side is not None
        beside.requests["colors"] = (degree, coeffs, with_depth)
        beside.requests["opacities"] = opacities
        rows = fully_fused_projection(*t, isect_grid=(ts, tw, th), beside=beside, **kw)
        lists = isect_tiles(rows[3], rows[2], rows[4], ts, tw, th, packed=True, n_cameras=C,
                            camera_ids=rows[0], gaussian_ids=rows[1])
        beside.join()
        for a, b in zip(plain, rows):
            assert (a is None and b is None) or torch.equal(a, b)
        for a, b in zip(want_lists, lists):
            assert torch.equal(a, b)
        assert torch.equal(beside.results["colors"], want_colors)
        assert torch.equal(beside.results["opacities"], want_opacities)
        # view_dependent_colors takes what was made instead of running its kernel
        taken = view_dependent_colors(degree, t[0], t[5], coeffs, rows[2], rows[4] if with_depth else None,
                                      rows[0], rows[1], precomputed=beside.results["colors"])
        assert taken is beside.results["colors"]


@pytest.mark.parametrize("use_covars", [False, True])
@pytest.mark.parametrize("use_vel", [False, True])
def test_projection_lidar(use_covars, use_vel):
    from splatad_amd import fully_fused_lidar_projection
    from scipy.spatial.transform import Rotation
    C, N = 2, 20000
    rng, means, quats, scales, vel = _gaussians(N, 11, spread=30.0, log_scale=-1.5)
    means[:, 2] *= 0.15
    vms = []
    for _ in range(C):
        vm = np.eye(4)
        vm[:3, :3] = Rotation.from_rotvec(rng.normal(size=3) * 0.1).as_matrix()
        vm[:3, 3] = rng.normal(size=3)
        vms.append(vm)
    viewmats = np.array(vms, np.float32)
    lin = (rng.normal(size=(C, 3)) * 5).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.2).astype(np.float32)
    rs = np.array([0.1, 0.0], np.float32)
    covars = _covars6(quats, scales) if use_covars else None
    kw = dict(eps2d=0.017, near_plane=1.0, far_plane=40.0, radius_clip=0.05, calc_compensations=True)
    args = (means, covars, None if use_covars else quats, None if use_covars else scales,
            vel if use_vel else None, viewmats, -20.0, 15.0, -170.0, 175.0, lin, ang, rs)
    ref32 = oracle.lidar_projection_fwd(*args, precision="f32", **kw)
    ref64 = oracle.lidar_projection_fwd(*args, precision="f64", **kw)
    t = [to_dev(a) if isinstance(a, np.ndarray) else a for a in args]
    # API order: (..., viewmats, lin, ang, rs, min_el, max_el, min_az, max_az)
    out = fully_fused_lidar_projection(t[0], t[1], t[2], t[3], t[4], t[5], t[10], t[11], t[12],
                                       t[6], t[7], t[8], t[9], **kw)
    _check_projection(out, ref32, ref64, lidar=True)


def test_isect_camera_reference_recipe():
    # input recipe of the reference's test_isect (tests/test_basic.py:704-712)
    from splatad_amd import isect_offset_encode, isect_tiles
    rng = np.random.default_rng(42)
    C, N, W, H, ts = 3, 1000, 40, 60, 16
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    means2d = (rng.normal(size=(C, N, 2)) * W).astype(np.float32)
    radii = rng.integers(0, W, (C, N, 2)).astype(np.int32)
    depths = rng.random((C, N)).astype(np.float32)
    for sort in (True, False):
        tpg, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), ts, tw, th, sort=sort)
        o_tpg, o_ids, o_flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th, sort=sort)
        np.testing.assert_array_equal(to_np(tpg), o_tpg)
        np.testing.assert_array_equal(to_np(ids), o_ids)
        np.testing.assert_array_equal(to_np(flat), o_flat)
        assert ids.dtype == torch.int64 and flat.dtype == torch.int32 and tpg.dtype == torch.int32
    offs = isect_offset_encode(ids if sort else to_dev(o_ids), C, tw, th)
    tpg, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    np.testing.assert_array_equal(to_np(offs), oracle.isect_offset_encode(to_np(ids), C, tw, th))


@pytest.mark.parametrize("n,C,W,H,ts,rmax", [(200000, 2, 640, 480, 16, 40), (3000, 1, 64, 64, 16, 600),
                                              (50000, 4, 200, 120, 8, 12), (0, 1, 64, 64, 16, 5),
                                              # 150 sensors x 256 coarse blocks: two binning launches
                                              (300, 150, 1024, 1024, 16, 30)])
def test_isect_camera_sizes_and_packed(n, C, W, H, ts, rmax):
    from splatad_amd import isect_offset_encode, isect_tiles
    rng = np.random.default_rng(n + C)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    means2d = np.stack([rng.uniform(-20, W + 20, (C, n)), rng.uniform(-20, H + 20, (C, n))], -1).astype(np.float32)
    radii = rng.integers(0, rmax, (C, n, 2)).astype(np.int32)
    depths = rng.uniform(0.01, 100, (C, n)).astype(np.float32)
    depths[:, : n // 10] = 7.5   # many exact depth ties: order must follow the flatten id
    tpg, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), ts, tw, th)
    o_tpg, o_ids, o_flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    np.testing.assert_array_equal(to_np(tpg), o_tpg)
    np.testing.assert_array_equal(to_np(ids), o_ids)
    np.testing.assert_array_equal(to_np(flat), o_flat)
    offs = isect_offset_encode(ids, C, tw, th)               # table kept by isect_tiles
    offs_k = isect_offset_encode(ids.clone(), C, tw, th)     # derived from the keys
    np.testing.assert_array_equal(to_np(offs), oracle.isect_offset_encode(o_ids, C, tw, th))
    np.testing.assert_array_equal(to_np(offs_k), to_np(offs))
    if n == 0:
        return
    # packed input gives the same keys; ids index the packed rows
    sel = np.nonzero(radii[..., 0].reshape(-1) > 0)[0]
    cam_ids = (sel // n).astype(np.int64)
    tpg_p, ids_p, flat_p = isect_tiles(
        to_dev(means2d.reshape(-1, 2)[sel]), to_dev(radii.reshape(-1, 2)[sel]),
        to_dev(depths.reshape(-1)[sel]), ts, tw, th, packed=True, n_cameras=C,
        camera_ids=to_dev(cam_ids), gaussian_ids=to_dev((sel % n).astype(np.int64)))
    np.testing.assert_array_equal(to_np(ids_p), o_ids)
    np.testing.assert_array_equal(sel[to_np(flat_p)], o_flat)


@pytest.mark.parametrize("n,tie_frac", [(1500, 0.8), (6000, 0.0), (6000, 0.5), (12000, 0.3),
                                        (20000, 0.1), (40000, 0.0), (40000, 0.4), (3000, 1.0),
                                        (60000, 0.4), (100000, 0.5), (400, 0.2), (300000, 0.0),
                                        (100000, 0.9)])
def test_isect_sort_long_segments_and_depth_ties(n, tie_frac):
    # every Gaussian covers all four tiles of the one coarse block.  The block's list is cut into
    # up to 16 depth slabs, and equal depths share a slab: the sizes and tie fractions exercise
    # every length class of the block sort, the lists it takes in parts (16000 to 50000 equal
    # depths, ordered by id alone; 18750 distinct depths per slab) and, with 90000 equal depths,
    # the list that is left to the per-tile segment sort with its own classes and oversized buckets
    from splatad_amd import isect_tiles
    rng = np.random.default_rng(n + int(10 * tie_frac))
    means2d = rng.uniform(10, 22, (1, n, 2)).astype(np.float32)
    radii = np.full((1, n, 2), 40, np.int32)
    depths = np.exp(rng.uniform(-3, 5, (1, n))).astype(np.float32)
    depths[0, rng.random(n) < tie_frac] = 3.25
    tpg, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), 16, 2, 2)
    o_tpg, o_ids, o_flat = oracle.isect_tiles(means2d, radii, depths, 16, 2, 2)
    assert o_ids.shape[0] == 4 * n
    np.testing.assert_array_equal(to_np(tpg), o_tpg)
    np.testing.assert_array_equal(to_np(ids), o_ids)
    np.testing.assert_array_equal(to_np(flat), o_flat)


@pytest.mark.parametrize("n,tie_frac,turns", [(3000, 0.3, 1), (3000, 0.5, 2), (20000, 0.9, 1), (30000, 0.6, 2),
                                              (120000, 0.9, 1)])
def test_isect_lidar_long_lists_ties_and_rectangles_wider_than_the_grid(n, tie_frac, turns):
    # a grid of 4 x 2 tiles (one coarse block) that every Gaussian covers; with turns == 2 the
    # rectangles are wider than the full turn, so a tile is listed twice by the same Gaussian and
    # the block's list holds equal keys.  Many equal depths put a slab's list beyond what one LDS
    # sort takes (taken in parts) and, with 108000 of them, beyond what the block sort takes at
    # all (the per-tile segment sort then).
    from splatad_amd import isect_lidar_tiles
    rng = np.random.default_rng(n + turns)
    eb = np.array([-20.0, 0.0, 20.0], np.float32)
    means2d = np.stack([rng.uniform(-180, 180, (1, n)), rng.uniform(-5, 5, (1, n))], -1).astype(np.float32)
    radii = np.empty((1, n, 2), np.float32)
    radii[..., 0] = 170.0 if turns == 1 else rng.uniform(185.0, 300.0, (1, n))
    radii[..., 1] = 30.0
    depths = np.exp(rng.uniform(-3, 5, (1, n))).astype(np.float32)
    depths[0, rng.random(n) < tie_frac] = 3.25
    got = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb), 90.0, -180.0)
    want = oracle.isect_lidar_tiles(means2d, radii, depths, eb, 90.0, -180.0)
    assert want[1].shape[0] >= 6 * n
    for g, w in zip(got, want):
        np.testing.assert_array_equal(to_np(g), w)


@pytest.mark.parametrize("n,spread", [(300, "even"), (1800, "even"), (1800, "far"), (7000, "even"),
                                      (1800, "infinite"), (5000, "infinite")])
def test_isect_sort_of_short_segments_by_depth_spread(n, spread):
    # The short-segment sort places entries by bins that are linear in the depth when no bin gets
    # too full, and by equalised buckets otherwise: depths spread evenly over their range take
    # the first way, a range stretched by a few far depths the second, and depths that are not
    # finite floats (their bit patterns still order the keys, rasterization.cu:77-84) are
    # never binned by value.
    from splatad_amd import isect_tiles
    rng = np.random.default_rng(n + len(spread))
    means2d = rng.uniform(10, 22, (1, n, 2)).astype(np.float32)
    radii = np.full((1, n, 2), 40, np.int32)
    depths = rng.uniform(0.5, 90.0, (1, n)).astype(np.float32)
    if spread == "far":
        depths[0, : n // 100] = rng.uniform(1e6, 1e9, n // 100)
    elif spread == "infinite":
        depths[0, rng.random(n) < 0.05] = np.inf
    tpg, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), 16, 2, 2)
    o_tpg, o_ids, o_flat = oracle.isect_tiles(means2d, radii, depths, 16, 2, 2)
    assert o_ids.shape[0] == 4 * n
    np.testing.assert_array_equal(to_np(tpg), o_tpg)
    np.testing.assert_array_equal(to_np(ids), o_ids)
    np.testing.assert_array_equal(to_np(flat), o_flat)


def test_isect_lidar_reference_recipe_and_wrap():
    # input recipe of the reference's test_isect_lidar (tests/test_basic.py:733-751)
    from splatad_amd import isect_lidar_tiles, isect_offset_encode
    rng = np.random.default_rng(42)
    C, N = 3, 100
    res, min_az = 0.2 * 16, -180.0
    n_az = math.ceil(360 / res)
    eb = np.linspace(-45.0, 45.0, 17).astype(np.float32)
    means2d = np.zeros((C, N, 2), np.float32)
    means2d[..., 0] = rng.random((C, N)) * 360 - 180
    means2d[..., 1] = rng.random((C, N)) * 90 - 45
    radii = (rng.random((C, N, 2)) / 2).astype(np.float32)
    depths = rng.random((C, N)).astype(np.float32)
    means2d[0, 0] = [-179.9, 0.0]; radii[0, 0] = [0.4, 0.3]
    means2d[0, 1] = [179.8, 10.0]; radii[0, 1] = [0.45, 0.2]
    for sort in (True, False):
        tpg, ids, flat = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb),
                                           res, min_az, sort=sort)
        o = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az, sort=sort)
        np.testing.assert_array_equal(to_np(tpg), o[0])
        np.testing.assert_array_equal(to_np(ids), o[1])
        np.testing.assert_array_equal(to_np(flat), o[2])
    tpg, ids, flat = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb), res, min_az)
    offs = isect_offset_encode(ids, C, n_az, 16)
    np.testing.assert_array_equal(to_np(offs), oracle.isect_offset_encode(to_np(ids), C, n_az, 16))
    np.testing.assert_array_equal(to_np(isect_offset_encode(ids.clone(), C, n_az, 16)), to_np(offs))
    ids.add_(0)  # an in-place change invalidates the kept table
    assert not (isect_offset_encode(ids, C, n_az, 16) is offs)


def test_isect_lidar_sector_of_tile_columns():
    """Tile columns that span 120 degrees only, reachable through the C entry points alone (the
    operator always passes a full turn of columns): Gaussians that straddle min_azim count zero
    tiles in the counting call and in the binning alike, so the lists have exactly n_isects
    entries and equal the oracle's."""
    from splatad_amd.hip import _backend
    rng = np.random.default_rng(11)
    C, N, n_az, res, min_az = 2, 40000, 16, 7.5, -60.0
    eb = np.sort(rng.uniform(-20, 20, 9)).astype(np.float32)
    means2d = np.stack([rng.uniform(-75, 75, (C, N)), rng.uniform(-25, 25, (C, N))], -1).astype(np.float32)
    radii = rng.exponential(3.0, (C, N, 2)).astype(np.float32)
    radii[rng.random((C, N)) < 0.2] = 0
    depths = rng.uniform(0.5, 80, (C, N)).astype(np.float32)
    straddle = (means2d[..., 0] - min_az - radii[..., 0] < 0) & (radii[..., 0] > 0)
    assert straddle.sum() > 100
    eb_dev = to_dev(eb)
    for sort in (True, False):
        got = _backend._C._isect(True, to_dev(means2d), to_dev(radii), to_dev(depths), None, None, C,
                                 (_backend._p(eb_dev), _backend._f32(res), _backend._f32(min_az)),
                                 n_az, 8, sort)
        want = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az, sort=sort, n_tiles_azim=n_az)
        assert (want[0] >= 0).all() and (want[0][straddle] == 0).all() and want[1].shape[0] > 1000
        for g, w in zip(got, want):
            np.testing.assert_array_equal(to_np(g), w)


@pytest.mark.parametrize("N", [100000, 750000])  # without and with depth slabs (4 per tile)
def test_isect_lidar_large_nonuniform(N):
    from splatad_amd import isect_lidar_tiles
    from splatad_amd import workloads
    rng = np.random.default_rng(5)
    C = 2
    elev = workloads.lidar_beam_elevations(128)
    eb = workloads.lidar_tile_elevation_boundaries(elev, 4).numpy()
    res, min_az = 360.0 / 2048 * 64, -180.0
    means2d = np.stack([rng.uniform(-180, 180, (C, N)), rng.uniform(-30, 20, (C, N))], -1).astype(np.float32)
    radii = (rng.exponential(1.5, (C, N, 2))).astype(np.float32)
    radii[rng.random((C, N)) < 0.2] = 0
    depths = rng.uniform(0.5, 80, (C, N)).astype(np.float32)
    tpg, ids, flat = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb), res, min_az)
    o = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az)
    np.testing.assert_array_equal(to_np(tpg), o[0])
    np.testing.assert_array_equal(to_np(ids), o[1])
    np.testing.assert_array_equal(to_np(flat), o[2])


@pytest.mark.parametrize("case", range(10))
def test_isect_random_grids_depth_distributions_and_slabs(case):
    """Random small grids with 500-4000 Gaussians per tile (depth slabs on in most), one to three
    sensors, and depth distributions that make slab bounds awkward: log-uniform over six decades,
    70 % equal, two tight clusters, all equal."""
    from splatad_amd import isect_lidar_tiles, isect_tiles
    rng = np.random.default_rng(1000 + case)
    lidar = case % 2 == 1
    C = int(rng.integers(1, 4))
    if lidar:
        tw, th = int(rng.choice([4, 8, 16])), int(rng.integers(2, 6))
        N = min(int(rng.integers(500, 4000)) * tw * th // C + 1, 80000)
        eb = np.sort(rng.uniform(-30, 30, th + 1)).astype(np.float32)
        means2d = np.stack([rng.uniform(-180, 180, (C, N)), rng.uniform(-35, 35, (C, N))], -1).astype(np.float32)
        radii = rng.exponential(8.0, (C, N, 2)).astype(np.float32)
    else:
        tw, th = int(rng.integers(1, 6)), int(rng.integers(1, 5))
        N = min(int(rng.integers(500, 4000)) * tw * th // C + 1, 60000)
        means2d = np.stack([rng.uniform(-10, tw * 16 + 10, (C, N)),
                            rng.uniform(-10, th * 16 + 10, (C, N))], -1).astype(np.float32)
        radii = rng.integers(0, 40, (C, N, 2)).astype(np.int32)
    radii[rng.random((C, N)) < 0.2] = 0
    depths = [rng.uniform(0.5, 80, (C, N)),
              np.exp(rng.uniform(-6, 8, (C, N))),
              np.where(rng.random((C, N)) < 0.7, 3.25, rng.uniform(1, 100, (C, N))),
              np.where(rng.random((C, N)) < 0.5, rng.normal(5, 0.01, (C, N)), rng.normal(50, 0.01, (C, N))).clip(0.1),
              np.full((C, N), 7.0)][case // 2].astype(np.float32)
    if lidar:
        res = 360.0 / tw
        got = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb), res, -180.0)
        want = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, -180.0)
    else:
        got = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), 16, tw, th)
        want = oracle.isect_tiles(means2d, radii, depths, 16, tw, th)
    assert want[1].shape[0] > 0
    for g, w in zip(got, want):
        np.testing.assert_array_equal(to_np(g), w)


def _projected_scene(C, N, W, H, D, seed, rs=(0.02, 0.0)):
    from splatad_amd import fully_fused_projection
    rng, means, quats, scales, vel = _gaussians(N, seed, log_scale=-2.6)
    viewmats, Ks = _cameras(rng, C, W, H, f=0.9 * W)
    lin = rng.normal(size=(C, 3)).astype(np.float32)
    ang = (rng.normal(size=(C, 3)) * 0.3).astype(np.float32)
    rs = np.array(rs[:C], np.float32)
    radii, means2d, depths, conics, _, pix_vels = fully_fused_projection(
        to_dev(means), None, to_dev(quats), to_dev(scales), to_dev(vel), to_dev(viewmats), to_dev(Ks),
        W, H, to_dev(lin), to_dev(ang), to_dev(rs))
    colors = rng.normal(size=(C, N, D)).astype(np.float32)
    opac = rng.uniform(0.05, 1.0, (C, N)).astype(np.float32)
    bg = rng.uniform(size=(C, D)).astype(np.float32)
    return dict(radii=radii, means2d=means2d, depths=depths, conics=conics, pix_vels=pix_vels,
                colors=to_dev(colors), opacities=to_dev(opac), backgrounds=to_dev(bg), rs=to_dev(rs))


@pytest.mark.parametrize("D,ts", [(3, 16), (4, 16), (1, 16), (32, 16), (33, 16), (7, 8), (64, 4), (70, 16)])
def test_rasterize_to_pixels(D, ts):
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_pixels
    C, N, W, H = 2, 2500, 200, 136
    s = _projected_scene(C, N, W, H, D, seed=20 + D)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    _, ids, flat = isect_tiles(s["means2d"], s["radii"], s["depths"], ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    for bg in (s["backgrounds"], None):
        rc, ra = rasterize_to_pixels(s["means2d"], s["conics"], s["colors"], s["opacities"],
                                     s["pix_vels"], W, H, ts, offs, flat,
                                     rolling_shutter_time=s["rs"], backgrounds=bg)
        args = [to_np(s[k]) for k in ("means2d", "conics", "colors", "opacities", "pix_vels", "rs")]

        def render():
            o = oracle.rasterize_to_pixels_fwd(*args, to_np(bg), W, H, ts, to_np(offs), to_np(flat),
                                               precision="f64")
            return dict(colors=o[0], alphas=o[1])

        assert rc.shape == (C, H, W, D) and ra.shape == (C, H, W, 1)
        assert_matches_oracle_decisions(dict(colors=to_np(rc), alphas=to_np(ra)), render_variants(render),
                                        dict(colors=(1e-4, 0.0), alphas=(1e-4, 0.0)), name=f"D={D}")
    lo, hi = float(ra.min()), float(ra.max())
    assert hi > 0.9 and lo < 0.9, (lo, hi)


def test_rasterize_to_pixels_last_ids_and_termination():
    # dense, opaque scene so that most pixels terminate early
    from splatad_amd.hip._backend import _C
    from splatad_amd import isect_offset_encode, isect_tiles
    C, N, W, H, D, ts = 1, 30000, 96, 64, 3, 16
    s = _projected_scene(C, N, W, H, D, seed=3, rs=(0.0,))
    s["opacities"] = torch.full_like(s["opacities"], 0.95)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    _, ids, flat = isect_tiles(s["means2d"], s["radii"], s["depths"], ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    rc, ra, last = _C.rasterize_to_pixels_fwd(s["means2d"], s["conics"], s["colors"], s["opacities"],
                                             s["pix_vels"], s["rs"], None, W, H, ts, offs, flat)
    args = [to_np(s[k]) for k in ("means2d", "conics", "colors", "opacities", "pix_vels", "rs")]
    lasts = []

    def render():
        o = oracle.rasterize_to_pixels_fwd(*args, None, W, H, ts, to_np(offs), to_np(flat), precision="f64")
        lasts.append(o[2])
        return dict(colors=o[0], alphas=o[1])

    variants = render_variants(render)
    o_ra = variants[0]["alphas"]
    # an opaque scene stops every pixel at the transmittance threshold: more of them hinge on it
    assert_matches_oracle_decisions(dict(colors=to_np(rc), alphas=to_np(ra)), variants,
                                    dict(colors=(1e-4, 0.0), alphas=(1e-4, 0.0)), max_attributed=5e-2)
    # the last composited list entry equals the oracle's for one of the decision outcomes
    assert np.logical_or.reduce([to_np(last) == l for l in lasts]).all()
    assert (to_np(last) == lasts[0]).mean() > 0.99
    assert (o_ra > 0.9998).mean() > 0.5   # the scene really saturates


def points_oracle(means2d, conics, feats, opac, pix_vels, dcomp, bg, raster_pts, W, H, tw, th, asum, threshold,
                  offs, flat, depth_idx):
    """The float64 oracle's lidar compositing of device tensors, as a dict of outputs."""
    o = oracle.rasterize_to_points_fwd(
        to_np(means2d), to_np(conics), to_np(feats), to_np(opac), to_np(pix_vels), to_np(dcomp),
        None if bg is None else to_np(bg), to_np(raster_pts), W, H, tw, th, asum, threshold, to_np(offs),
        to_np(flat), depth_idx, precision="f64")
    out = dict(features=o[0], alphas=o[1], median=o[4])
    if asum:
        out["alpha_sum"] = o[3]
    return out


def _lidar_scene(N, seed, H=16, W=256, tw=32, th=4, D=5, C=1):
    from splatad_amd import fully_fused_lidar_projection
    from splatad_amd import workloads
    l = workloads.lidar_sweep(n=N, seed=seed, n_beams=H, n_azimuth=W, feature_dim=D - 1,
                              tile_width=tw, tile_height=th, with_velocities=True)
    l["scales"] = l["scales"] * 3.0
    rng = np.random.default_rng(seed)
    rp = l["raster_pts"].numpy().copy()
    rp[..., 2] = rng.uniform(2, 60, rp.shape[:-1])
    rp[..., :2] += rng.normal(size=rp[..., :2].shape).astype(np.float32) * 0.01
    rp[0, 0, :7, 2] = 0.0
    rp[0, 3, 5, 2] = -1.0
    l["raster_pts"] = torch.from_numpy(rp)
    l["angular_velocity"] = torch.tensor([[0.0, 0.05, 0.3]])
    d = workloads.to_device(l, DEV)
    proj = fully_fused_lidar_projection(
        d["means"], None, d["quats"], d["scales"], d["velocities"], d["viewmats"],
        d["linear_velocity"], d["angular_velocity"], d["rolling_shutter_time"],
        d["min_elevation"], d["max_elevation"], d["min_azimuth"], d["max_azimuth"], eps2d=0.017)
    return d, proj


@pytest.mark.parametrize("D,asum,with_bg,tile", [
    (5, True, False, (32, 4)), (5, False, False, (32, 4)), (33, True, False, (32, 4)),
    (2, True, False, (32, 4)), (40, True, False, (32, 4)), (32, False, False, (32, 4)),
    (33, False, True, (32, 4)), (32, True, True, (32, 4)), (5, True, True, (32, 4)),
    # tiles that do not fill a wavefront (the workgroup is padded) and one of four wavefronts
    (5, True, False, (16, 2)), (33, True, True, (16, 1)), (3, False, False, (64, 4))])
def test_rasterize_to_points(D, asum, with_bg, tile):
    from splatad_amd import isect_lidar_tiles, isect_offset_encode, rasterize_to_points
    H, W = 16, 256
    tw, th = tile
    d, proj = _lidar_scene(8000, 30 + D, H, W, tw, th, D)
    radii, means2d, depths, conics, _, pix_vels, dcomp = proj
    res = d["azimuth_resolution"] * tw
    _, ids, flat = isect_lidar_tiles(means2d, radii, depths, d["tile_elevation_boundaries"], res, -180.0)
    offs = isect_offset_encode(ids, 1, W // tw, H // th)
    feats = torch.cat([d["lidar_features"], depths[..., None]], -1)
    opac = d["opacities"][None].contiguous()
    bg = None
    if with_bg:
        bg = torch.rand((1, D), device=DEV, generator=torch.Generator(device=DEV).manual_seed(D))
    rf, ra, rsum, med = rasterize_to_points(means2d, conics, feats, opac, pix_vels, dcomp,
                                            d["raster_pts"], W, H, tw, th, offs, flat, asum, 0.3,
                                            backgrounds=bg)
    variants = render_variants(lambda: points_oracle(
        means2d, conics, feats, opac, pix_vels, dcomp, bg, d["raster_pts"], W, H, tw, th, asum, 0.3, offs,
        flat, D - 1), lidar=True)
    got = dict(features=to_np(rf), alphas=to_np(ra), median=to_np(med))
    tols = dict(features=(2e-4, 1e-4), alphas=(1e-4, 0.0), median=(1e-3, 1e-4))
    if asum:
        got["alpha_sum"] = to_np(rsum)
        tols["alpha_sum"] = (1e-4, 1e-4)
    else:
        assert rsum is None
    assert_matches_oracle_decisions(got, variants, tols, name=f"D={D}")
    assert float(ra.max()) > 0.5
    assert (to_np(rf)[0, 0, :7] == 0).all() and (to_np(ra)[0, 3, 5] == 0).all()
    # features and ranges handed over separately: the same arithmetic on the same values
    split = rasterize_to_points(means2d, conics, d["lidar_features"].contiguous(), opac, pix_vels, dcomp,
                                d["raster_pts"], W, H, tw, th, offs, flat, asum, 0.3, backgrounds=bg,
                                ranges=depths)
    for got, want in zip(split, (rf, ra, rsum, med)):
        assert (got is None and want is None) or torch.equal(got, want)


@pytest.mark.parametrize("deg", [0, 1, 2, 3, 4])
def test_spherical_harmonics_forward(deg):
    from splatad_amd import spherical_harmonics
    rng = np.random.default_rng(deg)
    n, K = 5000, 25
    dirs = (rng.normal(size=(n, 3)) * 2).astype(np.float32)
    coeffs = rng.normal(size=(n, K, 3)).astype(np.float32)
    masks = rng.random(n) > 0.3
    col = spherical_harmonics(deg, to_dev(dirs), to_dev(coeffs))
    assert_close(to_np(col), oracle.spherical_harmonics(deg, dirs, coeffs, precision="f64"),
                 atol=1e-4, name="sh")
    colm = spherical_harmonics(deg, to_dev(dirs), to_dev(coeffs), masks=to_dev(masks))
    assert_close(to_np(colm), oracle.spherical_harmonics(deg, dirs, coeffs, masks, precision="f64"),
                 atol=1e-4, name="sh masked")
    # batched shapes [C, N, ...]
    col2 = spherical_harmonics(deg, to_dev(dirs.reshape(5, 1000, 3)), to_dev(coeffs.reshape(5, 1000, K, 3)))
    np.testing.assert_array_equal(to_np(col2).reshape(n, 3), to_np(col))


def test_isect_lidar_extent_beyond_a_full_turn():
    # regression: azimuth extents below -360 degrees must wrap inside the tile grid
    from splatad_amd import isect_lidar_tiles
    rng = np.random.default_rng(9)
    N = 2000
    means2d = np.stack([rng.uniform(-180, 180, (1, N)), rng.uniform(-20, 20, (1, N))], -1).astype(np.float32)
    radii = rng.uniform(0.0, 900.0, (1, N, 2)).astype(np.float32)
    depths = rng.uniform(0.1, 50, (1, N)).astype(np.float32)
    eb = np.linspace(-25, 25, 5).astype(np.float32)
    res = 360.0 / 16
    tpg, ids, flat = isect_lidar_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), to_dev(eb), res, -180.0)
    o = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, -180.0)
    np.testing.assert_array_equal(to_np(tpg), o[0])
    np.testing.assert_array_equal(to_np(ids), o[1])
    np.testing.assert_array_equal(to_np(flat), o[2])


def test_isect_fill_with_too_small_a_count_stays_inside_its_lists():
    """The C ABI trusts the caller's n_isects for the size of `lists` and of the outputs.  A count
    that is too small (a caller's mistake, or rows changed between the two calls) must not make
    any stage write outside them: every buffer is followed by guard bytes, which have to survive."""
    import ctypes
    from splatad_amd.hip import _backend as b
    lib = b.load_library()
    rng = np.random.default_rng(77)
    C, N, tile, tw, th = 1, 6000, 16, 20, 12
    means2d = to_dev(np.stack([rng.uniform(0, tw * tile, (C, N)), rng.uniform(0, th * tile, (C, N))], -1).astype(np.float32))
    radii = to_dev(rng.integers(1, 60, (C, N, 2)).astype(np.int32))
    depths = to_dev(rng.uniform(0.1, 50.0, (C, N)).astype(np.float32))
    total = C * N
    tiles_per_gauss = torch.empty((C, N), dtype=torch.int32, device=DEV)
    ws = b._workspace(lib.splatad_isect_workspace_bytes(b._u64(total), b._u32(C), b._u32(tw * th)), DEV)
    head = (b._u64(total), b._u32(N), b._p(None), b._p(means2d), b._p(radii), b._p(depths))
    tail = (b._u32(C), b._u32(tile), b._u32(tw), b._u32(th), b._i32(1))
    n_host = b._i64(0)
    b._check(lib.splatad_isect_tiles_count(*head, *tail, b._p(tiles_per_gauss), b._p(ws), ctypes.byref(n_host),
                                           b._stream(DEV)))
    n = int(n_host.value)
    assert n > 100_000
    small = n // 10
    guard = 8 << 20  # more than every list of the true size takes
    lists_bytes = lib.splatad_isect_lists_bytes(b._u64(total), b._i64(small))

    def guarded(nbytes):
        buf = torch.full((nbytes + guard,), 0xA5, dtype=torch.uint8, device=DEV)
        return buf, buf[nbytes:]

    lists, lists_guard = guarded(lists_bytes)
    ids, ids_guard = guarded(small * 8)
    flat, flat_guard = guarded(small * 4)
    offsets = torch.empty((C, th, tw), dtype=torch.int32, device=DEV)
    rc = lib.splatad_isect_tiles_fill(*head, *tail, b._i64(small), b._p(tiles_per_gauss), b._p(ws), b._p(lists),
                                      b._p(ids), b._p(flat), b._p(offsets), b._stream(DEV))
    torch.cuda.synchronize()
    assert rc == 0, lib.splatad_last_error()
    for name, g in (("lists", lists_guard), ("isect_ids", ids_guard), ("flatten_ids", flat_guard)):
        assert bool((g == 0xA5).all()), f"{name}: written beyond the size the caller gave"
    # and the library still gives the right lists for the right count afterwards
    _, o_ids, o_flat = oracle.isect_tiles(to_np(means2d), to_np(radii), to_np(depths), tile, tw, th)
    from splatad_amd.hip._backend import _C
    _, g_ids, g_flat = _C.isect_tiles(means2d, radii, depths, None, None, C, tile, tw, th, True, True)
    assert np.array_equal(to_np(g_ids), o_ids) and np.array_equal(to_np(g_flat), o_flat)
