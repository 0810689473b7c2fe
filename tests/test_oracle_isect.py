"""Pins for the oracle's tile intersection, sort and offset encoding (CPU only).

Brute force over every (Gaussian, tile) pair with a geometric overlap test in
float64, numpy's stable argsort, searchsorted for the offsets, the invariants the
reference's own tests assert (tests/test_basic.py:697-783) and the input recipes of
those tests re-drawn with numpy seeds.
"""
import math

import numpy as np

import oracle


def _decode(ids, n_tiles, C):
    tb = oracle.bit_width(n_tiles)
    hi = ids >> 32
    return hi >> tb, hi & ((1 << tb) - 1), (ids & 0xFFFFFFFF).astype(np.uint32)


def _recipe_camera(seed, C=3, N=1000, width=40, height=60):
    # tests/test_basic.py:704-712
    rng = np.random.default_rng(seed)
    means2d = (rng.normal(size=(C, N, 2)) * width).astype(np.float32)
    radii = rng.integers(0, width, (C, N, 2)).astype(np.int32)
    depths = rng.random((C, N)).astype(np.float32)
    return means2d, radii, depths


def test_camera_isect_brute_force_and_invariants():
    C, N, W, H, ts = 3, 1000, 40, 60, 16
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    means2d, radii, depths = _recipe_camera(0, C, N, W, H)
    tpg, ids, flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th, sort=False)
    # brute force: tile (tx,ty) is hit iff the box [mu-r, mu+r] overlaps [t*ts, (t+1)*ts)
    exp_ids, exp_flat = [], []
    tb = oracle.bit_width(tw * th)
    for c in range(C):
        for g in range(N):
            if radii[c, g, 0] <= 0:
                assert tpg[c, g] == 0
                continue
            mx, my = means2d[c, g].astype(np.float64)
            rx, ry = radii[c, g].astype(np.float64)
            cnt = 0
            for ty in range(th):
                for tx in range(tw):
                    hit = ((tx + 1) * ts > mx - rx) and (tx * ts < mx + rx) and \
                          ((ty + 1) * ts > my - ry) and (ty * ts < my + ry)
                    if hit:
                        cnt += 1
                        dbits = int(depths[c, g].view(np.int32))
                        exp_ids.append((c << (32 + tb)) | ((ty * tw + tx) << 32) | dbits)
                        exp_flat.append(c * N + g)
            assert tpg[c, g] == cnt, (c, g)
    assert tpg.sum() == ids.shape[0] == len(exp_ids)
    np.testing.assert_array_equal(ids, np.array(exp_ids, np.int64))
    np.testing.assert_array_equal(flat, np.array(exp_flat, np.int32))

    # sorted variant == numpy stable argsort of the emission order
    _, ids_s, flat_s = oracle.isect_tiles(means2d, radii, depths, ts, tw, th, sort=True)
    order = np.argsort(ids, kind="stable")
    np.testing.assert_array_equal(ids_s, ids[order])
    np.testing.assert_array_equal(flat_s, flat[order])
    assert (np.diff(ids_s) >= 0).all()

    # offsets == searchsorted of the (camera, tile) field; monotone; counts add up
    offs = oracle.isect_offset_encode(ids_s, C, tw, th)
    cam, tile, _ = _decode(ids_s, tw * th, C)
    lin = cam * (tw * th) + tile
    exp_off = np.searchsorted(lin, np.arange(C * tw * th), side="left").astype(np.int32)
    np.testing.assert_array_equal(offs.reshape(-1), exp_off)
    assert (np.diff(offs.reshape(-1)) >= 0).all()
    counts = np.diff(np.append(offs.reshape(-1), ids_s.shape[0]))
    np.testing.assert_array_equal(counts, np.bincount(lin, minlength=C * tw * th))


def test_camera_isect_saturating_casts_and_empty():
    # negative tile coordinates saturate to 0, huge ones to the grid size
    means2d = np.array([[[-1000.0, -1000.0], [1e6, 1e6], [8.0, 8.0], [20.0, 5.0]]], np.float32)
    radii = np.array([[[5, 5], [5, 5], [100000, 100000], [0, 3]]], np.int32)
    depths = np.array([[1.0, 2.0, 3.0, 4.0]], np.float32)
    tpg, ids, flat = oracle.isect_tiles(means2d, radii, depths, 16, 3, 4)
    assert tpg.tolist() == [[0, 0, 12, 0]]
    assert flat.tolist() == [2] * 12
    offs = oracle.isect_offset_encode(ids, 1, 3, 4)
    assert offs.reshape(-1).tolist() == list(range(12))
    # no intersections at all: offsets are all zero (rasterization.cu:281-283)
    tpg, ids, flat = oracle.isect_tiles(means2d, np.zeros_like(radii), depths, 16, 3, 4)
    assert ids.shape == (0,) and flat.shape == (0,)
    assert (oracle.isect_offset_encode(ids, 1, 3, 4) == 0).all()


def test_camera_isect_packed_matches_unpacked():
    C, N, W, H, ts = 3, 500, 64, 48, 16
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    means2d, radii, depths = _recipe_camera(5, C, N, W, H)
    _, ids_u, flat_u = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    sel = np.nonzero(radii[..., 0].reshape(-1) > 0)[0]
    cam_ids = (sel // N).astype(np.int64)
    tpg_p, ids_p, flat_p = oracle.isect_tiles(
        means2d.reshape(-1, 2)[sel], radii.reshape(-1, 2)[sel], depths.reshape(-1)[sel], ts, tw,
        th, n_cameras=C, camera_ids=cam_ids)
    np.testing.assert_array_equal(ids_p, ids_u)
    np.testing.assert_array_equal(sel[flat_p], flat_u)


def _recipe_lidar(seed, C=3, N=100):
    # tests/test_basic.py:733-751
    rng = np.random.default_rng(seed)
    width, height = 360.0, 90.0
    means2d = np.zeros((C, N, 2), np.float32)
    means2d[..., 0] = rng.random((C, N)) * width - width / 2
    means2d[..., 1] = rng.random((C, N)) * height - height / 2
    radii = (rng.random((C, N, 2)) / 2).astype(np.float32)
    depths = rng.random((C, N)).astype(np.float32)
    return means2d, radii, depths


def _lidar_brute(means2d, radii, depths, eb, res, min_az, n_az):
    C, N = depths.shape
    n_el = len(eb) - 1
    tb = oracle.bit_width(n_az * n_el)
    out_ids, out_flat, tpg = [], [], np.zeros((C, N), np.int32)
    eb = eb.astype(np.float64)
    for c in range(C):
        for g in range(N):
            if radii[c, g, 0] <= 0:
                continue
            a = float(means2d[c, g, 0]) - min_az
            lo, hi = a - float(radii[c, g, 0]), a + float(radii[c, g, 0])
            elo = float(means2d[c, g, 1]) - float(radii[c, g, 1])
            ehi = float(means2d[c, g, 1]) + float(radii[c, g, 1])
            # azimuth pieces in emission order: wrapped-left part, main part, wrapped-right part
            cols = []
            if lo < 0:
                cols += list(range(int(math.floor((lo + 360.0) / res)), n_az))
                first_main = 0
            else:
                first_main = int(math.floor(lo / res))
            if hi <= 360.0:
                cols += list(range(first_main, int(math.ceil(hi / res))))
            else:
                cols += list(range(first_main, n_az))
                cols += list(range(0, int(math.ceil((hi - 360.0) / res))))
            rows = [e for e in range(n_el) if eb[e] < ehi and eb[e + 1] >= elo]
            tpg[c, g] = len(rows) * len(cols)
            dbits = int(depths[c, g].view(np.int32))
            for e in rows:
                for k in cols:
                    out_ids.append((c << (32 + tb)) | ((e * n_az + k) << 32) | dbits)
                    out_flat.append(c * N + g)
    return tpg, np.array(out_ids, np.int64), np.array(out_flat, np.int32)


def test_lidar_isect_brute_force_with_wraparound():
    C, N = 3, 100
    means2d, radii, depths = _recipe_lidar(1, C, N)
    # force wrap-around on both sides and an oversized elevation extent
    means2d[0, 0] = [-179.9, 0.0]; radii[0, 0] = [0.4, 0.3]
    means2d[0, 1] = [179.8, 10.0]; radii[0, 1] = [0.45, 0.2]
    means2d[0, 2] = [0.0, 44.9]; radii[0, 2] = [0.2, 3.0]
    means2d[0, 3] = [10.0, -44.9]; radii[0, 3] = [0.2, 3.0]
    radii[1, 5, 0] = 0.0
    res, min_az = 0.2 * 16, -180.0
    n_az = math.ceil(360 / res)
    eb = np.linspace(-45.0, 45.0, 17).astype(np.float32)
    tpg, ids, flat = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az, sort=False)
    tpg_b, ids_b, flat_b = _lidar_brute(means2d, radii, depths, eb, res, min_az, n_az)
    np.testing.assert_array_equal(tpg, tpg_b)
    np.testing.assert_array_equal(ids, ids_b)
    np.testing.assert_array_equal(flat, flat_b)
    assert tpg[0, 0] >= 2 and tpg[0, 1] >= 2  # wrapped Gaussians touch both ends

    _, ids_s, flat_s = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az)
    order = np.argsort(ids, kind="stable")
    np.testing.assert_array_equal(ids_s, ids[order])
    np.testing.assert_array_equal(flat_s, flat[order])
    offs = oracle.isect_offset_encode(ids_s, C, n_az, 16)

    # containment invariants of the first tile, as in tests/test_basic.py:768-783
    first = flat_s[: offs[0, 0, 1]]
    m = means2d.reshape(-1, 2)[first]
    r = radii.reshape(-1, 2)[first]
    a_lo = m[:, 0] - r[:, 0] - min_az
    a_hi = m[:, 0] + r[:, 0] - min_az
    wraps = (a_lo < 0) | (a_hi > 360)
    assert (((a_lo < res) & (a_hi > 0)) | wraps).all()
    assert ((m[:, 1] - r[:, 1] <= eb[1]) & (m[:, 1] + r[:, 1] > eb[0])).all()


def test_lidar_isect_full_circle_tiles():
    # tile resolution that divides 360 exactly, non-uniform elevation boundaries
    C, N = 2, 400
    rng = np.random.default_rng(7)
    means2d = np.zeros((C, N, 2), np.float32)
    means2d[..., 0] = rng.uniform(-180, 180, (C, N))
    means2d[..., 1] = rng.uniform(-27, 17, (C, N))
    radii = rng.uniform(0.0, 6.0, (C, N, 2)).astype(np.float32)
    depths = rng.uniform(1, 80, (C, N)).astype(np.float32)
    res, min_az = 360.0 / 32, -180.0
    eb = np.array([-26, -20, -12, -7, -3, -1, 0.5, 2, 4, 7, 11, 16], np.float32)
    tpg, ids, flat = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az, sort=False)
    tpg_b, ids_b, flat_b = _lidar_brute(means2d, radii, depths, eb, res, min_az, 32)
    np.testing.assert_array_equal(tpg, tpg_b)
    np.testing.assert_array_equal(ids, ids_b)
    np.testing.assert_array_equal(flat, flat_b)


def test_lidar_isect_extent_beyond_a_full_turn():
    # A Gaussian next to the sensor can span more than 360 degrees: tile columns wrap with a
    # true modulo, every tile index stays inside the grid and the counts match the bounds.
    means2d = np.array([[[-100.0, 0.0], [120.0, 1.0]]], np.float32)
    radii = np.array([[[700.0, 2.0], [800.0, 1.0]]], np.float32)
    depths = np.array([[1.0, 2.0]], np.float32)
    eb = np.array([-30.0, 0.0, 30.0], np.float32)
    res = 360.0 / 8
    tpg, ids, flat = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, -180.0, sort=False)
    cam, tile, _ = _decode(ids, 8 * 2, 1)
    assert (cam == 0).all() and (tile >= 0).all() and (tile < 16).all()
    assert tpg.sum() == ids.shape[0] and (tpg > 16).all()
    # consecutive emissions walk the columns cyclically
    cols = tile[: tpg[0, 0] // 2] % 8
    assert ((np.diff(cols) % 8) == 1).all()


def test_lidar_isect_sector_of_tile_columns():
    # Tile columns that span 120 degrees only (the operator itself always uses a full turn,
    # rasterization.cu:435-436; a sector can only come through the kernel-level interface).
    # A Gaussian that straddles min_azim gets an empty column range and counts zero tiles
    # (the reference's count goes negative there); everything else is the brute-force
    # overlap, and the counts add up to the list length.
    res, n_az, min_az = 7.5, 16, -60.0
    eb = np.array([-20.0, -5.0, 0.0, 5.0, 20.0], np.float32)
    means2d = np.array([[[-60.2, 1.0],      # straddles min_azim: nothing
                         [-50.0, 1.0],      # inside, two columns
                         [0.0, -7.0],       # inside, crosses an elevation boundary
                         [59.0, 2.0],       # reaches the sector's upper edge
                         [30.0, 30.0]]],    # above every boundary
                       np.float32)
    radii = np.array([[[1.0, 1.0], [4.0, 1.0], [1.0, 3.0], [2.0, 1.0], [1.0, 1.0]]], np.float32)
    depths = np.array([[5.0, 4.0, 3.0, 2.0, 1.0]], np.float32)
    tpg, ids, flat = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, min_az, sort=False,
                                              n_tiles_azim=n_az)
    assert (tpg >= 0).all() and tpg.sum() == ids.shape[0] == flat.shape[0]
    assert tpg[0, 0] == 0 and tpg[0, 4] == 0
    for g in (1, 2, 3):
        a = means2d[0, g, 0] - min_az
        lo, hi = a - radii[0, g, 0], a + radii[0, g, 0]
        cols = list(range(int(math.floor(lo / res)), int(math.ceil(hi / res))))
        elo, ehi = means2d[0, g, 1] - radii[0, g, 1], means2d[0, g, 1] + radii[0, g, 1]
        rows = [e for e in range(4) if eb[e] < ehi and eb[e + 1] >= elo]
        assert tpg[0, g] == len(rows) * len(cols), g
        _, tile, _ = _decode(ids[flat == g], n_az * 4, 1)
        assert sorted(tile.tolist()) == sorted(e * n_az + (k % n_az) for e in rows for k in cols)
