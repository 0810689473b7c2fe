"""Pins of the oracle's lidar point binning (map_points_to_lidar_tiles,
points_mapping_offset_encode, populate_image_from_points) against independent numpy
restatements and the invariants of the reference's own tests (tests/test_basic.py:786-888)."""
import math

import numpy as np

import oracle


def _scene(C, N, n_el, res, seed, width=360.0, height=90.0):
    rng = np.random.default_rng(seed)
    pts = np.zeros((C, N, 2), np.float32)
    pts[..., 0] = rng.random((C, N)) * width - width / 2
    pts[..., 1] = rng.random((C, N)) * height - height / 2
    eb = np.linspace(-height / 2, height / 2, n_el + 1).astype(np.float32)
    return pts, eb


def _numpy_tiles(pts, eb, res, min_az, n_az):
    az = pts[..., 0] - np.float32(min_az)
    wrapped = np.where((az >= 0) & (az < 360), az, np.fmod(az + np.float32(360), np.float32(360)))
    x = (wrapped / np.float32(res)).astype(np.int32)
    n_el = eb.shape[0] - 1
    y = np.maximum(np.searchsorted(eb[:n_el], pts[..., 1], side="left") - 1, 0)
    return y * n_az + x


def test_map_points_matches_numpy_and_is_stable():
    C, N, n_el, res, min_az = 3, 20000, 16, 3.2, -180.0
    pts, eb = _scene(C, N, n_el, res, 1)
    n_az = math.ceil(360 / res)
    ids, flat = oracle.map_points_to_lidar_tiles(pts, eb, res, min_az, sort=False)
    tiles = _numpy_tiles(pts, eb, res, min_az, n_az).reshape(-1)
    cams = np.repeat(np.arange(C), N)
    np.testing.assert_array_equal(ids, (cams.astype(np.int64) << 32) | tiles)
    np.testing.assert_array_equal(flat, np.arange(C * N))
    s_ids, s_flat = oracle.map_points_to_lidar_tiles(pts, eb, res, min_az, sort=True)
    order = np.argsort(ids, kind="stable")
    np.testing.assert_array_equal(s_ids, ids[order])
    np.testing.assert_array_equal(s_flat, order)


def test_map_points_wraps_azimuth_and_clamps_elevation():
    eb = np.array([-10.0, 0.0, 10.0], np.float32)     # two rows
    pts = np.array([[[-190.0, -50.0],    # azimuth 350 after wrapping, below the first boundary
                     [179.0, 5.0],       # last column, upper row
                     [-180.0, 50.0],     # first column, above the last boundary -> top row
                     [10.0, 0.0]]], np.float32)   # elevation on a boundary belongs to the row below
    ids, _ = oracle.map_points_to_lidar_tiles(pts, eb, 90.0, -180.0, sort=False)
    # columns: (az + 180) / 90; rows by the boundaries below the point
    np.testing.assert_array_equal(ids, [0 * 4 + 3, 1 * 4 + 3, 1 * 4 + 0, 0 * 4 + 2])


def test_packed_points_use_camera_ids():
    pts, eb = _scene(2, 500, 8, 6.4, 3)
    sel = np.arange(0, 1000, 3)
    cam = (sel // 500).astype(np.int64)
    ids_p, flat_p = oracle.map_points_to_lidar_tiles(pts.reshape(-1, 2)[sel], eb, 6.4, -180.0,
                                                     n_cameras=2, camera_ids=cam)
    ids, flat = oracle.map_points_to_lidar_tiles(pts, eb, 6.4, -180.0, sort=False)
    order = np.argsort(ids[sel], kind="stable")
    np.testing.assert_array_equal(ids_p, ids[sel][order])
    np.testing.assert_array_equal(flat_p, order)


def test_offsets_match_searchsorted_and_reference_invariants():
    # recipe of the reference's test_map_points_to_lidar_tiles
    C, N, n_el = 3, 100_000, 16
    res = 0.2 * 16
    n_az = math.ceil(360 / res)
    pts, eb = _scene(C, N, n_el, res, 42)
    ids, flat = oracle.map_points_to_lidar_tiles(pts, eb, res, -180.0)
    offs = oracle.points_mapping_offset_encode(ids, C, n_az, n_el)
    lin = (ids >> 32) * (n_az * n_el) + (ids & 0xFFFFFFFF)
    np.testing.assert_array_equal(offs.reshape(-1),
                                  np.searchsorted(lin, np.arange(C * n_az * n_el), side="left"))
    cams = ids >> 32
    for c in range(C):
        assert (cams[c * N:(c + 1) * N] == c).all()
        o = offs[c].reshape(-1)
        assert (np.diff(o) > 0).all()                       # every tile holds points
        last = pts.reshape(-1, 2)[flat[c * N:(c + 1) * N][-10:]]
        assert (last[:, 0] >= 180 - res).all() and (last[:, 1] >= eb[-2]).all()
    assert (oracle.points_mapping_offset_encode(np.zeros(0, np.int64), 2, 4, 3) == 0).all()


def test_populate_image_fills_tiles_in_order():
    C, N, th, tw, n_ch = 2, 30000, 4, 8, 16
    res = 360.0 / 128 * tw                     # 16 azimuth tiles of 8 columns
    rng = np.random.default_rng(5)
    pts = np.zeros((C, N, 5), np.float32)
    pts[..., 0] = rng.uniform(-180, 180, (C, N))
    pts[..., 1] = rng.uniform(-20, 20, (C, N))
    pts[..., 2:] = rng.uniform(0.5, 100, (C, N, 3))
    eb = np.linspace(-20.01, 20.01, n_ch // th + 1).astype(np.float32)
    ids, flat = oracle.map_points_to_lidar_tiles(pts[..., :2], eb, res, -180.0)
    gw, gh = 16, n_ch // th
    offs = oracle.points_mapping_offset_encode(ids, C, gw, gh)
    img = oracle.populate_image_from_points(pts, gw * tw, n_ch, tw, th, offs, flat)
    assert img.shape == (C, n_ch, gw * tw, 5) and img.all()    # reference: raster_pts_image.all()
    flat_pts = pts.reshape(-1, 5)
    ends = np.append(offs.reshape(-1)[1:], C * N)
    for c, ty, tx in [(0, 0, 0), (1, 3, 15), (0, 2, 7)]:
        start = offs[c, ty, tx]
        assert ends[(c * gh + ty) * gw + tx] - start >= tw * th
        tile = img[c, ty * th:(ty + 1) * th, tx * tw:(tx + 1) * tw].reshape(-1, 5)
        np.testing.assert_array_equal(tile, flat_pts[flat[start:start + tw * th]])
    # a tile with fewer points than pixels leaves the rest zero; image smaller than the grid
    few = pts[:, :40]
    ids2, flat2 = oracle.map_points_to_lidar_tiles(few[..., :2], eb, res, -180.0)
    offs2 = oracle.points_mapping_offset_encode(ids2, C, gw, gh)
    img2 = oracle.populate_image_from_points(few, gw * tw - 3, n_ch - 1, tw, th, offs2, flat2)
    assert img2.shape == (C, n_ch - 1, gw * tw - 3, 5)
    assert (img2[..., 2] > 0).sum() <= C * 40 and (img2[..., 2] > 0).sum() > 0
