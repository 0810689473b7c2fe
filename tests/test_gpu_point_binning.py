"""GPU parity of the lidar point binning against the oracle: bit-exact keys, order, offsets
and populated images (reference tests: tests/test_basic.py:786-888)."""
import math

import numpy as np
import pytest
import torch

import oracle
from tests.gpu_util import to_dev, to_np

pytestmark = pytest.mark.gpu


def _points(C, N, seed, width=360.0, height=90.0):
    rng = np.random.default_rng(seed)
    pts = np.zeros((C, N, 5), np.float32)
    pts[..., 0] = rng.random((C, N)) * width - width / 2
    pts[..., 1] = rng.random((C, N)) * height - height / 2
    pts[..., 2:] = rng.uniform(0.5, 100.0, (C, N, 3))
    return pts


@pytest.mark.parametrize("C,N,n_el,res", [(3, 100_000, 16, 3.2), (1, 262_144, 32, 360.0 / 2048 * 64),
                                          (2, 777, 5, 7.0), (1, 50, 1, 360.0), (1, 0, 4, 10.0)])
def test_map_points_offsets_and_image(C, N, n_el, res):
    from splatad_amd import (map_points_to_lidar_tiles, points_mapping_offset_encode,
                             populate_image_from_points)
    pts = _points(C, N, C * 1000 + N)
    pts[:, : N // 50, 0] += 400.0      # azimuths outside [-180, 180) wrap
    eb = np.linspace(-45.0, 45.0, n_el + 1).astype(np.float32)
    n_az = int(math.ceil(float(np.float32(360.0) / np.float32(res))))
    for sort in (True, False):
        ids, flat = map_points_to_lidar_tiles(to_dev(pts[..., :2].copy()), to_dev(eb), res, -180.0, sort=sort)
        o_ids, o_flat = oracle.map_points_to_lidar_tiles(pts[..., :2], eb, res, -180.0, sort=sort)
        assert ids.dtype == torch.int64 and flat.dtype == torch.int32
        np.testing.assert_array_equal(to_np(ids), o_ids)
        np.testing.assert_array_equal(to_np(flat), o_flat)
    ids, flat = map_points_to_lidar_tiles(to_dev(pts[..., :2].copy()), to_dev(eb), res, -180.0)
    offs = points_mapping_offset_encode(ids, C, n_az, n_el)
    o_offs = oracle.points_mapping_offset_encode(to_np(ids), C, n_az, n_el)
    np.testing.assert_array_equal(to_np(offs), o_offs)
    tw, th = 8, 4
    W, H = n_az * tw - (3 if n_az * tw > 3 else 0), n_el * th
    img = populate_image_from_points(to_dev(pts), W, H, tw, th, offs, flat)
    o_img = oracle.populate_image_from_points(pts, W, H, tw, th, o_offs, to_np(flat))
    assert img.shape == (C, H, W, 5)
    np.testing.assert_array_equal(to_np(img), o_img)


def test_map_points_packed():
    from splatad_amd import map_points_to_lidar_tiles
    C, N = 4, 5000
    pts = _points(C, N, 11)[..., :2].reshape(-1, 2)
    sel = np.nonzero(np.random.default_rng(1).random(C * N) < 0.6)[0]
    cam = (sel // N).astype(np.int64)
    eb = np.linspace(-45.0, 45.0, 9).astype(np.float32)
    ids, flat = map_points_to_lidar_tiles(to_dev(pts[sel]), to_dev(eb), 5.0, -180.0, packed=True,
                                          n_cameras=C, camera_ids=to_dev(cam))
    o_ids, o_flat = oracle.map_points_to_lidar_tiles(pts[sel], eb, 5.0, -180.0, n_cameras=C, camera_ids=cam)
    np.testing.assert_array_equal(to_np(ids), o_ids)
    np.testing.assert_array_equal(to_np(flat), o_flat)


def test_binned_points_feed_the_lidar_rasterizer_layout():
    # the reference's recipe: a regular grid of points, binned and populated, gives back the grid
    from splatad_amd import (map_points_to_lidar_tiles, points_mapping_offset_encode,
                             populate_image_from_points, workloads)
    elev = workloads.lidar_beam_elevations(16)
    eb = workloads.lidar_tile_elevation_boundaries(elev, 4).numpy()
    n_cols, tw, th = 256, 32, 4
    az = -180.0 + (np.arange(n_cols) + 0.5) * 360.0 / n_cols
    grid = np.zeros((1, 16, n_cols, 5), np.float32)
    grid[0, :, :, 0] = az[None, :]
    grid[0, :, :, 1] = elev.numpy()[:, None]
    grid[0, :, :, 2] = 50.0
    grid[0, :, :, 3] = np.linspace(0, 1, n_cols)[None, :]
    grid[0, :, :, 4] = 1.0
    pts = grid.reshape(1, -1, 5)
    perm = np.random.default_rng(3).permutation(pts.shape[1])
    pts = np.ascontiguousarray(pts[:, perm])
    res = 360.0 / n_cols * tw
    ids, flat = map_points_to_lidar_tiles(to_dev(pts[..., :2].copy()), to_dev(eb), res, -180.0)
    offs = points_mapping_offset_encode(ids, 1, n_cols // tw, 4)
    img = to_np(populate_image_from_points(to_dev(pts), n_cols, 16, tw, th, offs, flat))
    # every tile holds exactly its tw*th points; inside a tile they come in shuffled order
    for ty in range(4):
        for tx in range(n_cols // tw):
            got = img[0, ty * th:(ty + 1) * th, tx * tw:(tx + 1) * tw].reshape(-1, 5)
            want = grid[0, ty * th:(ty + 1) * th, tx * tw:(tx + 1) * tw].reshape(-1, 5)
            key = lambda a: a[np.lexsort((a[:, 0], a[:, 1]))]
            np.testing.assert_array_equal(key(got), key(want))
