"""The entry point that allocates nothing (splatad_map_points_to_lidar_tiles_noalloc) against the
existing splatad_map_points_to_lidar_tiles, through the C ABI: identical keys and order
(bit-exact, as for every integer output), on two calls in a row, the second with a smaller input
(both share the library's static scratch), and a clear error beyond its limits."""
import ctypes
import math

import numpy as np
import pytest
import torch

from tests.gpu_util import DEV, to_dev, to_np

pytestmark = pytest.mark.gpu


def _call(lib, name, pts, eb, C, N, n_az, n_el, res, min_az, sort, workspace):
    from splatad_amd.hip import _backend as b
    total = C * N
    ids = torch.full((total,), -1, dtype=torch.int64, device=DEV)
    flat = torch.full((total,), -1, dtype=torch.int32, device=DEV)
    head = (b._u64(total), b._u32(N), b._p(None), b._p(pts), b._u32(C), b._p(eb), b._f32(res), b._f32(min_az),
            b._u32(n_az), b._u32(n_el), b._i32(sort))
    tail = (b._p(ids), b._p(flat), b._stream(DEV))
    fn = getattr(lib, name)
    rc = fn(*head, b._p(workspace), *tail) if workspace is not None else fn(*head, *tail)
    return rc, ids, flat


def _case(lib, C, N, n_el, res, seed):
    from splatad_amd.hip import _backend as b
    rng = np.random.default_rng(seed)
    pts = np.stack([rng.uniform(-180, 220, (C, N)), rng.uniform(-45, 45, (C, N))], -1).astype(np.float32)
    eb = to_dev(np.linspace(-45.0, 45.0, n_el + 1).astype(np.float32))
    n_az = int(math.ceil(float(np.float32(360.0) / np.float32(res))))
    d_pts = to_dev(pts)
    for sort in (1, 0):
        ws = b._workspace(lib.splatad_map_points_to_lidar_tiles_workspace_bytes(
            b._u64(C * N), b._u32(C), b._u32(n_az * n_el)), DEV)
        rc, ids, flat = _call(lib, "splatad_map_points_to_lidar_tiles", d_pts, eb, C, N, n_az, n_el, res, -180.0,
                              sort, ws)
        assert rc == 0, lib.splatad_last_error()
        rc, ids2, flat2 = _call(lib, "splatad_map_points_to_lidar_tiles_noalloc", d_pts, eb, C, N, n_az, n_el, res,
                                -180.0, sort, None)
        assert rc == 0, lib.splatad_last_error()
        torch.cuda.synchronize()
        assert int(ids.min()) >= 0 and int(flat.min()) >= 0
        np.testing.assert_array_equal(to_np(ids2), to_np(ids))
        np.testing.assert_array_equal(to_np(flat2), to_np(flat))


def test_noalloc_point_binning_matches_the_workspace_entry_point():
    from splatad_amd.hip import _backend as b
    lib = b.load_library()
    # a full 128 x 2048 sweep on 32 x 32 tiles, then a smaller call on another grid: the second
    # call finds the first one's leftovers in the scratch
    _case(lib, 1, 262_144, 32, 360.0 / 2048 * 64, seed=1)
    _case(lib, 2, 3_000, 5, 7.0, seed=2)
    _case(lib, 3, 100_000, 16, 3.2, seed=3)
    # beyond the limits: refused with a message, nothing launched
    eb = to_dev(np.linspace(-45.0, 45.0, 3).astype(np.float32))
    pts = to_dev(np.zeros((1, 8, 2), np.float32))
    rc, _, _ = _call(lib, "splatad_map_points_to_lidar_tiles_noalloc", pts, eb, 1, 8, 20000, 2, 0.018, -180.0, 1, None)
    assert rc != 0 and b"exceed the limit" in lib.splatad_last_error()
    lib.splatad_map_points_to_lidar_tiles_noalloc_max_points.restype = ctypes.c_uint64
    big = lib.splatad_map_points_to_lidar_tiles_noalloc_max_points() + 1
    rc = lib.splatad_map_points_to_lidar_tiles_noalloc(
        b._u64(big), b._u32(big), b._p(None), b._p(pts), b._u32(1), b._p(eb), b._f32(10.0), b._f32(-180.0),
        b._u32(36), b._u32(2), b._i32(1), b._p(pts), b._p(pts), b._stream(DEV))
    assert rc != 0 and b"exceed the limit" in lib.splatad_last_error()


def test_noalloc_point_binning_replays_from_a_graph():
    """After one eager call on the device (which does the one-time setup), the entry point
    enqueues kernels only: captured into a graph and replayed over changing inputs, with eager
    work and synchronisations between the replays, it gives the workspace entry point's result
    every time."""
    from splatad_amd.hip import _backend as b
    lib = b.load_library()
    C, N, n_el, res = 1, 50_000, 8, 360.0 / 64
    n_az = int(math.ceil(float(np.float32(360.0) / np.float32(res))))
    eb = to_dev(np.linspace(-45.0, 45.0, n_el + 1).astype(np.float32))
    pts = torch.empty((C, N, 2), device=DEV)
    ids = torch.full((C * N,), -1, dtype=torch.int64, device=DEV)
    flat = torch.full((C * N,), -1, dtype=torch.int32, device=DEV)

    def enqueue():
        rc = lib.splatad_map_points_to_lidar_tiles_noalloc(
            b._u64(C * N), b._u32(N), b._p(None), b._p(pts), b._u32(C), b._p(eb), b._f32(res), b._f32(-180.0),
            b._u32(n_az), b._u32(n_el), b._i32(1), b._p(ids), b._p(flat), b._stream(DEV))
        assert rc == 0, lib.splatad_last_error()

    def fill(seed):
        g = torch.Generator(device=DEV).manual_seed(seed)
        pts[..., 0] = torch.rand((C, N), device=DEV, generator=g) * 400.0 - 180.0
        pts[..., 1] = torch.rand((C, N), device=DEV, generator=g) * 90.0 - 45.0

    fill(0)
    enqueue()  # eager: the one-time setup happens here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        enqueue()
    for seed in (1, 2, 3):
        fill(seed)
        ids.fill_(-1)
        flat.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        ws = b._workspace(lib.splatad_map_points_to_lidar_tiles_workspace_bytes(
            b._u64(C * N), b._u32(C), b._u32(n_az * n_el)), DEV)
        rc, want_ids, want_flat = _call(lib, "splatad_map_points_to_lidar_tiles", pts, eb, C, N, n_az, n_el, res,
                                        -180.0, 1, ws)
        assert rc == 0, lib.splatad_last_error()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(to_np(ids), to_np(want_ids))
        np.testing.assert_array_equal(to_np(flat), to_np(want_flat))
