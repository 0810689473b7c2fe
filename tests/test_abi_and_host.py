"""CPU checks of the C ABI and of the host-side logic (no GPU, no compute calls into HIP)."""
import ctypes
import math
import os
import re

import numpy as np
import pytest
import torch

from tests.oracle_backend import OracleOps

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "splatad_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(splatad_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from splatad_amd import build
    path = build.build()
    lib = ctypes.CDLL(path)
    names = _declared_symbols()
    assert len(names) >= 20, names
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/splatad_hip.h but not exported"
    lib.splatad_abi_version.restype = ctypes.c_int
    assert lib.splatad_abi_version() == 11
    lib.splatad_last_error.restype = ctypes.c_char_p
    assert isinstance(lib.splatad_last_error(), bytes)
    # size queries are pure host code
    lib.splatad_isect_workspace_bytes.restype = ctypes.c_size_t
    lib.splatad_isect_lists_bytes.restype = ctypes.c_size_t
    assert lib.splatad_isect_workspace_bytes(ctypes.c_uint64(1000), ctypes.c_uint32(2), ctypes.c_uint32(100)) >= 3 * 256
    a = lib.splatad_isect_lists_bytes(ctypes.c_uint64(1000), ctypes.c_int64(0))
    b = lib.splatad_isect_lists_bytes(ctypes.c_uint64(1000), ctypes.c_int64(5000))
    assert a >= 1000 * 8 and b >= 5000 * 24
    lib.splatad_projection_packed_workspace_bytes.restype = ctypes.c_size_t
    assert lib.splatad_projection_packed_workspace_bytes(ctypes.c_uint32(2), ctypes.c_uint32(1000)) >= 2000 * 48


def test_host_argument_errors_need_no_gpu():
    # invalid arguments are rejected by the C entry points before any kernel launch
    from splatad_amd import build
    lib = ctypes.CDLL(build.build())
    lib.splatad_last_error.restype = ctypes.c_char_p
    null = ctypes.c_void_p(0)
    rc = lib.splatad_sh_fwd(ctypes.c_uint32(10), ctypes.c_uint32(4), ctypes.c_uint32(5), null, null, null, null, null)
    assert rc != 0 and b"degree" in lib.splatad_last_error()
    rc = lib.splatad_rasterize_to_pixels_fwd(
        ctypes.c_uint32(1), ctypes.c_int64(0), ctypes.c_uint32(0), null, null, null, null, null, null, null,
        ctypes.c_uint32(8), ctypes.c_uint32(8), ctypes.c_uint32(16), ctypes.c_uint32(1), ctypes.c_uint32(1),
        null, null, null, null, null, null)
    assert rc != 0 and b"channels" in lib.splatad_last_error()


def test_ops_fail_loudly_without_library_or_gpu(monkeypatch):
    from splatad_amd.hip import _backend
    from splatad_amd import fully_fused_projection
    z = torch.zeros
    args = (z(4, 3), None, z(4, 4), z(4, 3), None, torch.eye(4)[None], torch.eye(3)[None], 8, 8, z(1, 3), z(1, 3), z(1))
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        fully_fused_projection(*args)
    monkeypatch.setattr(_backend, "_lib", None)
    monkeypatch.setattr(_backend, "LIB_PATH", "/nonexistent/libsplatad_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fully_fused_projection(*args)


@pytest.fixture
def oracle_ops(monkeypatch):
    from splatad_amd.hip import _backend
    monkeypatch.setattr(_backend, "_C", OracleOps())


def _camera_inputs(N=300, C=2, seed=0):
    g = torch.Generator().manual_seed(seed)
    means = torch.rand(N, 3, generator=g) * 2 - 1
    quats = torch.randn(N, 4, generator=g)
    scales = torch.rand(N, 3, generator=g) * 0.1 + 0.02
    opac = torch.rand(N, generator=g)
    viewmats = torch.eye(4)[None].repeat(C, 1, 1)
    viewmats[:, 2, 3] = 3.0
    viewmats[1:, 0, 3] = 0.3
    Ks = torch.tensor([[60.0, 0, 32.0], [0, 60.0, 24.0], [0, 0, 1]])[None].repeat(C, 1, 1)
    return means, quats, scales, opac, viewmats, Ks, g


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("render_mode", ["RGB", "RGB+D", "D", "ED", "RGB+ED"])
@pytest.mark.parametrize("sh_degree", [None, 2])
def test_rasterization_shapes_and_meta(oracle_ops, packed, render_mode, sh_degree):
    # mirrors the reference's shape test (tests/test_rasterization.py:17-80)
    from splatad_amd import rasterization
    N, C, W, H = 300, 2, 64, 48
    means, quats, scales, opac, viewmats, Ks, g = _camera_inputs(N, C)
    colors = torch.rand(N, 9, 3, generator=g) if sh_degree is not None else torch.rand(C, N, 3, generator=g)
    bg = torch.rand(C, 3, generator=g)
    rc, ra, meta = rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, W, H,
                                 sh_degree=sh_degree, packed=packed, render_mode=render_mode, backgrounds=bg)
    X = {"RGB": 3, "RGB+D": 4, "RGB+ED": 4, "D": 1, "ED": 1}[render_mode]
    assert rc.shape == (C, H, W, X) and ra.shape == (C, H, W, 1)
    assert set(meta) == {"camera_ids", "gaussian_ids", "radii", "means2d", "depths", "conics", "opacities",
                         "pix_vels", "tile_width", "tile_height", "tiles_per_gauss", "isect_ids",
                         "flatten_ids", "isect_offsets", "width", "height", "tile_size", "n_cameras"}
    assert meta["tile_width"] == 4 and meta["tile_height"] == 3 and meta["n_cameras"] == C
    if packed:
        nnz = meta["camera_ids"].shape[0]
        assert meta["means2d"].shape == (nnz, 2) and meta["opacities"].shape == (nnz,)
        assert meta["gaussian_ids"].dtype == torch.int64
    else:
        assert meta["camera_ids"] is None and meta["means2d"].shape == (C, N, 2)
    assert meta["isect_offsets"].shape == (C, 3, 4)
    assert float(ra.max()) > 0.05


def test_rasterization_packed_equals_unpacked_and_chunking(oracle_ops):
    from splatad_amd import rasterization
    N, C, W, H = 300, 2, 64, 48
    means, quats, scales, opac, viewmats, Ks, g = _camera_inputs(N, C, seed=3)
    colors = torch.rand(N, 7, generator=g)
    lin = torch.randn(C, 3, generator=g)
    rs = torch.tensor([0.02, 0.0])
    kw = dict(linear_velocity=lin, rolling_shutter_time=rs, render_mode="RGB+ED")
    a = rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, W, H, packed=False, **kw)
    b = rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, W, H, packed=True, **kw)
    torch.testing.assert_close(a[0], b[0], rtol=0, atol=1e-6)
    torch.testing.assert_close(a[1], b[1], rtol=0, atol=1e-6)
    c = rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, W, H, packed=False,
                      channel_chunk=3, **kw)
    torch.testing.assert_close(a[0], c[0], rtol=0, atol=1e-6)
    # antialiased mode multiplies opacities by the compensation
    d = rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, W, H, packed=False,
                      rasterize_mode="antialiased", **kw)
    assert (d[2]["opacities"] <= a[2]["opacities"] + 1e-7).all()


def _lidar_inputs(N=400, D=6, seed=1):
    from splatad_amd import workloads
    s = workloads.lidar_sweep(n=N, seed=seed, n_beams=16, n_azimuth=128, feature_dim=D, tile_width=32,
                              tile_height=4)
    s["scales"] = s["scales"] * 6
    return s


@pytest.mark.parametrize("D,chunk", [(6, 32), (40, 32), (63, 32), (31, 32), (5, 4)])
def test_lidar_rasterization_shapes_chunks_and_meta(oracle_ops, D, chunk):
    from splatad_amd import lidar_rasterization
    s = _lidar_inputs(D=D)
    rf, ra, asum, meta = lidar_rasterization(
        s["means"], s["quats"], s["scales"], s["opacities"], s["lidar_features"], None, s["viewmats"],
        s["raster_pts"], s["tile_elevation_boundaries"], s["linear_velocity"], s["angular_velocity"],
        s["rolling_shutter_time"], min_elevation=-26.0, max_elevation=16.0, n_elevation_channels=16,
        azimuth_resolution=s["azimuth_resolution"], tile_width=32, tile_height=4, channel_chunk=chunk)
    H, W = 16, 128
    if D + 1 > chunk:
        n_chunks = (D + chunk) // chunk
        rendered = min(D, n_chunks * (chunk - 1))     # the reference's chunking drops the rest
        assert rf.shape == (1, H, W, rendered + 1)
        assert meta["median_depths"].shape == (1, H, W, n_chunks)
    else:
        assert rf.shape == (1, H, W, D + 1)
        assert meta["median_depths"].shape == (1, H, W, 1)
    assert ra.shape == (1, H, W, 1) and asum.shape == (1, H, W, 1)
    for k in ("tile_grid_width", "tile_grid_height", "tile_width", "tile_height", "median_depths", "pix_vels"):
        assert k in meta
    assert meta["tile_grid_width"] == 4 and meta["tile_grid_height"] == 4
    assert meta["radii"].dtype == torch.float32 and meta["pix_vels"].shape[-1] == 3


def test_lidar_chunked_equals_single_pass(oracle_ops):
    from splatad_amd import lidar_rasterization
    s = _lidar_inputs(D=9, seed=4)

    def run(**kw):
        return lidar_rasterization(
            s["means"], s["quats"], s["scales"], s["opacities"], s["lidar_features"], None, s["viewmats"],
            s["raster_pts"], s["tile_elevation_boundaries"], s["linear_velocity"], s["angular_velocity"],
            s["rolling_shutter_time"], min_elevation=-26.0, max_elevation=16.0, n_elevation_channels=16,
            azimuth_resolution=s["azimuth_resolution"], tile_width=32, tile_height=4, **kw)
    a = run()
    b = run(channel_chunk=4)      # 3 chunks of 3 features + range
    torch.testing.assert_close(a[0], b[0], rtol=0, atol=1e-5)
    torch.testing.assert_close(a[1], b[1], rtol=0, atol=1e-6)
    c = run(use_depth_compensation=False)
    assert not torch.equal(a[0][..., -1], c[0][..., -1])
    torch.testing.assert_close(a[0][..., :-1], c[0][..., :-1], rtol=0, atol=1e-6)
    d = run(compute_alpha_sum_until_points=False)
    assert d[2] is None


def test_argument_checks_match_the_reference(oracle_ops):
    from splatad_amd import lidar_rasterization, rasterization, rasterize_to_pixels
    means, quats, scales, opac, viewmats, Ks, g = _camera_inputs(50, 1)
    colors = torch.rand(50, 3)
    with pytest.raises(AssertionError):
        rasterization(means, quats[:, :3], scales, opac, colors, None, viewmats, Ks, 32, 32)
    with pytest.raises(AssertionError):
        rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, 32, 32, render_mode="XYZ")
    with pytest.raises(AssertionError):   # SH degree needs (deg+1)^2 bases
        rasterization(means, quats, scales, opac, torch.rand(50, 4, 3), None, viewmats, Ks, 32, 32, sh_degree=2)
    with pytest.raises(AssertionError, match="sparse_grad"):
        rasterization(means, quats, scales, opac, colors, None, viewmats, Ks, 32, 32, packed=False, sparse_grad=True)
    z = torch.zeros
    with pytest.raises(ValueError, match="Unsupported number of color channels"):
        rasterize_to_pixels(z(1, 5, 2), z(1, 5, 3), z(1, 5, 514), z(1, 5), z(1, 5, 2), 16, 16, 16,
                            z(1, 1, 1, dtype=torch.int32), z(0, dtype=torch.int32))
    s = _lidar_inputs(N=50, D=3)
    common = (s["means"], s["quats"], s["scales"], s["opacities"], s["lidar_features"], None, s["viewmats"],
              s["raster_pts"], s["tile_elevation_boundaries"])
    with pytest.raises(NotImplementedError):
        lidar_rasterization(*common, n_elevation_channels=16, tile_height=4, tile_width=32, packed=True,
                            min_elevation=-26, max_elevation=16)
    with pytest.raises(AssertionError):   # elevation range beyond +-85 degrees
        lidar_rasterization(*common, n_elevation_channels=16, tile_height=4, tile_width=32, max_elevation=89)
    with pytest.raises(AssertionError):   # tile larger than 256 points
        lidar_rasterization(*common, n_elevation_channels=16, tile_height=16, tile_width=32,
                            min_elevation=-26, max_elevation=16)
