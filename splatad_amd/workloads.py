"""Synthetic scenes for the benchmark configurations and the parity tests.

Every generator draws on the CPU from a seeded ``torch.Generator`` (so the
same numbers come out with or without a GPU) and returns a dict of CPU float32
tensors; callers move them to the device.  ``n`` can be lowered to get a small
instance of the same distribution for oracle-sized tests.
"""
import math
from typing import Dict, Optional

import torch


def _gen(seed: int) -> torch.Generator:
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    return g


def _quats(n, g):
    q = torch.randn(n, 4, generator=g)
    return q / q.norm(dim=-1, keepdim=True)


def camera_small(n: int = 10_000, seed: int = 0, width: int = 320, height: int = 240) -> Dict:
    """10k Gaussians in [-2,2]^3 in front of a 320x240 pinhole camera (fx=fy=300),
    no rolling shutter, RGB colours."""
    g = _gen(seed)
    means = torch.rand(n, 3, generator=g) * 4.0 - 2.0
    viewmats = torch.eye(4)[None].clone()
    viewmats[0, 2, 3] = 3.0  # camera 3 m behind the cube: depths 1..5
    scales = torch.exp(torch.randn(n, 3, generator=g) * 0.5 - 3.0)
    quats = _quats(n, g)
    opacities = torch.sigmoid(torch.randn(n, generator=g))
    colors = torch.rand(n, 3, generator=g)
    Ks = torch.tensor([[[300.0, 0.0, width / 2.0], [0.0, 300.0, height / 2.0], [0.0, 0.0, 1.0]]])
    return dict(means=means, quats=quats, scales=scales, opacities=opacities, colors=colors,
                velocities=None, viewmats=viewmats, Ks=Ks, width=width, height=height,
                linear_velocity=None, angular_velocity=None, rolling_shutter_time=None,
                sh_degree=None, near_plane=0.01, far_plane=1e10, eps2d=0.3, tile_size=16)


def camera_driving(n: int = 1_000_000, seed: int = 1, width: int = 1920, height: int = 1080,
                   n_cameras: int = 1, with_velocities: bool = False,
                   sh_degree: Optional[int] = 3) -> Dict:
    """Driving camera with rolling shutter: Gaussians in a 100 x 40 x 10 m box ahead of
    a 1920x1080 pinhole (fx=fy=1000), SH degree-3 colours, ego motion over a 30 ms
    row-wise readout.  With ``n_cameras`` > 1 the cameras are yawed around the
    sensor (0, +-60, +-120, 180 degrees) and the box is centred on it."""
    g = _gen(seed)
    surround = n_cameras > 1
    x = torch.rand(n, generator=g) * 40.0 - 20.0
    y = torch.rand(n, generator=g) * 10.0 - 5.0
    z = torch.rand(n, generator=g) * 100.0 - (50.0 if surround else 0.0)
    means = torch.stack([x, y, z], dim=-1)
    scales = torch.exp(torch.randn(n, 3, generator=g) * 0.7 - 2.0)
    quats = _quats(n, g)
    opacities = torch.sigmoid(torch.randn(n, generator=g))
    if sh_degree is None:
        colors = torch.rand(n, 3, generator=g)
    else:
        colors = torch.randn(n, 16, 3, generator=g) * 0.3
    velocities = torch.randn(n, 3, generator=g) if with_velocities else None
    fx = 1000.0 * width / 1920.0
    K = torch.tensor([[fx, 0.0, width / 2.0], [0.0, fx, height / 2.0], [0.0, 0.0, 1.0]])
    Ks = K[None].repeat(n_cameras, 1, 1)
    viewmats = torch.eye(4)[None].repeat(n_cameras, 1, 1)
    yaws = [0.0, 60.0, -60.0, 120.0, -120.0, 180.0]
    for c in range(n_cameras):
        a = math.radians(yaws[c % len(yaws)])
        # rotation about the camera's y (down) axis
        viewmats[c, 0, 0] = math.cos(a); viewmats[c, 0, 2] = -math.sin(a)
        viewmats[c, 2, 0] = math.sin(a); viewmats[c, 2, 2] = math.cos(a)
    lin = torch.randn(n_cameras, 3, generator=g) * 10.0
    ang = torch.randn(n_cameras, 3, generator=g) * 0.2
    rs = torch.full((n_cameras,), 0.03)
    return dict(means=means, quats=quats, scales=scales, opacities=opacities, colors=colors,
                velocities=velocities, viewmats=viewmats, Ks=Ks, width=width, height=height,
                linear_velocity=lin, angular_velocity=ang, rolling_shutter_time=rs,
                sh_degree=sh_degree, near_plane=0.01, far_plane=1e10, eps2d=0.3, tile_size=16)


def lidar_beam_elevations(n_beams: int = 128) -> torch.Tensor:
    """Non-uniform beam elevations in degrees, -25..+15, denser near 0."""
    u = torch.linspace(-1.0, 1.0, n_beams)
    return torch.where(u < 0, -25.0 * u.abs() ** 1.5, 15.0 * u.abs() ** 1.5)


def lidar_tile_elevation_boundaries(elev: torch.Tensor, tile_height: int) -> torch.Tensor:
    """[e0-1, midpoints between rows 4k-1 and 4k, e_last+1]."""
    n = elev.shape[0]
    inner = [(elev[k - 1] + elev[k]) * 0.5 for k in range(tile_height, n, tile_height)]
    return torch.stack([elev[0] - 1.0, *inner, elev[-1] + 1.0])


def lidar_sweep(n: int = 1_000_000, seed: int = 2, n_beams: int = 128, n_azimuth: int = 2048,
                feature_dim: int = 32, tile_width: int = 64, tile_height: int = 4,
                with_velocities: bool = False) -> Dict:
    """128-beam spinning lidar mid-box (x fwd, y left, z up), 2048 azimuth columns over
    360 degrees, 100 ms sweep with ego velocity, 32-dim features per Gaussian."""
    g = _gen(seed)
    x = torch.rand(n, generator=g) * 100.0 - 50.0
    y = torch.rand(n, generator=g) * 40.0 - 20.0
    z = torch.rand(n, generator=g) * 10.0 - 5.0
    means = torch.stack([x, y, z], dim=-1)
    scales = torch.exp(torch.randn(n, 3, generator=g) * 0.7 - 2.0)
    quats = _quats(n, g)
    opacities = torch.sigmoid(torch.randn(n, generator=g))
    features = torch.randn(1, n, feature_dim, generator=g)
    velocities = torch.randn(n, 3, generator=g) if with_velocities else None
    elev = lidar_beam_elevations(n_beams)
    az_res = 360.0 / n_azimuth
    az = -180.0 + (torch.arange(n_azimuth, dtype=torch.float32) + 0.5) * az_res
    boundaries = lidar_tile_elevation_boundaries(elev, tile_height)
    t = (torch.arange(n_azimuth, dtype=torch.float32) / max(n_azimuth - 1, 1) - 0.5) * 0.1
    raster_pts = torch.empty(1, n_beams, n_azimuth, 4)
    raster_pts[0, :, :, 0] = az[None, :]
    raster_pts[0, :, :, 1] = elev[:, None]
    raster_pts[0, :, :, 2] = 50.0
    raster_pts[0, :, :, 3] = t[None, :]
    lin = torch.randn(1, 3, generator=g) * 10.0
    ang = torch.zeros(1, 3)
    rs = torch.full((1,), 0.1)
    return dict(means=means, quats=quats, scales=scales, opacities=opacities,
                lidar_features=features, velocities=velocities, viewmats=torch.eye(4)[None].clone(),
                raster_pts=raster_pts, tile_elevation_boundaries=boundaries,
                linear_velocity=lin, angular_velocity=ang, rolling_shutter_time=rs,
                min_azimuth=-180.0, max_azimuth=180.0, min_elevation=-26.0, max_elevation=16.0,
                n_elevation_channels=n_beams, azimuth_resolution=az_res, tile_width=tile_width,
                tile_height=tile_height, near_plane=0.01, far_plane=1e10, eps2d=0.017)


def to_device(scene: Dict, device) -> Dict:
    return {k: (v.to(device) if torch.is_tensor(v) else v) for k, v in scene.items()}
