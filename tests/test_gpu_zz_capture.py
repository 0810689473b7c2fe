"""The two-call operators hand a count to the waiting host, which a stream under graph capture
would never deliver: they have to refuse with an error instead of waiting for ever."""
import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = torch.device("cuda:0")


def _inputs():
    g = torch.Generator(device=DEV).manual_seed(5)
    C, N = 1, 2000
    means2d = torch.rand((C, N, 2), device=DEV, generator=g) * 256
    radii = torch.randint(1, 20, (C, N, 2), device=DEV, dtype=torch.int32, generator=g)
    depths = torch.rand((C, N), device=DEV, generator=g) * 10 + 0.1
    return means2d, radii, depths


def test_isect_refuses_graph_capture():
    from splatad_amd.hip._backend import _C
    means2d, radii, depths = _inputs()
    # the same call outside a capture works
    out = _C.isect_tiles(means2d, radii, depths, None, None, 1, 16, 16, 16, True, True)
    assert out[1].numel() > 0
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="captured"):
        with torch.cuda.graph(graph):
            _C.isect_tiles(means2d, radii, depths, None, None, 1, 16, 16, 16, True, True)
    torch.cuda.synchronize()
    # and the library is still usable afterwards
    again = _C.isect_tiles(means2d, radii, depths, None, None, 1, 16, 16, 16, True, True)
    assert torch.equal(again[1], out[1]) and torch.equal(again[2], out[2])


def test_packed_projection_refuses_graph_capture():
    from splatad_amd import workloads
    from splatad_amd.hip._backend import _C
    s = workloads.to_device(workloads.camera_driving(n=3000), DEV)
    args = (s["means"], None, s["quats"], s["scales"], s["velocities"], s["viewmats"], s["Ks"],
            s["width"], s["height"], s["linear_velocity"], s["angular_velocity"],
            s["rolling_shutter_time"], s["eps2d"], s["near_plane"], s["far_plane"], 0.0, False)
    out = _C.fully_fused_projection_packed_fwd(*args)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with pytest.raises(RuntimeError, match="captured"):
        with torch.cuda.graph(graph):
            _C.fully_fused_projection_packed_fwd(*args)
    torch.cuda.synchronize()
    again = _C.fully_fused_projection_packed_fwd(*args)
    assert torch.equal(again[1], out[1]) and torch.equal(again[2], out[2])
