"""`rasterize_to_pixels_with_sh` -- the compositing kernel that evaluates the view-dependent
colours of the entries it stages -- against the two operators it stands for,
`view_dependent_colors` (gsplat/rendering.py:325-347 of the reference: directions, spherical
harmonics, max(c + 1/2, 0)) followed by `rasterize_to_pixels` (rasterization.cu:1360-1518),
which other tests compare with the oracle.  The bar is equality bit for bit: both paths run
the same instructions on the same values.
"""
import math

import pytest
import torch

from splatad_amd import workloads
from tests.gpu_util import DEV

pytestmark = pytest.mark.gpu


def _projected(C, N, W, H, tile_size, packed, seed):
    from splatad_amd import fully_fused_projection, isect_offset_encode, isect_tiles
    s = workloads.camera_driving(n=N, seed=seed, width=W, height=H, n_cameras=C, with_velocities=True)
    d = workloads.to_device(s, DEV)
    proj = fully_fused_projection(d["means"], None, d["quats"], d["scales"], d["velocities"], d["viewmats"],
                                  d["Ks"], W, H, d["linear_velocity"], d["angular_velocity"],
                                  d["rolling_shutter_time"], eps2d=d["eps2d"], near_plane=d["near_plane"],
                                  far_plane=d["far_plane"], packed=packed)
    if packed:
        camera_ids, gaussian_ids, radii, means2d, depths, conics, _, pix_vels = proj
        opacities = d["opacities"][gaussian_ids]
    else:
        radii, means2d, depths, conics, _, pix_vels = proj
        camera_ids = gaussian_ids = None
        opacities = d["opacities"].expand(C, -1).contiguous()
    tw, th = math.ceil(W / tile_size), math.ceil(H / tile_size)
    _, isect_ids, flatten_ids = isect_tiles(means2d, radii, depths, tile_size, tw, th, packed=packed,
                                            n_cameras=C, camera_ids=camera_ids, gaussian_ids=gaussian_ids)
    offsets = isect_offset_encode(isect_ids, C, tw, th)
    return d, dict(radii=radii, means2d=means2d, depths=depths, conics=conics, pix_vels=pix_vels,
                   opacities=opacities, camera_ids=camera_ids, gaussian_ids=gaussian_ids,
                   offsets=offsets, flatten_ids=flatten_ids)


@pytest.mark.parametrize("C,degree,per_sensor,with_depth,tile_size,packed", [
    (1, 3, False, True, 16, False),   # the driving camera's case: two pixels per lane, RGB+D
    (1, 3, False, False, 16, False),
    (3, 3, True, True, 16, False),    # coefficients of their own per camera
    (2, 0, False, True, 16, False),
    (2, 1, False, False, 16, True),
    (2, 2, True, True, 16, True),
    (2, 4, False, True, 16, True),    # 25 coefficients
    (2, 4, True, False, 8, False),
    (1, 3, False, True, 4, False),    # one pixel per lane
    (2, 3, False, True, 8, True),
])
def test_colours_evaluated_while_compositing_equal_the_two_operators(C, degree, per_sensor, with_depth,
                                                                      tile_size, packed):
    from splatad_amd.hip._wrapper import (rasterize_to_pixels, rasterize_to_pixels_with_sh,
                                          view_dependent_colors)
    N, W, H = 6000, 200, 120
    d, p = _projected(C, N, W, H, tile_size, packed, seed=20 + degree)
    g = torch.Generator(device=DEV).manual_seed(3)
    K = (degree + 1) ** 2 + (2 if degree == 2 else 0)  # more coefficients than the degree uses, once
    coeffs = torch.randn(((C, N) if per_sensor else (N,)) + (K, 3), device=DEV, generator=g) * 0.4
    bg = torch.rand((C, 4 if with_depth else 3), device=DEV, generator=g)
    depths = p["depths"] if with_depth else None
    with torch.no_grad():
        colors = view_dependent_colors(degree, d["means"], d["viewmats"], coeffs, p["radii"], depths,
                                       p["camera_ids"], p["gaussian_ids"])
        want = rasterize_to_pixels(p["means2d"], p["conics"], colors, p["opacities"], p["pix_vels"], W, H,
                                   tile_size, p["offsets"], p["flatten_ids"], d["rolling_shutter_time"],
                                   backgrounds=bg, packed=packed)
        got = rasterize_to_pixels_with_sh(degree, d["means"], d["viewmats"], coeffs, depths, p["means2d"],
                                          p["conics"], p["opacities"], p["pix_vels"], W, H, tile_size,
                                          p["offsets"], p["flatten_ids"], d["rolling_shutter_time"],
                                          backgrounds=bg, gaussian_ids=p["gaussian_ids"])
    assert got[0].shape == want[0].shape == (C, H, W, 4 if with_depth else 3)
    assert float(want[1].max()) > 0.5 and float(want[1].min()) < 0.5  # rendered, and not everywhere
    assert torch.equal(got[1], want[1])
    assert torch.equal(got[0], want[0])


@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("with_depth", [False, True])
def test_colour_cache_empty_or_filled_by_the_opacity_a_tile_carries(packed, with_depth):
    """view_dependent_color_cache leaves every row NaN where the visible Gaussians carry enough
    opacity per tile for tiles to saturate early, and otherwise holds what view_dependent_colors
    makes for the visible rows; compositing renders the same image from either."""
    from splatad_amd.hip._wrapper import (MIN_OPACITY_PER_TILE, rasterize_to_pixels,
                                          rasterize_to_pixels_with_sh, view_dependent_color_cache,
                                          view_dependent_colors)
    C, N, W, H, ts = 2, 6000, 200, 120, 16
    d, p = _projected(C, N, W, H, ts, packed, seed=31)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    coeffs = torch.randn((N, 16, 3), device=DEV, generator=torch.Generator(device=DEV).manual_seed(8)) * 0.4
    depths = p["depths"] if with_depth else None
    visible = p["radii"][..., 0] > 0
    # the estimate the kernels make, restated: opacity x tiles met (from the radii, at most the grid)
    gid = p["gaussian_ids"] if packed else torch.arange(N, device=DEV).expand(C, N)
    r = p["radii"].float()
    tiles = (2 * r[..., 0] / ts + 1).clamp(max=tw) * (2 * r[..., 1] / ts + 1).clamp(max=th)
    estimate = float((d["opacities"][gid] * tiles)[visible & (p["radii"][..., 1] > 0)].sum()) / (C * tw * th)
    assert 4 < estimate < 0.5 * MIN_OPACITY_PER_TILE  # a sparse little scene: the default fills
    with torch.no_grad():
        colors = view_dependent_colors(3, d["means"], d["viewmats"], coeffs, p["radii"], depths,
                                       p["camera_ids"], p["gaussian_ids"])
        want = rasterize_to_pixels(p["means2d"], p["conics"], colors, p["opacities"], p["pix_vels"], W, H,
                                   ts, p["offsets"], p["flatten_ids"], d["rolling_shutter_time"], packed=packed)
        for limit, filled in ((0.0, False), (0.5 * estimate, False), (2.0 * estimate, True),
                              (float("inf"), True), (None, True)):
            cache = view_dependent_color_cache(3, d["means"], d["viewmats"], coeffs, p["radii"], depths,
                                               d["opacities"], ts, tw, th, p["camera_ids"], p["gaussian_ids"],
                                               min_opacity_per_tile=limit)
            assert cache.shape == tuple(visible.shape) + (4,)
            if filled:
                assert torch.equal(cache[visible][:, :3], colors[visible][:, :3])
                assert torch.equal(cache[visible][:, 3],
                                   depths[visible] if with_depth else torch.zeros_like(cache[visible][:, 3]))
                assert bool(torch.isnan(cache[~visible]).all())
            else:
                assert bool(torch.isnan(cache).all())
            got = rasterize_to_pixels_with_sh(3, d["means"], d["viewmats"], coeffs, depths, p["means2d"],
                                              p["conics"], p["opacities"], p["pix_vels"], W, H, ts, p["offsets"],
                                              p["flatten_ids"], d["rolling_shutter_time"],
                                              gaussian_ids=p["gaussian_ids"], color_cache=cache)
            assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
            if not filled:  # the rows that tiles staged now hold their colours, the others still NaN
                held = ~torch.isnan(cache[..., 0])
                assert bool(held.any()) and not bool(held[~visible].any())
                assert torch.equal(cache[held][:, :3], colors[held][:, :3])


def test_colours_while_compositing_checks_its_rows_and_what_a_gradient_needs():
    from splatad_amd.hip._wrapper import rasterize_to_pixels_with_sh
    d, p = _projected(1, 500, 64, 48, 16, False, seed=4)
    coeffs = torch.zeros((500, 16, 3), device=DEV)
    args = (3, d["means"], d["viewmats"], coeffs, None, p["means2d"], p["conics"], p["opacities"],
            p["pix_vels"], 64, 48, 16, p["offsets"], p["flatten_ids"])
    rc, ra = rasterize_to_pixels_with_sh(*args)
    # zero coefficients: every colour is max(0 + 1/2, 0), so a pixel holds alpha / 2
    torch.testing.assert_close(rc, (0.5 * ra).expand(-1, -1, -1, 3), atol=1e-6, rtol=1e-6)
    with pytest.raises(ValueError, match="gradients need `radii`"):
        rasterize_to_pixels_with_sh(3, d["means"], d["viewmats"], coeffs.clone().requires_grad_(), *args[4:])
    with pytest.raises(ValueError, match="view matrices"):
        rasterize_to_pixels_with_sh(3, d["means"], d["viewmats"].clone().requires_grad_(), *args[3:],
                                    radii=p["radii"])
    with pytest.raises(AssertionError):  # degree 4 needs 25 coefficients
        rasterize_to_pixels_with_sh(4, *args[1:])


@pytest.mark.parametrize("C,degree,with_depth,packed,absgrad", [
    (1, 3, True, False, False),   # the driving camera's training step
    (2, 3, False, False, True),
    (2, 2, True, True, False),
    (2, 1, True, True, True),
])
def test_gradients_through_colours_evaluated_while_compositing_equal_the_two_operators(C, degree, with_depth,
                                                                                      packed, absgrad):
    """The backward pass of `rasterize_to_pixels_with_sh` composites with the colours the forward
    kernel left in its cache (rows no tile staged count as zero: no pixel's gradient reaches
    them) and sends the colour gradients through the colour kernel's backward pass.  Every
    gradient has to equal the one of `view_dependent_colors` + `rasterize_to_pixels`, which
    other tests compare with the float64 oracle, up to the order of the float32 sums."""
    from splatad_amd.hip._wrapper import (rasterize_to_pixels, rasterize_to_pixels_with_sh,
                                          view_dependent_colors)
    N, W, H, ts = 5000, 160, 96, 16
    d, p = _projected(C, N, W, H, ts, packed, seed=40 + degree)
    g = torch.Generator(device=DEV).manual_seed(5)
    coeffs0 = torch.randn((N, (degree + 1) ** 2, 3), device=DEV, generator=g) * 0.4
    bg0 = torch.rand((C, 4 if with_depth else 3), device=DEV, generator=g)
    weights = torch.rand((C, H, W, 5 if with_depth else 4), device=DEV, generator=g)
    names = ("means", "coeffs", "depths", "means2d", "conics", "opacities", "backgrounds")

    def leaves():
        out = dict(means=d["means"], coeffs=coeffs0, depths=p["depths"] if with_depth else None,
                   means2d=p["means2d"], conics=p["conics"], opacities=p["opacities"], backgrounds=bg0)
        return {k: (None if v is None else v.detach().clone().requires_grad_()) for k, v in out.items()}

    def loss(render):
        return (torch.cat(render, dim=-1) * weights).sum()

    a = leaves()
    if absgrad:
        a["means2d"].absgrad = None
    colors = view_dependent_colors(degree, a["means"], d["viewmats"], a["coeffs"], p["radii"], a["depths"],
                                   p["camera_ids"], p["gaussian_ids"])
    want = rasterize_to_pixels(a["means2d"], a["conics"], colors, a["opacities"], p["pix_vels"], W, H, ts,
                               p["offsets"], p["flatten_ids"], d["rolling_shutter_time"],
                               backgrounds=a["backgrounds"], packed=packed, absgrad=absgrad)
    loss(want).backward()
    b = leaves()
    got = rasterize_to_pixels_with_sh(degree, b["means"], d["viewmats"], b["coeffs"], b["depths"], b["means2d"],
                                      b["conics"], b["opacities"], p["pix_vels"], W, H, ts, p["offsets"],
                                      p["flatten_ids"], d["rolling_shutter_time"], backgrounds=b["backgrounds"],
                                      gaussian_ids=p["gaussian_ids"], radii=p["radii"],
                                      camera_ids=p["camera_ids"], absgrad=absgrad)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
    loss(got).backward()
    for k in names:
        if a[k] is None:
            continue
        assert b[k].grad is not None and float(a[k].grad.abs().max()) > 0, k
        scale = float(a[k].grad.abs().max())
        torch.testing.assert_close(b[k].grad, a[k].grad, atol=2e-5 * scale, rtol=1e-4, msg=lambda m, k=k: f"{k}: {m}")
    if absgrad:
        scale = float(a["means2d"].absgrad.abs().max())
        torch.testing.assert_close(b["means2d"].absgrad, a["means2d"].absgrad, atol=2e-5 * scale, rtol=1e-4)


def test_rasterization_renders_the_same_image_when_a_gradient_is_wanted():
    """rasterization() renders the same image, bit for bit, whether or not an input takes a
    gradient, and the gradient reaches the coefficients."""
    from splatad_amd import rasterization
    s = workloads.camera_driving(n=8000, width=256, height=144, n_cameras=2)
    d = workloads.to_device(s, DEV)
    kw = dict(near_plane=d["near_plane"], far_plane=d["far_plane"], eps2d=d["eps2d"], tile_size=16,
              sh_degree=3, render_mode="RGB+ED", backgrounds=torch.rand((2, 3), device=DEV))
    rest = (d["velocities"], d["viewmats"], d["Ks"], d["width"], d["height"], d["linear_velocity"],
            d["angular_velocity"], d["rolling_shutter_time"])
    for packed in (False, True):
        with torch.no_grad():
            plain = rasterization(d["means"], d["quats"], d["scales"], d["opacities"], d["colors"], *rest,
                                  packed=packed, **kw)
        leaf = d["colors"].clone().requires_grad_()
        grad = rasterization(d["means"], d["quats"], d["scales"], d["opacities"], leaf, *rest, packed=packed, **kw)
        assert grad[0].requires_grad and not plain[0].requires_grad
        assert torch.equal(grad[0].detach(), plain[0]) and torch.equal(grad[1].detach(), plain[1])
        grad[0].sum().backward()
        assert float(leaf.grad.abs().sum()) > 0


def test_colours_that_are_not_numbers_equal_the_two_operators():
    """A colour cache row that is "not evaluated" is told by NaN; a row whose evaluated colour is
    itself NaN (infinite or NaN coefficients, a NaN depth channel) therefore stays "not
    evaluated" and every workgroup that stages it evaluates it again, to the same bits.  The
    render has to equal the two operators' there too, NaN for NaN."""
    from splatad_amd.hip._wrapper import (rasterize_to_pixels, rasterize_to_pixels_with_sh,
                                          view_dependent_colors)
    C, N, W, H, degree = 2, 6000, 200, 120, 3
    d, p = _projected(C, N, W, H, 16, False, seed=31)
    g = torch.Generator(device=DEV).manual_seed(5)
    coeffs = torch.randn((N, 16, 3), device=DEV, generator=g) * 0.4
    bad = torch.randperm(N, generator=torch.Generator().manual_seed(6))[:300].to(DEV)
    coeffs[bad[:100], 0, 0] = float("nan")
    coeffs[bad[100:200], 5, 1] = float("inf")
    coeffs[bad[200:300], 9, 2] = -float("inf")
    depths = p["depths"].clone()
    depths[:, bad[250:]] = float("nan")
    with torch.no_grad():
        colors = view_dependent_colors(degree, d["means"], d["viewmats"], coeffs, p["radii"], depths)
        want = rasterize_to_pixels(p["means2d"], p["conics"], colors, p["opacities"], p["pix_vels"], W, H, 16,
                                   p["offsets"], p["flatten_ids"], d["rolling_shutter_time"])
        got = rasterize_to_pixels_with_sh(degree, d["means"], d["viewmats"], coeffs, depths, p["means2d"],
                                          p["conics"], p["opacities"], p["pix_vels"], W, H, 16, p["offsets"],
                                          p["flatten_ids"], d["rolling_shutter_time"])
    assert torch.isnan(want[0]).any() and not torch.isnan(want[0]).all()
    assert torch.equal(torch.isnan(got[0]), torch.isnan(want[0]))
    assert torch.equal(torch.nan_to_num(got[0], nan=-1.0), torch.nan_to_num(want[0], nan=-1.0))
    assert torch.equal(got[1], want[1])


def test_work_beside_the_sort_is_done_once_and_joined():
    """isect_tiles(beside_work=...) calls the callable exactly once, from inside the fill call with
    the library's launches on a stream of the sort's, and what it enqueued is complete for the
    caller's stream when the call returns: the colour cache made there (with every row evaluated,
    i.e. its filling kernel at work) equals the one made afterwards; the lists are the same; a
    call that sorts nothing, a call without intersections and a failing callable behave."""
    from splatad_amd import fully_fused_projection, isect_tiles
    from splatad_amd.hip._wrapper import view_dependent_color_cache
    C, N, W, H, ts = 2, 50000, 320, 192, 16
    d = workloads.to_device(workloads.camera_driving(n=N, seed=3, width=W, height=H, n_cameras=C), DEV)
    radii, means2d, depths, conics, _, pix_vels = fully_fused_projection(
        d["means"], None, d["quats"], d["scales"], d["velocities"], d["viewmats"], d["Ks"], W, H,
        d["linear_velocity"], d["angular_velocity"], d["rolling_shutter_time"], eps2d=d["eps2d"],
        near_plane=d["near_plane"], far_plane=d["far_plane"], packed=False)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    cache_args = (3, d["means"], d["viewmats"], d["colors"], radii, depths, d["opacities"], ts, tw, th, None, None)
    made = []

    def work():
        # (a threshold that no scene reaches: the second launch evaluates every visible row)
        made.append(view_dependent_color_cache(*cache_args, min_opacity_per_tile=1e30))

    for sort in (True, False):
        made.clear()
        got = isect_tiles(means2d, radii, depths, ts, tw, th, sort=sort, beside_work=work)
        want = isect_tiles(means2d, radii, depths, ts, tw, th, sort=sort)
        assert len(made) == 1
        for g, w in zip(got, want):
            assert torch.equal(g, w)
        direct = view_dependent_color_cache(*cache_args, min_opacity_per_tile=1e30)
        visible = radii[..., 0] > 0
        assert visible.any() and not torch.isnan(made[0][visible]).any()
        assert torch.equal(made[0][visible], direct[visible]) and torch.isnan(made[0][~visible]).all()
    # nothing to intersect: the work is still done, on the caller's stream
    made.clear()
    none = isect_tiles(means2d, torch.zeros_like(radii), depths, ts, tw, th, beside_work=work)
    assert len(made) == 1 and none[1].numel() == 0

    def failing():
        raise ValueError("from the callable")

    with pytest.raises(ValueError, match="from the callable"):
        isect_tiles(means2d, radii, depths, ts, tw, th, beside_work=failing)
    # and the library is in order afterwards
    again = isect_tiles(means2d, radii, depths, ts, tw, th)
    assert again[1].numel() == want[1].numel() > 0
