"""GPU parity of the (Gaussian, pixel) index lists and of compositing over them.

  * lists of the HIP kernels against the CPU oracle's on the same inputs: identical per pixel
    on all but a sliver of the pixels (a pair whose alpha or transmittance sits within float32
    rounding of a threshold may legitimately fall on either side; the kernel evaluates exp2 of
    a pre-scaled exponent, the oracle exp);
  * the recipe of the reference's tests/test_basic.py:893-1013 and :1016-1200: compositing the
    lists in plain torch (`_rasterize_to_pixels`, `_rasterize_to_points`) must reproduce the
    fused kernels, values and autograd gradients against the hand-written backward kernels.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from tests.gpu_util import DEV, assert_close, to_dev, to_np
from tests.test_gpu_backward import _raster_scene, assert_grad_close
from tests.test_gpu_forward import _lidar_scene, _projected_scene

pytestmark = pytest.mark.gpu

LIST_FRAC = 0.999  # pixels whose whole list must be identical (at most two may differ on small images)


def _pixel_signature(g, rays, n_rays):
    """Per pixel: (number of pairs, order-sensitive checksum of its Gaussian ids)."""
    counts = np.bincount(rays, minlength=n_rays)
    starts = np.cumsum(counts) - counts
    rank = np.arange(rays.shape[0]) - starts[rays]
    check = np.bincount(rays, weights=((g + 1) * (rank % 1021 + 1)).astype(np.float64), minlength=n_rays)
    return counts, check


def _assert_lists_match(got, want, n_rays, hw, name):
    g_g, p_g, c_g = (to_np(t) for t in got)
    g_o, p_o, c_o = want
    assert g_g.dtype == np.int64 and p_g.dtype == np.int64 and c_g.dtype == np.int64
    rays_g, rays_o = c_g * hw + p_g, c_o * hw + p_o
    assert (np.diff(rays_g) >= 0).all(), f"{name}: pixels out of order"
    cnt_g, chk_g = _pixel_signature(g_g, rays_g, n_rays)
    cnt_o, chk_o = _pixel_signature(g_o, rays_o, n_rays)
    same = (cnt_g == cnt_o) & (chk_g == chk_o)
    n_diff, allowed = int((~same).sum()), max(2, int((1 - LIST_FRAC) * n_rays))
    assert n_diff <= allowed, f"{name}: {n_diff} of {n_rays} pixel lists differ"
    assert abs(int(cnt_g.sum()) - int(cnt_o.sum())) <= 2e-3 * max(1, int(cnt_o.sum())), name
    if same.all():
        np.testing.assert_array_equal(g_g, g_o)
        np.testing.assert_array_equal(p_g, p_o)
    return int(cnt_o.sum())


@pytest.mark.parametrize("ts,W,H", [(16, 200, 136), (8, 77, 50), (4, 30, 21), (5, 33, 17)])
def test_indices_in_range_against_oracle(ts, W, H):
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_indices_in_range
    C, N = 2, 2500
    s = _projected_scene(C, N, W, H, 3, seed=70 + ts)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    _, ids, flat = isect_tiles(s["means2d"], s["radii"], s["depths"], ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    rng = np.random.default_rng(ts)
    longest = int(np.diff(np.append(to_np(offs).reshape(-1), flat.shape[0])).max())
    n_batches = math.ceil(longest / (ts * ts))
    windows = [(0, 10 ** 10, np.ones((C, H, W), np.float32)),
               (1, max(2, n_batches // 2), rng.uniform(0.0, 1.0, (C, H, W)).astype(np.float32)),
               (n_batches, n_batches + 5, np.ones((C, H, W), np.float32))]
    args_o = [to_np(s[k]) for k in ("means2d", "conics", "opacities", "pix_vels")]
    total = 0
    for lo, hi, T in windows:
        got = rasterize_to_indices_in_range(lo, hi, to_dev(T), s["means2d"], s["conics"], s["opacities"],
                                            s["pix_vels"], W, H, ts, offs, flat, s["rs"])
        want = oracle.rasterize_to_indices_in_range(lo, hi, T, *args_o, W, H, ts, to_np(offs),
                                                    to_np(flat), to_np(s["rs"]))
        total += _assert_lists_match(got, want, C * H * W, H * W, f"ts={ts} [{lo},{hi})")
        if lo == n_batches:
            assert got[0].shape == (0,)
    assert total > 5 * H * W
    # without a rolling-shutter time the pixels are taken at the mid-exposure pose
    got = rasterize_to_indices_in_range(0, 3, to_dev(windows[0][2]), s["means2d"], s["conics"],
                                        s["opacities"], s["pix_vels"], W, H, ts, offs, flat)
    want = oracle.rasterize_to_indices_in_range(0, 3, windows[0][2], *args_o, W, H, ts, to_np(offs), to_np(flat))
    _assert_lists_match(got, want, C * H * W, H * W, "no rolling shutter")


def test_indices_in_range_saturating_scene_and_empty_inputs():
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_indices_in_range
    C, N, W, H, ts = 1, 30000, 96, 64, 16
    s = _projected_scene(C, N, W, H, 3, seed=3, rs=(0.0,))
    s["opacities"] = torch.full_like(s["opacities"], 0.95)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    _, ids, flat = isect_tiles(s["means2d"], s["radii"], s["depths"], ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    ones = np.ones((C, H, W), np.float32)
    got = rasterize_to_indices_in_range(0, 10 ** 10, to_dev(ones), s["means2d"], s["conics"], s["opacities"],
                                        s["pix_vels"], W, H, ts, offs, flat, s["rs"])
    want = oracle.rasterize_to_indices_in_range(0, 10 ** 10, ones, to_np(s["means2d"]), to_np(s["conics"]),
                                                to_np(s["opacities"]), to_np(s["pix_vels"]), W, H, ts,
                                                to_np(offs), to_np(flat), to_np(s["rs"]))
    n = _assert_lists_match(got, want, H * W, H * W, "saturating")
    assert n > H * W
    # no intersections at all
    e = rasterize_to_indices_in_range(0, 5, to_dev(ones), s["means2d"], s["conics"], s["opacities"],
                                      s["pix_vels"], W, H, ts, torch.zeros_like(offs), flat[:0], s["rs"])
    assert all(t.shape == (0,) and t.dtype == torch.int64 for t in e)
    # zero transmittance everywhere: the first pair of every pixel already stops it
    e = rasterize_to_indices_in_range(0, 5, to_dev(0 * ones), s["means2d"], s["conics"], s["opacities"],
                                      s["pix_vels"], W, H, ts, offs, flat, s["rs"])
    assert e[0].shape == (0,)
    with pytest.raises(RuntimeError, match="not ordered"):
        rasterize_to_indices_in_range(4, 2, to_dev(ones), s["means2d"], s["conics"], s["opacities"],
                                      s["pix_vels"], W, H, ts, offs, flat, s["rs"])


@pytest.mark.parametrize("tw,th,W,H", [(32, 4, 256, 16), (16, 4, 120, 14), (8, 2, 100, 9)])
def test_indices_in_range_lidar_against_oracle(tw, th, W, H):
    from splatad_amd import isect_lidar_tiles, isect_offset_encode, rasterize_to_indices_in_range_lidar
    H_s, W_s = math.ceil(H / th) * th, math.ceil(W / tw) * tw
    d, proj = _lidar_scene(8000, 80 + tw, H_s, W_s, tw, th, 5)
    radii, means2d, depths, conics, _, pix_vels, _ = proj
    res = d["azimuth_resolution"] * tw
    _, ids, flat = isect_lidar_tiles(means2d, radii, depths, d["tile_elevation_boundaries"], res, -180.0)
    offs = isect_offset_encode(ids, 1, W_s // tw, H_s // th)
    pts = d["raster_pts"][:, :H, :W].contiguous()      # a point image the tile grid overhangs
    opac = d["opacities"][None].contiguous()
    rng = np.random.default_rng(tw)
    args_o = [to_np(t) for t in (means2d, conics, opac, pix_vels, pts)]
    for lo, hi, T in [(0, 10 ** 10, np.ones((1, H, W), np.float32)),
                      (1, 4, rng.uniform(0, 1, (1, H, W)).astype(np.float32))]:
        got = rasterize_to_indices_in_range_lidar(lo, hi, to_dev(T), means2d, conics, opac, pix_vels, pts,
                                                  W, H, tw, th, offs, flat)
        want = oracle.rasterize_to_indices_in_range_lidar(lo, hi, T, *args_o, W, H, tw, th, to_np(offs),
                                                          to_np(flat))
        n = _assert_lists_match(got, want, H * W, H * W, f"lidar {tw}x{th} [{lo},{hi})")
        assert n > H * W
        inactive = np.nonzero(to_np(pts)[0, :, :, 2].reshape(-1) <= 0)[0]
        assert inactive.shape[0] >= 7 and not np.isin(to_np(got[1]), inactive).any()


@pytest.mark.parametrize("D,ts,per_iter", [(3, 16, 100), (5, 8, 100), (3, 4, 1000)])
def test_list_compositing_reproduces_fused_pixels_with_gradients(D, ts, per_iter):
    from splatad_amd import isect_offset_encode, isect_tiles, rasterize_to_pixels
    from splatad_amd.hip._torch_impl import _rasterize_to_pixels
    C, N, W, H = 2, 600, 72, 40
    means2d, conics, colors, opac, depths, pix_vels, radii, bg = _raster_scene(90 + D, C, N, W, H, D)
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    rs = to_dev(np.array([0.03, 0.0], np.float32))
    _, ids, flat = isect_tiles(to_dev(means2d), to_dev(radii), to_dev(depths), ts, tw, th)
    offs = isect_offset_encode(ids, C, tw, th)
    names = ("means2d", "conics", "colors", "opacities", "pix_vels", "backgrounds")
    fused = [to_dev(x).requires_grad_() for x in (means2d, conics, colors, opac, pix_vels, bg)]
    lists = [to_dev(x).requires_grad_() for x in (means2d, conics, colors, opac, pix_vels, bg)]
    rc, ra = rasterize_to_pixels(fused[0], fused[1], fused[2], fused[3], fused[4], W, H, ts, offs, flat,
                                 rolling_shutter_time=rs, backgrounds=fused[5])
    l_rc, l_ra = _rasterize_to_pixels(lists[0], lists[1], lists[2], lists[3], lists[4], W, H, ts, offs, flat,
                                      rs, backgrounds=lists[5], batch_per_iter=per_iter)
    assert_close(to_np(l_rc), to_np(rc), atol=1e-4, name="colors")
    assert_close(to_np(l_ra), to_np(ra), atol=1e-4, name="alphas")
    rng = np.random.default_rng(1)
    wc = to_dev(rng.normal(size=tuple(rc.shape)).astype(np.float32))
    wa = to_dev(rng.normal(size=tuple(ra.shape)).astype(np.float32))
    g_f = torch.autograd.grad((rc * wc).sum() + (ra * wa).sum(), fused)
    g_l = torch.autograd.grad((l_rc * wc).sum() + (l_ra * wa).sum(), lists)
    for n, a, b in zip(names, g_f, g_l):
        assert_grad_close(to_np(a), to_np(b), f"{n} D={D}")


@pytest.mark.parametrize("asum", [True, False])
def test_list_compositing_reproduces_fused_points_with_gradients(asum):
    from splatad_amd import isect_lidar_tiles, isect_offset_encode, rasterize_to_points
    from splatad_amd.hip._torch_impl import _rasterize_to_points
    H, W, tw, th, D = 16, 256, 32, 4, 5
    d, proj = _lidar_scene(3000, 95, H, W, tw, th, D)
    radii, means2d, depths, conics, _, pix_vels, dcomp = proj
    res = d["azimuth_resolution"] * tw
    _, ids, flat = isect_lidar_tiles(means2d, radii, depths, d["tile_elevation_boundaries"], res, -180.0)
    offs = isect_offset_encode(ids, 1, W // tw, H // th)
    feats = torch.cat([d["lidar_features"], depths[..., None]], -1)
    opac = d["opacities"][None].contiguous()
    names = ("means2d", "conics", "features", "opacities", "pix_vels", "depth_compensations")
    base = (means2d, conics, feats, opac, pix_vels, dcomp)
    fused = [t.detach().clone().requires_grad_() for t in base]
    lists = [t.detach().clone().requires_grad_() for t in base]
    rf, ra, rsum, _ = rasterize_to_points(*fused, d["raster_pts"], W, H, tw, th, offs, flat, asum, 0.3)
    l_rf, l_ra, l_sum = _rasterize_to_points(*lists, d["raster_pts"], W, H, tw, th, offs, flat, asum, 0.3)
    assert_close(to_np(l_rf), to_np(rf), atol=2e-4, rtol=1e-4, name="features")
    assert_close(to_np(l_ra), to_np(ra), atol=1e-4, name="alphas")
    rng = np.random.default_rng(2)
    wf = to_dev(rng.normal(size=tuple(rf.shape)).astype(np.float32))
    wa = to_dev(rng.normal(size=tuple(ra.shape)).astype(np.float32))
    loss_f, loss_l = (rf * wf).sum() + (ra * wa).sum(), (l_rf * wf).sum() + (l_ra * wa).sum()
    if asum:
        assert_close(to_np(l_sum), to_np(rsum), atol=1e-4, rtol=1e-4, name="alpha_sum")
        ws = to_dev(rng.normal(size=tuple(rsum.shape)).astype(np.float32))
        loss_f, loss_l = loss_f + (rsum * ws).sum(), loss_l + (l_sum * ws).sum()
    else:
        assert l_sum is None
    g_f = torch.autograd.grad(loss_f, fused)
    g_l = torch.autograd.grad(loss_l, lists)
    for n, a, b in zip(names, g_f, g_l):
        assert_grad_close(to_np(a), to_np(b), n)
