"""Pins for the oracle's index lists and list compositing, and for the torch compositing that
ships in splatad_amd.hip._torch_impl (CPU only; that module is plain torch and runs anywhere).

  * index lists: closed-form counts for stacks of identical Gaussians (geometric transmittance,
    batch windows, a start transmittance below 1); agreement with the separately pinned fused
    compositing oracle (the last pair of a pixel is its `last_ids` entry, compositing the lists
    reproduces the fused render -- the recipe of the reference's tests/test_basic.py:893-1013,
    which compares `rasterize_to_pixels` with `_rasterize_to_pixels`); windows over batches
    concatenate to the one-step list when no pixel saturates; lidar: wrap-around pairs exist,
    points with range <= 0 have none;
  * list compositing (`_composite_rays`, the restated nerfacc definitions): geometric closed
    form and the fused oracle as above;
  * torch `accumulate` / `accumulate_lidar`: against the numpy oracle on the same lists,
    closed form for `_weights_along_rays`, gradcheck in float64.
"""
import math

import numpy as np
import pytest
import torch

import oracle
from test_oracle_raster import _all_tiles_scene, _lidar_grid


def _stack_scene(n, opacity, W=4, H=4):
    """n identical, huge Gaussians over a WxH image: alpha == opacity at every pixel."""
    means2d = np.full((1, n, 2), 2.0, np.float32)
    conics = np.tile(np.array([[[1e-12, 0.0, 1e-12]]], np.float32), (1, n, 1))
    opac = np.full((1, n), opacity, np.float32)
    pix_vels = np.zeros((1, n, 2), np.float32)
    return means2d, conics, opac, pix_vels


def test_index_counts_closed_form_geometric_stack():
    # T after k Gaussians is (1 - o)^k; Gaussian k+1 is taken iff (1 - o)^(k+1) > 1e-4
    ts, W, H, n = 2, 4, 4, 40
    means2d, conics, opac, pv = _stack_scene(n, 0.5)
    tw = th = 2
    flat = np.tile(np.arange(n, dtype=np.int32), tw * th)
    offs = (np.arange(tw * th, dtype=np.int32) * n).reshape(1, th, tw)
    ones = np.ones((1, H, W), np.float32)
    g, p, c = oracle.rasterize_to_indices_in_range(0, 10 ** 10, ones, means2d, conics, opac, pv,
                                                   W, H, ts, offs, flat)
    taken = max(k for k in range(n) if 0.5 ** k > 1e-4)          # 13
    assert taken == 13 and g.shape[0] == taken * W * H
    assert (c == 0).all()
    # row-major pixels, each with Gaussians 0..12 in order
    np.testing.assert_array_equal(p, np.repeat(np.arange(W * H), taken))
    np.testing.assert_array_equal(g, np.tile(np.arange(taken), W * H))
    # batches are ts*ts = 4 entries: window [1, 3) covers entries 4..11; starting from
    # T = 0.5^4 the stop comes where 0.5^4 * 0.5^k <= 1e-4 -> 9 more could be taken, 8 exist
    T4 = np.full((1, H, W), 0.5 ** 4, np.float32)
    g, p, c = oracle.rasterize_to_indices_in_range(1, 3, T4, means2d, conics, opac, pv, W, H, ts,
                                                   offs, flat)
    np.testing.assert_array_equal(g, np.tile(np.arange(4, 12), W * H))
    # window [3, 100) from T = 0.5^12: only entry 12 still passes
    T12 = np.full((1, H, W), 0.5 ** 12, np.float32)
    g, _, _ = oracle.rasterize_to_indices_in_range(3, 100, T12, means2d, conics, opac, pv, W, H,
                                                   ts, offs, flat)
    np.testing.assert_array_equal(g, np.full(W * H, 12))
    # a window past the end of every list, and an empty window
    for lo, hi in ((10, 20), (2, 2)):
        g, _, _ = oracle.rasterize_to_indices_in_range(lo, hi, ones, means2d, conics, opac, pv, W,
                                                       H, ts, offs, flat)
        assert g.shape == (0,)
    # below 1/255 nothing is taken; gaussian ids are reduced modulo N for several cameras
    means2, conics2, opac2, pv2 = (np.concatenate([a, a]) for a in (means2d, conics, opac, pv))
    opac2[0] = 1.0 / 300.0
    flat2 = np.concatenate([flat, flat + n]); offs2 = np.concatenate([offs, offs + flat.shape[0]])
    g, p, c = oracle.rasterize_to_indices_in_range(0, 100, np.ones((2, H, W), np.float32), means2,
                                                   conics2, opac2, pv2, W, H, ts, offs2, flat2)
    assert (c == 1).all() and g.max() == taken - 1 and g.shape[0] == taken * W * H


@pytest.mark.parametrize("big", [False, True])
def test_lists_agree_with_fused_compositing_oracle(big):
    C, N, W, H, ts, D = 2, 300 if big else 120, 40, 24, 8, 3
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    means2d, conics, colors, opac, depths, pix_vels, radii = _all_tiles_scene(5, C, N, W, H, D, big)
    rs = np.array([0.03, 0.0], np.float32)
    _, ids, flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    offs = oracle.isect_offset_encode(ids, C, tw, th)
    ones = np.ones((C, H, W), np.float32)
    rc, ra, last = oracle.rasterize_to_pixels_fwd(means2d, conics, colors, opac, pix_vels, rs, None,
                                                  W, H, ts, offs, flat, precision="f64")
    g, p, c = oracle.rasterize_to_indices_in_range(0, 10 ** 6, ones, means2d, conics, opac,
                                                   pix_vels, W, H, ts, offs, flat, rs,
                                                   precision="f64")
    rays = c * H * W + p
    assert (np.diff(rays) >= 0).all()                      # row-major pixels, camera by camera
    # last pair of every non-empty pixel = the fused loop's last contributing Gaussian
    ends = np.nonzero(np.append(np.diff(rays) != 0, True))[0]
    np.testing.assert_array_equal(g[ends], flat[last.reshape(-1)[rays[ends]]] % N)
    # a pixel without pairs rendered nothing
    empty = np.ones(C * H * W, bool); empty[rays] = False
    assert (ra.reshape(-1)[empty] == 0).all()
    # depth order within a pixel
    same = np.diff(rays) == 0
    assert (np.diff(depths[c, g])[same] >= 0).all()
    # compositing the lists reproduces the fused render
    img, acc = oracle.accumulate(means2d, conics, opac, colors, pix_vels, rs, g, p, c, W, H)
    np.testing.assert_allclose(img, rc, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(acc, ra, rtol=1e-9, atol=1e-12)
    if big:
        assert (ra > 0.9998).mean() > 0.2                  # saturating pixels are covered


def test_batch_windows_concatenate_when_nothing_saturates():
    C, N, W, H, ts = 1, 200, 24, 16, 4
    tw, th = W // ts, H // ts
    means2d, conics, _, opac, depths, pix_vels, radii = _all_tiles_scene(9, C, N, W, H, 1)
    opac = (opac * 0.02).astype(np.float32) + 0.004        # some below 1/255, none saturates
    _, ids, flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    offs = oracle.isect_offset_encode(ids, C, tw, th)
    ones = np.ones((C, H, W), np.float32)
    full = oracle.rasterize_to_indices_in_range(0, 10 ** 9, ones, means2d, conics, opac, pix_vels,
                                                W, H, ts, offs, flat)
    parts = [oracle.rasterize_to_indices_in_range(lo, lo + 3, ones, means2d, conics, opac,
                                                  pix_vels, W, H, ts, offs, flat)
             for lo in range(0, math.ceil(N / (ts * ts)), 3)]
    g = np.concatenate([q[0] for q in parts]); p = np.concatenate([q[1] for q in parts])
    order = np.argsort(p, kind="stable")                   # windows are in front-to-back order
    np.testing.assert_array_equal(p[order], full[1])
    np.testing.assert_array_equal(g[order], full[0])
    assert full[0].shape[0] > 1000


def test_lidar_lists_wrap_inactive_points_and_fused_oracle():
    H, W, tw, th, D = 8, 64, 16, 4, 4
    rng = np.random.default_rng(4)
    N = 90
    rp = _lidar_grid(H, W)
    rp[0, :, :, 2] = rng.uniform(5, 60, (H, W)); rp[0, :, :, 3] = rng.normal(size=(H, W)) * 0.05
    rp[0, 0, :5, 2] = 0.0; rp[0, 5, 7, 2] = -3.0
    means2d = np.stack([rng.uniform(-180, 180, N), rng.uniform(-25, 25, N)], -1)[None].astype(np.float32)
    means2d[0, 0] = (179.5, 0.0)                           # reaches the points at -177.2 across the seam
    s = rng.uniform(4.0, 30.0, (N, 2)); s[0] = (3.0, 30.0)
    conics = np.stack([1 / s[:, 0] ** 2, np.zeros(N), 1 / s[:, 1] ** 2], -1)[None].astype(np.float32)
    depths = rng.uniform(1, 70, (1, N)).astype(np.float32); depths[0, 0] = 0.5
    feats = np.concatenate([rng.normal(size=(1, N, D - 1)).astype(np.float32), depths[..., None]], -1)
    opac = rng.uniform(0.05, 0.6, (1, N)).astype(np.float32); opac[0, 0] = 0.9
    pv = (rng.normal(size=(1, N, 3)) * 20).astype(np.float32); pv[0, 0] = 0
    dc = (rng.normal(size=(1, N, 2)) * 0.5).astype(np.float32)
    n_tiles = (W // tw) * (H // th)
    flat = np.tile(np.argsort(depths[0], kind="stable").astype(np.int32), n_tiles)
    offs = (np.arange(n_tiles, dtype=np.int32) * N).reshape(1, H // th, W // tw)
    ones = np.ones((1, H, W), np.float32)
    g, p, c = oracle.rasterize_to_indices_in_range_lidar(0, 10 ** 6, ones, means2d, conics, opac, pv,
                                                         rp, W, H, tw, th, offs, flat, precision="f64")
    inactive = np.nonzero(rp[0, :, :, 2].reshape(-1) <= 0)[0]
    assert inactive.shape[0] == 6 and not np.isin(p, inactive).any()
    # Gaussian 0 (azimuth 179.5, sigma 3 deg) is the first pair of the point at azimuth -177.2
    # (3.3 deg away through the seam), elevation row 4
    pix = 4 * W + 0
    assert abs(rp[0, 4, 0, 0] + 177.1875) < 1e-3
    assert g[p == pix][0] == 0
    rc, ra, _, asum, _ = oracle.rasterize_to_points_fwd(means2d, conics, feats, opac, pv, dc, None, rp,
                                                        W, H, tw, th, True, 0.3, offs, flat, D - 1,
                                                        precision="f64")
    img, acc, s_acc = oracle.accumulate_lidar(means2d, conics, opac, feats, pv, dc, rp, g, p, c, W, H,
                                              True, 0.3)
    np.testing.assert_allclose(img, rc, rtol=1e-9, atol=1e-11)
    np.testing.assert_allclose(acc, ra, rtol=1e-9, atol=1e-12)
    np.testing.assert_allclose(s_acc, asum, rtol=1e-9, atol=1e-12)


def test_composite_rays_geometric_closed_form():
    a, n = 0.3, 7
    alphas = np.full(2 * n + 1, a); rays = np.array([2] * n + [5] * n + [6])
    vals = np.ones((2 * n + 1, 2)); vals[:, 1] = np.arange(2 * n + 1)
    out, acc = oracle._composite_rays(alphas, vals, rays, 8)
    np.testing.assert_allclose(acc[[2, 5], 0], 1 - (1 - a) ** n, rtol=1e-12)
    np.testing.assert_allclose(acc[6, 0], a)
    w = a * (1 - a) ** np.arange(n)
    np.testing.assert_allclose(out[5, 1], w @ np.arange(n, 2 * n), rtol=1e-12)
    assert (out[[0, 1, 3, 4, 7]] == 0).all()


# ------------------------------------------------------------------- shipped torch compositing
def _t(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype)


def test_torch_weights_along_rays_closed_form_and_long_lists():
    from splatad_amd.hip._torch_impl import _sum_along_rays, _weights_along_rays
    a, n = 0.25, 9
    alphas = torch.full((3 * n,), a)
    rays = torch.tensor([0] * n + [3] * n + [4] * n)
    w, T = _weights_along_rays(alphas, rays)
    expect = (1 - a) ** np.arange(n)
    for k in range(3):
        np.testing.assert_allclose(T[k * n:(k + 1) * n].numpy(), expect, rtol=1e-6)
    np.testing.assert_allclose(w.numpy(), np.tile(a * expect, 3), rtol=1e-6)
    acc = _sum_along_rays(w, None, rays, 6)
    np.testing.assert_allclose(acc[:, 0].numpy(), [1 - (1 - a) ** n, 0, 0, 1 - (1 - a) ** n,
                                                   1 - (1 - a) ** n, 0], rtol=1e-6, atol=1e-7)
    # two million samples in rays of 20: the one cumulative sum must not lose the small rays
    m = 2_000_000
    rng = np.random.default_rng(0)
    al = torch.from_numpy(rng.uniform(0.004, 0.999, m).astype(np.float32))
    ry = torch.arange(m) // 20
    _, T = _weights_along_rays(al, ry)
    ref = np.cumprod(1 - al.double().numpy().reshape(-1, 20), axis=1)
    ref = np.concatenate([np.ones((m // 20, 1)), ref[:, :-1]], axis=1).reshape(-1)
    np.testing.assert_allclose(T.numpy(), ref, rtol=2e-6, atol=1e-30)
    assert _weights_along_rays(al[:0], ry[:0])[0].shape == (0,)


def test_torch_accumulate_against_oracle_lists():
    from splatad_amd.hip._torch_impl import accumulate
    C, N, W, H, ts, D = 2, 150, 24, 16, 8, 5
    tw, th = W // ts, H // ts
    means2d, conics, colors, opac, depths, pix_vels, radii = _all_tiles_scene(2, C, N, W, H, D)
    rs = np.array([0.03, -0.01], np.float32)
    _, ids, flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    offs = oracle.isect_offset_encode(ids, C, tw, th)
    g, p, c = oracle.rasterize_to_indices_in_range(0, 10 ** 6, np.ones((C, H, W), np.float32), means2d,
                                                   conics, opac, pix_vels, W, H, ts, offs, flat, rs)
    img, acc = oracle.accumulate(means2d, conics, opac, colors, pix_vels, rs, g, p, c, W, H)
    t_img, t_acc = accumulate(_t(means2d), _t(conics), _t(opac), _t(colors), _t(pix_vels), _t(rs),
                              _t(g, torch.int64), _t(p, torch.int64), _t(c, torch.int64), W, H)
    assert t_img.shape == (C, H, W, D) and t_acc.shape == (C, H, W, 1)
    np.testing.assert_allclose(t_img.numpy(), img, atol=2e-5, rtol=1e-4)
    np.testing.assert_allclose(t_acc.numpy(), acc, atol=1e-5, rtol=1e-5)
    # empty list
    e = torch.zeros(0, dtype=torch.int64)
    z_img, z_acc = accumulate(_t(means2d), _t(conics), _t(opac), _t(colors), _t(pix_vels), _t(rs),
                              e, e, e, W, H)
    assert float(z_img.abs().max()) == 0 and float(z_acc.abs().max()) == 0


def test_torch_accumulate_lidar_against_oracle_lists_and_gradcheck():
    from splatad_amd.hip._torch_impl import accumulate_lidar
    H, W, tw, th, D, N = 4, 32, 16, 4, 3, 40
    rng = np.random.default_rng(8)
    rp = _lidar_grid(H, W)
    rp[0, :, :, 2] = rng.uniform(5, 60, (H, W)); rp[0, :, :, 3] = rng.normal(size=(H, W)) * 0.05
    rp[0, 1, 3, 2] = 0.0
    means2d = np.stack([rng.uniform(-180, 180, N), rng.uniform(-25, 25, N)], -1)[None].astype(np.float32)
    s = rng.uniform(6.0, 40.0, (N, 2))
    conics = np.stack([1 / s[:, 0] ** 2, rng.uniform(-0.3, 0.3, N) / (s[:, 0] * s[:, 1]),
                       1 / s[:, 1] ** 2], -1)[None].astype(np.float32)
    depths = rng.uniform(1, 70, (1, N)).astype(np.float32)
    feats = np.concatenate([rng.normal(size=(1, N, D - 1)).astype(np.float32), depths[..., None]], -1)
    opac = rng.uniform(0.05, 0.6, (1, N)).astype(np.float32)
    pv = (rng.normal(size=(1, N, 3)) * 20).astype(np.float32)
    dc = (rng.normal(size=(1, N, 2)) * 0.5).astype(np.float32)
    n_tiles = (W // tw) * (H // th)
    flat = np.tile(np.argsort(depths[0], kind="stable").astype(np.int32), n_tiles)
    offs = (np.arange(n_tiles, dtype=np.int32) * N).reshape(1, H // th, W // tw)
    g, p, c = oracle.rasterize_to_indices_in_range_lidar(0, 100, np.ones((1, H, W), np.float32),
                                                         means2d, conics, opac, pv, rp, W, H, tw, th,
                                                         offs, flat)
    ref = oracle.accumulate_lidar(means2d, conics, opac, feats, pv, dc, rp, g, p, c, W, H, True, 0.3)
    ids = [_t(a, torch.int64) for a in (g, p, c)]
    out = accumulate_lidar(_t(means2d), _t(conics), _t(opac), _t(feats), _t(pv), _t(dc), _t(rp), *ids,
                           W, H, True, 0.3)
    for got, want, name in zip(out, ref, ("features", "alphas", "alpha_sum")):
        np.testing.assert_allclose(got.numpy(), want, atol=5e-5, rtol=1e-4, err_msg=name)
    assert accumulate_lidar(_t(means2d), _t(conics), _t(opac), _t(feats), _t(pv), _t(dc), _t(rp), *ids,
                            W, H, False, 0.3)[2] is None
    # autograd through the compositing (float64, a slice of the list)
    keep = p < 12
    ids = [_t(a[keep], torch.int64) for a in (g, p, c)]
    leaves = [_t(a, torch.float64).requires_grad_() for a in (means2d, conics, opac, feats, pv, dc)]

    def f(*x):
        r, a, s_ = accumulate_lidar(*x, _t(rp, torch.float64), *ids, W, H, True, 0.3)
        return r, a, s_

    assert torch.autograd.gradcheck(f, leaves, eps=1e-6, atol=1e-5, rtol=1e-4, nondet_tol=1e-12)
