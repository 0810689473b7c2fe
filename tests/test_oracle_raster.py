"""Pins for the oracle's compositing loops and spherical harmonics (CPU only).

  * compositing: a vectorised numpy restatement (cumprod over the depth-sorted list,
    no sequential loop) on scenes where every Gaussian reaches every tile, so the tile
    lists are the global depth order; single-Gaussian closed form; termination rule;
  * lidar extras: the 10 co-located Gaussians known-answer case of the reference's
    tests/test_basic.py:1257-1281 for alpha_sum_until_points; median depth; wrap-around
    of the angular difference; inactive points (range <= 0) stay zero;
  * SH: real spherical harmonics from scipy.special (Condon-Shortley phase kept) and
    orthonormality under quadrature.
"""
import math

import numpy as np
import pytest
import scipy.special

import oracle


def _vectorised_composite(alpha_raw, sigma):
    """alpha_raw, sigma: [P, G] in depth order. Returns weights [P, G] and final T [P]."""
    valid = (sigma >= 0) & (alpha_raw >= 1.0 / 255.0)
    a = np.where(valid, alpha_raw, 0.0)
    T_incl = np.cumprod(1.0 - a, axis=1)
    T_excl = np.concatenate([np.ones((a.shape[0], 1)), T_incl[:, :-1]], axis=1)
    stop = valid & (T_incl <= 1e-4)
    alive = np.cumsum(stop, axis=1) == 0
    w = a * T_excl * alive
    Tf = np.prod(np.where(alive, 1.0 - a, 1.0), axis=1)
    return w, Tf, alive & valid


def _all_tiles_scene(seed, C, N, W, H, D, big_opacity=False):
    rng = np.random.default_rng(seed)
    means2d = np.stack([rng.uniform(0, W, (C, N)), rng.uniform(0, H, (C, N))], -1).astype(np.float32)
    s = rng.uniform(2.0, 12.0, (C, N, 2))
    rho = rng.uniform(-0.7, 0.7, (C, N))
    cov = np.zeros((C, N, 2, 2))
    cov[..., 0, 0] = s[..., 0] ** 2; cov[..., 1, 1] = s[..., 1] ** 2
    cov[..., 0, 1] = cov[..., 1, 0] = rho * s[..., 0] * s[..., 1]
    inv = np.linalg.inv(cov)
    conics = np.stack([inv[..., 0, 0], inv[..., 0, 1], inv[..., 1, 1]], -1).astype(np.float32)
    colors = rng.normal(size=(C, N, D)).astype(np.float32)
    opac = (rng.uniform(0.5, 1.0, (C, N)) if big_opacity else rng.uniform(0.05, 0.9, (C, N))).astype(np.float32)
    depths = rng.uniform(1, 10, (C, N)).astype(np.float32)
    pix_vels = (rng.normal(size=(C, N, 2)) * 30).astype(np.float32)
    radii = np.full((C, N, 2), 10000, np.int32)
    return means2d, conics, colors, opac, depths, pix_vels, radii


@pytest.mark.parametrize("D,big", [(3, False), (5, True)])
def test_pixels_against_vectorised_restatement(D, big):
    C, N, W, H, ts = 2, 150 if not big else 400, 40, 24, 8
    tw, th = math.ceil(W / ts), math.ceil(H / ts)
    means2d, conics, colors, opac, depths, pix_vels, radii = _all_tiles_scene(11, C, N, W, H, D, big)
    rs = np.array([0.02, 0.0], np.float32)
    bg = np.random.default_rng(1).uniform(size=(C, D)).astype(np.float32)
    _, ids, flat = oracle.isect_tiles(means2d, radii, depths, ts, tw, th)
    offs = oracle.isect_offset_encode(ids, C, tw, th)
    rc, ra, last = oracle.rasterize_to_pixels_fwd(means2d, conics, colors, opac, pix_vels, rs, bg,
                                                  W, H, ts, offs, flat, precision="f64")
    n_stopped = 0
    for c in range(C):
        order = np.argsort(depths[c], kind="stable")
        jj, ii = np.meshgrid(np.arange(W), np.arange(H))
        px = (jj + 0.5).reshape(-1, 1); py = (ii + 0.5).reshape(-1, 1)
        roll = rs[c] * (ii.reshape(-1, 1) / (H - 1) - 0.5)
        m = means2d[c][order].astype(np.float64); v = pix_vels[c][order].astype(np.float64)
        q = conics[c][order].astype(np.float64)
        dx = m[None, :, 0] + roll * v[None, :, 0] - px
        dy = m[None, :, 1] + roll * v[None, :, 1] - py
        sigma = 0.5 * (q[None, :, 0] * dx * dx + q[None, :, 2] * dy * dy) + q[None, :, 1] * dx * dy
        alpha = np.minimum(0.999, opac[c][order].astype(np.float64)[None] * np.exp(-sigma))
        w, Tf, used = _vectorised_composite(alpha, sigma)
        img = w @ colors[c][order].astype(np.float64) + Tf[:, None] * bg[c].astype(np.float64)
        np.testing.assert_allclose(rc[c].reshape(-1, D), img, rtol=1e-9, atol=1e-9)
        np.testing.assert_allclose(ra[c].reshape(-1), 1 - Tf, rtol=1e-9, atol=1e-12)
        n_stopped += int((used.sum(1) < ((sigma >= 0) & (alpha >= 1 / 255)).sum(1)).sum())
        # last_ids: position (in the sorted list) of the last contributing Gaussian
        any_used = used.any(1)
        last_pos = np.where(any_used, used.shape[1] - 1 - np.argmax(used[:, ::-1], axis=1), 0)
        tile_of_pix = (ii // ts * tw + jj // ts).reshape(-1)
        exp_last = np.where(any_used, offs[c].reshape(-1)[tile_of_pix] + last_pos, 0)
        np.testing.assert_array_equal(last[c].reshape(-1), exp_last)
    if big:
        assert n_stopped > 100  # the early-termination rule was exercised


def test_pixels_single_gaussian_closed_form_and_f32():
    W, H, ts = 16, 16, 16
    means2d = np.array([[[8.5, 8.5]]], np.float32)
    conics = np.array([[[0.1, 0.0, 0.1]]], np.float32)
    colors = np.array([[[0.2, 0.5, 0.9]]], np.float32)
    opac = np.array([[0.8]], np.float32)
    zeros2 = np.zeros((1, 1, 2), np.float32)
    bg = np.array([[1.0, 0.0, 0.5]], np.float32)
    offs = np.zeros((1, 1, 1), np.int32)
    flat = np.zeros((1,), np.int32)
    for prec, tol in (("f64", 1e-7), ("f32", 1e-6)):
        rc, ra, last = oracle.rasterize_to_pixels_fwd(means2d, conics, colors, opac, zeros2,
                                                      np.zeros(1, np.float32), bg, W, H, ts, offs,
                                                      flat, precision=prec)
        a = 0.8  # centre pixel (8, 8): delta = 0
        np.testing.assert_allclose(rc[0, 8, 8], a * colors[0, 0] + (1 - a) * bg[0], atol=tol)
        np.testing.assert_allclose(ra[0, 8, 8, 0], a, atol=tol)
        # pixel (8, 11): delta = (-3, 0) -> sigma = 0.45
        a = 0.8 * math.exp(-0.45)
        np.testing.assert_allclose(rc[0, 8, 11], a * colors[0, 0] + (1 - a) * bg[0], atol=tol)
        # far corner: alpha < 1/255 -> background only, alpha 0
        np.testing.assert_allclose(rc[0, 0, 0], bg[0], atol=tol)
        assert ra[0, 0, 0, 0] == 0


def test_pixels_opaque_stack_terminates_exclusively():
    # alpha is capped at 0.999: T after 1, 2 Gaussians = 1e-3, 1e-6.  The second one would take
    # T below 1e-4, so the pixel stops BEFORE adding it (rasterization.cu:1485-1488).
    W = H = ts = 4
    n = 3
    means2d = np.tile(np.array([[[2.5, 2.5]]], np.float32), (1, n, 1))
    conics = np.tile(np.array([[[1e-6, 0.0, 1e-6]]], np.float32), (1, n, 1))
    colors = np.array([[[1.0], [10.0], [100.0]]], np.float32)
    opac = np.ones((1, n), np.float32)
    offs = np.zeros((1, 1, 1), np.int32)
    flat = np.arange(n, dtype=np.int32)
    rc, ra, last = oracle.rasterize_to_pixels_fwd(means2d, conics, colors, opac,
                                                  np.zeros((1, n, 2), np.float32),
                                                  np.zeros(1, np.float32), None, W, H, ts, offs,
                                                  flat, precision="f64")
    np.testing.assert_allclose(rc[0, 2, 2, 0], 0.999 * 1.0, rtol=1e-6)
    np.testing.assert_allclose(ra[0, 2, 2, 0], 0.999, rtol=1e-6)
    assert last[0, 2, 2] == 0


def _lidar_grid(H, W, rng_val=50.0):
    az = -180.0 + (np.arange(W) + 0.5) * 360.0 / W
    el = np.linspace(-20, 20, H)
    rp = np.zeros((1, H, W, 4), np.float32)
    rp[0, :, :, 0] = az[None]; rp[0, :, :, 1] = el[:, None]; rp[0, :, :, 2] = rng_val
    return rp


def test_points_alpha_sum_known_answer_case():
    # tests/test_basic.py:1257-1281: 10 Gaussians co-located 0.1 deg off one test point at
    # range 85, depths linspace(20, 120, 10), threshold 0.5 -> the first six are in front.
    H, W, tw, th = 32, 1800, 64, 4
    el = np.linspace(-45.01, 45.01, H)
    az = np.linspace(-180 + 0.1, 180 - 0.1, W)
    rp = np.zeros((1, H, W, 4), np.float32)
    rp[0, :, :, 0] = az[None]; rp[0, :, :, 1] = el[:, None]
    ti, tj, trange = 16, 900, 85.0
    rp[0, ti, tj, 2] = trange
    n = 10
    means2d = np.tile((rp[0, ti, tj, :2] + 0.1)[None, None], (1, n, 1)).astype(np.float32)
    radii = np.ones((1, n, 2), np.float32)
    conics = np.tile(np.array([[[1.0, 0.0, 1.0]]], np.float32), (1, n, 1))
    depths = np.linspace(20.0, 120.0, n, dtype=np.float32)[None]
    opac = np.full((1, n), 0.3, np.float32)
    feats = np.concatenate([np.random.default_rng(0).normal(size=(1, n, 5)).astype(np.float32),
                            depths[..., None]], -1)
    eb = np.linspace(-45.02, 45.02, H // th + 1).astype(np.float32)
    res = 0.2 * tw
    n_az = math.ceil(360 / res)
    _, ids, flat = oracle.isect_lidar_tiles(means2d, radii, depths, eb, res, -180.0)
    offs = oracle.isect_offset_encode(ids, 1, n_az, H // th)
    rc, ra, last, asum, med = oracle.rasterize_to_points_fwd(
        means2d, conics, feats, opac, np.zeros((1, n, 3), np.float32),
        np.zeros((1, n, 2), np.float32), None, rp, W, H, tw, th, True, 0.5, offs, flat, 5,
        precision="f64")
    d = means2d[0, 0].astype(np.float64) - rp[0, ti, tj, :2].astype(np.float64)
    a = 0.3 * math.exp(-0.5 * (d[0] ** 2 + d[1] ** 2))
    np.testing.assert_allclose(asum[0, ti, tj, 0], 6 * a, rtol=1e-6)
    np.testing.assert_allclose(ra[0, ti, tj, 0], 1 - (1 - a) ** n, rtol=1e-6)
    w = a * (1 - a) ** np.arange(n)
    np.testing.assert_allclose(rc[0, ti, tj], w @ feats[0].astype(np.float64), rtol=1e-6, atol=1e-9)
    # T crosses 0.5 at the 2nd Gaussian (0.7^2 = 0.49): median depth is its depth
    assert (1 - a) > 0.5 >= (1 - a) ** 2
    np.testing.assert_allclose(med[0, ti, tj, 0], depths[0, 1], rtol=1e-6)
    # every other point has range 0 -> inactive, outputs stay zero
    mask = np.ones((H, W), bool); mask[ti, tj] = False
    assert (rc[0][mask] == 0).all() and (ra[0][mask] == 0).all() and (asum[0][mask] == 0).all()


def test_points_against_vectorised_restatement_with_wrap_and_depth_terms():
    H, W, tw, th, D = 8, 64, 16, 4, 4   # D-1 features + depth channel
    rng = np.random.default_rng(3)
    N = 120
    rp = _lidar_grid(H, W)
    rp[0, :, :, 2] = rng.uniform(5, 60, (H, W))
    rp[0, :, :, 3] = rng.normal(size=(H, W)) * 0.05
    rp[0, 0, :5, 2] = 0.0                       # inactive points
    means2d = np.stack([rng.uniform(-180, 180, N), rng.uniform(-25, 25, N)], -1)[None].astype(np.float32)
    s = rng.uniform(4.0, 30.0, (N, 2))
    conics = np.stack([1 / s[:, 0] ** 2, np.zeros(N), 1 / s[:, 1] ** 2], -1)[None].astype(np.float32)
    conics[0, :, 1] = rng.uniform(-0.3, 0.3, N) / (s[:, 0] * s[:, 1])
    depths = rng.uniform(1, 70, (1, N)).astype(np.float32)
    feats = np.concatenate([rng.normal(size=(1, N, D - 1)).astype(np.float32), depths[..., None]], -1)
    opac = rng.uniform(0.05, 0.6, (1, N)).astype(np.float32)
    pv = (rng.normal(size=(1, N, 3)) * 20).astype(np.float32)
    dc = (rng.normal(size=(1, N, 2)) * 0.5).astype(np.float32)
    # hand-made tile lists: every tile holds all N Gaussians in depth order
    n_tiles = (W // tw) * (H // th)
    order0 = np.argsort(depths[0], kind="stable").astype(np.int32)
    flat = np.tile(order0, n_tiles)
    offs = (np.arange(n_tiles, dtype=np.int32) * N).reshape(1, H // th, W // tw)
    thr = 0.3
    rc, ra, last, asum, med = oracle.rasterize_to_points_fwd(
        means2d, conics, feats, opac, pv, dc, None, rp, W, H, tw, th, True, thr, offs, flat, D - 1,
        precision="f64")
    order = np.argsort(depths[0], kind="stable")
    P = rp[0].reshape(-1, 4).astype(np.float64)
    m = means2d[0][order].astype(np.float64); v = pv[0][order].astype(np.float64)
    q = conics[0][order].astype(np.float64); k = dc[0][order].astype(np.float64)

    def wrap(d):  # signed angular difference in (-180, 180]
        return (d + 180.0) % 360.0 - 180.0

    dx = wrap(m[None, :, 0] + P[:, 3:4] * v[None, :, 0] - P[:, 0:1])
    dy = wrap(m[None, :, 1] + P[:, 3:4] * v[None, :, 1] - P[:, 1:2])
    sigma = 0.5 * (q[None, :, 0] * dx * dx + q[None, :, 2] * dy * dy) + q[None, :, 1] * dx * dy
    alpha = np.minimum(0.999, opac[0][order].astype(np.float64)[None] * np.exp(-sigma))
    w, Tf, used = _vectorised_composite(alpha, sigma)
    active = P[:, 2] > 0
    f = feats[0][order].astype(np.float64)
    img = w @ f
    extra = k[None, :, 0] * dx + k[None, :, 1] * dy + v[None, :, 2] * P[:, 3:4]
    img[:, D - 1] += (w * extra).sum(1)
    img *= active[:, None]
    np.testing.assert_allclose(rc[0].reshape(-1, D), img, rtol=1e-8, atol=1e-8)
    np.testing.assert_allclose(ra[0].reshape(-1), (1 - Tf) * active, rtol=1e-9, atol=1e-12)
    before = f[None, :, D - 1] < (P[:, 2:3] - thr)
    np.testing.assert_allclose(asum[0].reshape(-1), (alpha * used * before).sum(1) * active,
                               rtol=1e-9, atol=1e-12)
    # median depth: the used Gaussian at which T crosses 0.5
    a_eff = np.where(used, alpha, 0.0)
    T_incl = np.cumprod(1 - a_eff, axis=1)
    T_excl = np.concatenate([np.ones((len(P), 1)), T_incl[:, :-1]], 1)
    cross = used & (T_excl > 0.5) & (T_incl <= 0.5)
    exp_med = ((f[None, :, D - 1] + extra) * cross).sum(1) * active
    np.testing.assert_allclose(med[0].reshape(-1), exp_med, rtol=1e-9, atol=1e-9)
    assert cross.any() and (np.abs(dx) > 170).any()   # both features were exercised


# ------------------------------------------------------------------ SH
def _real_sh_scipy(deg, dirs):
    x, y, z = (dirs / np.linalg.norm(dirs, axis=-1, keepdims=True)).T
    theta = np.arctan2(y, x)          # azimuth
    phi = np.arccos(np.clip(z, -1, 1))  # polar
    out = []
    for l in range(deg + 1):
        for m in range(-l, l + 1):
            Y = scipy.special.sph_harm_y(l, abs(m), phi, theta)  # includes (-1)^m
            if m == 0:
                out.append(Y.real)
            elif m > 0:
                out.append(math.sqrt(2) * Y.real)
            else:
                out.append(math.sqrt(2) * Y.imag)
    return np.stack(out, -1)


@pytest.mark.parametrize("deg", [0, 1, 2, 3, 4])
def test_sh_against_scipy_and_orthonormality(deg):
    rng = np.random.default_rng(deg)
    n, K = 500, 25
    dirs = rng.normal(size=(n, 3)).astype(np.float32) * 3.0   # not normalised on purpose
    nb = (deg + 1) ** 2
    basis_ref = _real_sh_scipy(deg, dirs.astype(np.float64))
    # basis function k of the oracle = colour with a one-hot coefficient
    for k in range(nb):
        coeffs = np.zeros((n, K, 3), np.float32)
        coeffs[:, k, :] = [1.0, 2.0, -1.0]
        col = oracle.spherical_harmonics(deg, dirs, coeffs, precision="f64")
        np.testing.assert_allclose(col[:, 0], basis_ref[:, k], atol=2e-7)
        np.testing.assert_allclose(col[:, 1], 2 * col[:, 0], atol=1e-12)
        np.testing.assert_allclose(col[:, 2], -col[:, 0], atol=1e-12)
    # coefficients beyond the active degree are ignored; masks zero the row
    coeffs = rng.normal(size=(n, K, 3)).astype(np.float32)
    col = oracle.spherical_harmonics(deg, dirs, coeffs, precision="f64")
    np.testing.assert_allclose(col, np.einsum("nk,nkc->nc", basis_ref, coeffs[:, :nb].astype(np.float64)),
                               atol=5e-6)
    masks = rng.random(n) > 0.5
    colm = oracle.spherical_harmonics(deg, dirs, coeffs, masks=masks, precision="f64")
    assert (colm[~masks] == 0).all()
    np.testing.assert_array_equal(colm[masks], col[masks])
    if deg == 0:
        np.testing.assert_allclose(col, 0.2820947917738781 * coeffs[:, 0].astype(np.float64), rtol=1e-7)


def test_sh_constants_orthonormal_under_quadrature():
    # Gauss-Legendre in cos(polar) x uniform in azimuth integrates degree-8 polynomials exactly
    xs, ws = np.polynomial.legendre.leggauss(12)
    az = (np.arange(24) + 0.5) * 2 * math.pi / 24
    Z, A = np.meshgrid(xs, az, indexing="ij")
    Wt = (ws[:, None] * np.full_like(A, 2 * math.pi / 24)).reshape(-1)
    s = np.sqrt(1 - Z ** 2)
    dirs = np.stack([s * np.cos(A), s * np.sin(A), Z], -1).reshape(-1, 3).astype(np.float32)
    n = dirs.shape[0]
    B = []
    for k in range(25):
        coeffs = np.zeros((n, 25, 3), np.float32)
        coeffs[:, k, 0] = 1.0
        B.append(oracle.spherical_harmonics(4, dirs, coeffs, precision="f64")[:, 0])
    B = np.stack(B, -1)
    gram = B.T @ (B * Wt[:, None])
    np.testing.assert_allclose(gram, np.eye(25), atol=2e-6)
