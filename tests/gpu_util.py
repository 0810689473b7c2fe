"""Helpers shared by the GPU parity tests."""
import itertools

import numpy as np
import torch

import oracle

DEV = torch.device("cuda:0")


def to_np(t):
    if t is None or isinstance(t, np.ndarray):
        return t
    return t.detach().cpu().numpy()


def to_dev(a, dtype=None):
    if a is None:
        return None
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def assert_close(actual, expected, atol, rtol=0.0, frac=1.0, name="", outlier_bound=None):
    """|a - e| <= atol + rtol |e| on at least `frac` of the elements, and |a - e| <=
    outlier_bound on every element (required when frac < 1: no element may differ by an
    arbitrary amount)."""
    a = np.asarray(actual, dtype=np.float64)
    e = np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (name, a.shape, e.shape)
    assert frac >= 1.0 or outlier_bound is not None, f"{name}: a tolerated fraction needs an outlier bound"
    if a.size == 0:
        return
    diff = np.abs(a - e)
    bad = ~(diff <= atol + rtol * np.abs(e))
    ok_frac = 1.0 - bad.mean()
    worst = float(diff.max()) if np.isfinite(diff).all() else float("inf")
    if ok_frac < frac or (outlier_bound is not None and not worst <= outlier_bound):
        idx = np.argwhere(bad)[:5]
        raise AssertionError(
            f"{name}: {bad.sum()}/{a.size} elements off (max |diff| {worst:.3e}, atol {atol}, "
            f"rtol {rtol}, outlier bound {outlier_bound}); first at {idx.tolist()}: got {a[tuple(idx[0])]}, "
            f"want {e[tuple(idx[0])]}")


# Compositing takes discontinuous decisions per (pixel, Gaussian): alpha >= 1/255, next
# transmittance <= 1e-4, and for lidar points the transmittance crossing 0.5 (median depth) and
# depth < range - threshold (alpha sum).  A float32 kernel whose alpha or transmittance differs
# from the float64 oracle's in the last bits lands on the other side for inputs within rounding
# distance of a threshold; that pixel then differs by up to ~alpha * colour.  The comparison
# below finds those pixels instead of tolerating a fraction blindly: the oracle renders again
# with the thresholds moved by a few float32 rounding errors (relative 3e-5 on alpha, whose
# float32 error is ~1e-6 of the exponent; 3e-4 on the transmittance, which accumulates one
# rounding per composited Gaussian).  A pixel whose oracle value is the same under every such
# move depends on no near-threshold decision and must meet the tolerance, no exception.  A pixel
# whose value moves must equal one of the variants.
ALPHA_NUDGE = 3e-5
T_NUDGE = 3e-4
MEDIAN_NUDGE = 3e-5  # the transmittance near 0.5 carries ~1e-6 of relative float32 error
ASUM_NUDGE = 1e-4  # metres, absolute (float32 spacing at 100 m is 8e-6)


def decision_variants(lidar=False):
    """Keyword sets for oracle.nudged_thresholds: the nominal one first."""
    out = []
    for da, dt in itertools.product((0.0, ALPHA_NUDGE, -ALPHA_NUDGE), (0.0, T_NUDGE, -T_NUDGE)):
        out.append(dict(alpha_scale=1.0 + da, t_scale=1.0 + dt))
    if lidar:
        for dm in (MEDIAN_NUDGE, -MEDIAN_NUDGE):
            out.append(dict(median_scale=1.0 + dm))
        for ds in (ASUM_NUDGE, -ASUM_NUDGE):
            out.append(dict(asum_shift=ds))
    return out


def render_variants(render, lidar=False):
    """render() -> dict name -> float64 array [..., channels]; returns the list of such dicts,
    one per decision variant (nominal first), rendered by the float64 oracle."""
    outs = []
    for kw in decision_variants(lidar):
        with oracle.nudged_thresholds("f64", **kw):
            outs.append(render())
    return outs


def assert_matches_oracle_decisions(got, variants, tols, name="", max_attributed=1.5e-2, max_ambiguous=None):
    """got: dict name -> array [..., ch]; variants: list of such dicts from render_variants();
    tols: dict name -> (atol, rtol).  Per output and pixel (all leading axes):
      * oracle value identical under every variant -> |got - nominal| <= atol + rtol |nominal|
        on every channel, no exception;
      * otherwise (a decision of that pixel sits within a few rounding errors of its
        threshold) got must meet the tolerance against one of the variants; at most
        `max_ambiguous` pixels per output may match none (two near-threshold decisions in one
        pixel, moved in opposite directions), and those must lie within the variants' spread.
        By default none (no test of this suite, up to the 1920x1080 frames, has needed one);
        the number used is printed and returned.
    The near-threshold pixels may be at most `max_attributed` of all pixels (a plausibility
    bound: every saturating pixel ends on a transmittance decision, and a window of 6e-4 around
    1e-4 catches about half a per cent of them; measured 0.67 % on the 1920x1080 benchmark frame).
    Returns {name: (attributed pixels, pixels that differ from the nominal render, ambiguous pixels)}."""
    report = {}
    for key, (atol, rtol) in tols.items():
        g = np.asarray(got[key], np.float64)
        vs = [np.asarray(v[key], np.float64) for v in variants]
        nominal = vs[0]
        assert g.shape == nominal.shape, (name, key, g.shape, nominal.shape)
        assert np.isfinite(g).all(), f"{name} {key}: non-finite values"
        ok = [(np.abs(g - v) <= atol + rtol * np.abs(v)).all(-1) for v in vs]
        attributed = np.zeros(nominal.shape[:-1], bool)
        for v in vs[1:]:
            attributed |= (v != nominal).any(-1)
        unattributed_bad = ~ok[0] & ~attributed
        if unattributed_bad.any():
            idx = tuple(np.argwhere(unattributed_bad)[0])
            raise AssertionError(
                f"{name} {key}: {int(unattributed_bad.sum())} pixels off with no decision near a threshold "
                f"(max |diff| {np.abs(g - nominal)[unattributed_bad].max():.3e}, atol {atol}, rtol {rtol}); "
                f"first at {idx}: got {g[idx]}, want {nominal[idx]}")
        ok_any = np.logical_or.reduce(ok)
        ambiguous = ~ok_any
        stack = np.stack(vs)
        lo, hi = stack.min(0), stack.max(0)
        pad = atol + rtol * np.maximum(np.abs(lo), np.abs(hi)) + (hi - lo)
        inside = ((g >= lo - pad) & (g <= hi + pad)).all(-1)
        n_pix = max(attributed.size, 1)
        allowed_ambiguous = 0 if max_ambiguous is None else max_ambiguous
        assert int(ambiguous.sum()) <= allowed_ambiguous and inside[ambiguous].all(), (
            f"{name} {key}: {int(ambiguous.sum())} near-threshold pixels match no decision variant "
            f"(allowed {allowed_ambiguous})")
        # every point crosses T = 0.5 somewhere, in steps of ~alpha / 2: the median hinges on its
        # threshold five times as often as the other outputs on theirs
        allowed = max_attributed * (5 if key == "median" else 1)
        assert attributed.sum() <= max(allowed * n_pix, 3), (
            f"{name} {key}: {int(attributed.sum())}/{n_pix} pixels depend on a near-threshold decision")
        report[key] = (int(attributed.sum()), int((~ok[0]).sum()), int(ambiguous.sum()))
    print(f"{name}: per output (pixels on a near-threshold decision, pixels that differ from the nominal "
          f"oracle render, pixels that match no variant): {report}")
    return report
