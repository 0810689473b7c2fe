"""Helpers shared by the GPU parity tests."""
import numpy as np
import torch

DEV = torch.device("cuda:0")


def to_np(t):
    return None if t is None else t.detach().cpu().numpy()


def to_dev(a, dtype=None):
    if a is None:
        return None
    t = torch.as_tensor(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.to(DEV)


def assert_close(actual, expected, atol, rtol=0.0, frac=1.0, name=""):
    """|a - e| <= atol + rtol |e| on at least `frac` of the elements."""
    a = np.asarray(actual, dtype=np.float64)
    e = np.asarray(expected, dtype=np.float64)
    assert a.shape == e.shape, (name, a.shape, e.shape)
    bad = ~(np.abs(a - e) <= atol + rtol * np.abs(e))
    if a.size == 0:
        return
    ok_frac = 1.0 - bad.mean()
    if ok_frac < frac:
        idx = np.argwhere(bad)[:5]
        worst = np.abs(a - e)[bad].max()
        raise AssertionError(
            f"{name}: {bad.sum()}/{a.size} elements off (max |diff| {worst:.3e}, atol {atol}, "
            f"rtol {rtol}); first at {idx.tolist()}: got {a[tuple(idx[0])]}, want {e[tuple(idx[0])]}")
