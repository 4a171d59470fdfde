"""Accuracy metrics.  Test infrastructure only (see ``oracle/__init__.py``).

``calc_diff`` restates src/misc.py:133-174 (1 - 2*sum(xy)/sum(x^2+y^2) in float64).
Pins: closed forms (identical inputs -> 0, y = -x -> 2, y = 0 -> 1, y = c*x -> 1-2c/(1+c^2)).
"""
import numpy as np


def _f64(x):
    if hasattr(x, "detach"):
        x = x.detach().float().cpu().numpy()
    return np.asarray(x, dtype=np.float64)


def calc_diff(x, y):
    x, y = _f64(x), _f64(y)
    den = (x * x + y * y).sum()
    if den == 0:
        return 0.0
    return float(1.0 - 2.0 * (x * y).sum() / den)


def cosine(x, y):
    x, y = _f64(x).ravel(), _f64(y).ravel()
    den = np.sqrt((x * x).sum() * (y * y).sum())
    return 1.0 if den == 0 else float((x * y).sum() / den)


def max_err_over_rms(out, ref):
    """max|out - ref| / rms(ref)"""
    out, ref = _f64(out), _f64(ref)
    rms = np.sqrt(np.mean(ref * ref))
    return float(np.max(np.abs(out - ref)) / (rms if rms > 0 else 1.0))
