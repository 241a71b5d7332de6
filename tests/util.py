"""Shared helpers for the parity tests.

Parity bar for floating-point tensors (stated once, used everywhere):
  rel_l2(a, b)  = ||a - b||_2 / ||b||_2                      <= 1e-3
  max_rel(a, b) = max_i |a_i - b_i| / max(|b_i|, rms(b))     <= 2e-2
The floor rms(b) in max_rel keeps elements that are (nearly) zero in the
reference from dividing by zero; integer / index results must be bit-exact.
"""
import numpy as np

REL_L2_TOL = 1e-3
MAX_REL_TOL = 2e-2


def f64(a):
    return np.asarray(a, dtype=np.float64)


def rel_l2(a, b):
    a, b = f64(a), f64(b)
    den = np.linalg.norm(b.ravel())
    num = np.linalg.norm((a - b).ravel())
    return num / den if den > 0 else num


def max_rel(a, b):
    a, b = f64(a), f64(b)
    rms = np.sqrt(np.mean(b * b)) if b.size else 0.0
    den = np.maximum(np.abs(b), rms if rms > 0 else 1.0)
    return float(np.max(np.abs(a - b) / den)) if b.size else 0.0


def assert_parity(a, b, name="", l2=REL_L2_TOL, mx=MAX_REL_TOL):
    assert a.shape == b.shape, (name, a.shape, b.shape)
    assert np.all(np.isfinite(f64(a))), name + ": non-finite values"
    e2, em = rel_l2(a, b), max_rel(a, b)
    assert e2 <= l2, "%s: rel_l2 %.3e > %.1e" % (name, e2, l2)
    assert em <= mx, "%s: max_rel %.3e > %.1e" % (name, em, mx)
    return e2, em


def rng(seed):
    return np.random.default_rng(seed)


def randn16(r, shape, std=1.0):
    return (r.standard_normal(shape) * std).astype(np.float16)
