"""Shared helpers for the parity tests: seeded inputs (numpy PCG64) and error metrics."""
import numpy as np


def normal(seed, shape, scale=1.0):
    """f32 ~ N(0, scale^2) from numpy's PCG64 — the synthetic-input recipe used by tests and bench."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return (rng.standard_normal(shape, dtype=np.float32) * np.float32(scale)).astype(np.float32)


def rel_l2(got, want):
    got = np.asarray(got, dtype=np.float64).reshape(-1)
    want = np.asarray(want, dtype=np.float64).reshape(-1)
    den = np.linalg.norm(want)
    return float(np.linalg.norm(got - want) / (den if den > 0 else 1.0))


def bits_equal_or_both_nan(a, b):
    """Bitwise equality of two f32 / f16 arrays, treating any-NaN == any-NaN."""
    a = np.asarray(a)
    b = np.asarray(b)
    assert a.dtype == b.dtype and a.shape == b.shape
    u = {2: np.uint16, 4: np.uint32}[a.dtype.itemsize]
    same = a.view(u) == b.view(u)
    both_nan = np.isnan(a) & np.isnan(b)
    return bool(np.all(same | both_nan))
