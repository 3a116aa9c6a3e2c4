"""Helpers shared by the parity tests."""
import numpy as np

FP32_TOL = 1e-5   # relative Frobenius error allowed for float32 results
FP16_TOL = 2e-3   # ... and for float16 results (fp16 storage, fp32 accumulate)


def rng(seed):
    return np.random.default_rng(seed)


def ints(r, shape, hi=50):
    """rand() % hi as floats, the reference tests' input recipe (test/TestUtils.h:22-26)."""
    return r.integers(0, hi, size=shape).astype(np.float32)


def uni(r, shape):
    return r.uniform(-1.0, 1.0, size=shape).astype(np.float32)


def nrm(r, shape, sigma=1.0):
    return (r.standard_normal(size=shape) * sigma).astype(np.float32)


def rel_fro(got, want):
    g = np.asarray(got, np.float64).ravel()
    w = np.asarray(want, np.float64).ravel()
    d = np.linalg.norm(w)
    return float(np.linalg.norm(g - w) / d) if d else float(np.linalg.norm(g))


def h(a):
    """round to fp16 storage"""
    return np.asarray(a, np.float32).astype(np.float16)


def f(a):
    return np.asarray(a).astype(np.float32)
