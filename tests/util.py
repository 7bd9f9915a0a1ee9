"""Helpers shared by the tests: deterministic inputs in both storage types and the comparison metrics the tolerances refer to."""
import numpy as np

import oracle as O


def init_for_test(shape, shift, scale=1.0):
    """The reference tests' deterministic fill sin(i / 10 + shift) * scale (src/utils/testing_util.cpp:46-55)."""
    n = int(np.prod(shape))
    i = np.arange(n, dtype=np.float32)
    return (np.sin(i / np.float32(10.0) + np.float32(shift)) * np.float32(scale)).astype(np.float32).reshape(shape)


def storage(a, dtype):
    """fp32 values -> the storage type under test ("float32" array or "float16" bit patterns, truncating like the reference)."""
    a = np.ascontiguousarray(a, np.float32)
    return O.to_half(a) if dtype == "float16" else a


def random_tensor(rng, shape, dtype, scale=1.0):
    return storage(rng.standard_normal(shape) * scale, dtype)


def values(a):
    return O.as_float(np.asarray(a)).astype(np.float64)


def max_abs_rel(got, want):
    """max |got - want| / max |want| — the "relative error (max-abs)" of the tolerance statements."""
    g, w = values(got), values(want)
    if g.size == 0:
        return 0.0
    return float(np.abs(g - w).max() / max(1e-30, np.abs(w).max()))


def mean_abs_diff(got, want):
    """testing::diffForTest of the reference (src/utils/testing_util.cpp:330-366): mean absolute difference."""
    g, w = values(got), values(want)
    return float(np.abs(g - w).mean()) if g.size else 0.0


def mismatches(got, want):
    return int((np.asarray(got) != np.asarray(want)).sum())


TOL = {"float32": 1e-4, "float16": 1e-2}
