"""Shared pieces of the parity tests."""

import numpy as np

MODES = ("values", "gradients", "hessians")

# Tolerances of the reference's own device-vs-host test
# (python/tests/test_cupy.py:22-49): rtol = atol = 1e-5 in float32, 1e-12 in float64.
TOLERANCE = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}


def same_numbers(a, b):
    a = np.asarray(a)
    b = np.asarray(b)
    return (a == b) | (np.isnan(a) & np.isnan(b))


def within_tolerance(got, want):
    """|got - want| <= tol * max(1, |want|) where `want` is finite; both non-finite elsewhere."""
    got = np.asarray(got)
    want = np.asarray(want)
    tol = TOLERANCE[want.dtype]
    finite = np.isfinite(want)
    ok = np.empty(want.shape, dtype=bool)
    ok[finite] = np.abs(got[finite] - want[finite]) <= tol * np.maximum(1.0, np.abs(want[finite]))
    ok[~finite] = ~np.isfinite(got[~finite])
    return ok


def special_points(dtype, rng, n):
    """Random points with the awkward ones in front: the +-z axis, the other axes, a tiny and a large radius."""
    xyz = rng.normal(size=(n, 3))
    fixed = np.array(
        [
            [0.0, 0.0, 1.5],
            [0.0, 0.0, -0.7],
            [1.0, 0.0, 0.0],
            [0.0, 2.0, 0.0],
            [-3.0, 0.0, 0.0],
            [1e-3, -2e-3, 5e-4],
            [30.0, -40.0, 25.0],
        ]
    )
    k = min(n, len(fixed))
    xyz[:k] = fixed[:k]
    return xyz.astype(dtype)
