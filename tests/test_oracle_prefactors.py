"""The oracle's prefactor table against closed forms (no formula of the oracle is retyped here).

F_l^m = (-1)^m sqrt((2l+1)/(2 pi) (l-m)!/(l+m)!), with an extra 1/sqrt(2) for m = 0;
Q_l^l = (-1)^l (2l-1)!!; recursion constant -1/((l+m+1)(l-m)) for m < l.
Reference: sphericart/include/templates.hpp:54-97, docs/src/maths.rst:36-65.
"""

from fractions import Fraction
from math import factorial, pi, sqrt

import numpy as np
import pytest

L = 24


def _double_factorial(n):
    out = 1
    while n > 1:
        out *= n
        n -= 2
    return out


def test_layout_and_closed_forms_f64(oracle):
    table = oracle.prefactors(L, np.float64)
    nq = (L + 1) * (L + 2) // 2
    assert table.shape == (2 * nq,)
    F, Q = table[:nq], table[nq:]
    for l in range(L + 1):
        for m in range(l + 1):
            k = l * (l + 1) // 2 + m
            ratio = Fraction(factorial(l - m), factorial(l + m))
            want = (-1) ** m * sqrt((2 * l + 1) / (2 * pi) * float(ratio))
            if m == 0:
                want /= sqrt(2.0)
            assert F[k] == pytest.approx(want, rel=1e-13), (l, m)
            if m == l:
                assert Q[k] == pytest.approx((-1) ** l * _double_factorial(2 * l - 1), rel=1e-13)
            else:
                assert Q[k] == -1.0 / ((l + m + 1) * (l - m))


def test_table_is_independent_of_l_max(oracle):
    """Entries depend on (l, m) only: a smaller table is a prefix of each block of a larger one."""
    for dtype in (np.float32, np.float64):
        big = oracle.prefactors(L, dtype)
        nbig = (L + 1) * (L + 2) // 2
        for small_l in (0, 1, 5, 11):
            small = oracle.prefactors(small_l, dtype)
            n = (small_l + 1) * (small_l + 2) // 2
            assert np.array_equal(small[:n], big[:n])
            assert np.array_equal(small[n:], big[nbig : nbig + n])


def test_f32_table_rounds_like_float(oracle):
    """The float table is computed in float: close to the double one, and Q_l^l overflows at l = 29."""
    f32 = oracle.prefactors(32, np.float32)
    f64 = oracle.prefactors(32, np.float64)
    nq = 33 * 34 // 2
    finite = np.isfinite(f32) & (np.abs(f64) > 1e-30) & (np.abs(f64) < 1e30)
    assert np.allclose(f32[finite], f64[finite], rtol=2e-5)
    for l in range(33):
        qll = f32[nq + l * (l + 1) // 2 + l]
        assert np.isfinite(qll) == (l < 29), l


def test_library_table_matches_oracle(oracle, library):
    """The table the kernels use (include/sphx_launch.h: sphx_prefactors_*) is the oracle's, bit for bit."""
    for dtype, fn in ((np.float32, library.sphx_prefactors_f32), (np.float64, library.sphx_prefactors_f64)):
        for l_max in (0, 1, 6, 17, 32, 64):
            out = np.empty((l_max + 1) * (l_max + 2), dtype=dtype)
            assert fn(l_max, out.ctypes.data) == 0
            want = oracle.prefactors(l_max, dtype)
            assert ((out == want) | (np.isnan(out) & np.isnan(want))).all(), (dtype, l_max)
    out = np.empty(8, dtype=np.float64)
    assert library.sphx_prefactors_f64(65, out.ctypes.data) == 2  # SPHX_ERR_UNSUPPORTED
    assert library.sphx_prefactors_f64(-1, out.ctypes.data) == 1  # SPHX_ERR_ARGUMENT
