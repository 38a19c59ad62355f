"""The oracle's values against independent mathematics.

* scipy.special.sph_harm_y combined into real harmonics exactly as the
  reference's own truth test does (python/tests/test_vs_scipy.py:12-61);
* the Unsold sum rule sum_m Y_lm^2 = (2l+1)/(4 pi);
* the +-z axis, where only m = 0 survives: Y_l0 = sqrt((2l+1)/(4 pi)) (+-1)^l;
* the constants the reference documents for l = 0, 1 (macros.hpp:51,76-79);
* closed-form polynomials of l = 2 (docs/src/maths.rst, julia/test/test_solidharmonics.jl:18-48).
"""

from math import pi, sqrt

import numpy as np
import pytest
import scipy.special

L_MAX = 20


def scipy_real_sph(xyz, l, m):
    x, y, z = xyz[:, 0], xyz[:, 1], xyz[:, 2]
    r = np.sqrt(x**2 + y**2 + z**2)
    theta = np.arccos(z / r)
    phi = np.arctan2(y, x)
    plus = scipy.special.sph_harm_y(l, m, theta, phi)
    minus = scipy.special.sph_harm_y(l, -m, theta, phi)
    if m > 0:
        return ((minus + (-1) ** m * plus) / np.sqrt(2.0)).real
    if m < 0:
        return ((-plus + (-1) ** m * minus) / np.sqrt(2.0)).imag
    return plus.real


@pytest.fixture(scope="module")
def xyz():
    rng = np.random.default_rng(0)
    return rng.random((100, 3)) * 2.0 - 0.7


@pytest.mark.parametrize("mode", ["values", "gradients", "hessians"])
def test_against_scipy(oracle, xyz, mode):
    """Every (l, m) up to 20, spherical and solid; also the values that come with derivatives,
    which take the recursion route from l = 2 (with Hessians) instead of the closed forms."""
    r = np.linalg.norm(xyz, axis=1)
    sph = oracle.compute(xyz, L_MAX, True, mode)[0]
    solid = oracle.compute(xyz, L_MAX, False, mode)[0]
    for l in range(L_MAX + 1):
        for m in range(-l, l + 1):
            want = scipy_real_sph(xyz, l, m)
            k = l * l + l + m
            assert np.allclose(sph[:, k], want, rtol=1e-9, atol=1e-11), (l, m)
            assert np.allclose(solid[:, k] / r**l, want, rtol=1e-9, atol=1e-11), (l, m)


def test_against_scipy_small_l_max(oracle, xyz):
    """l_max <= 6 takes the all-closed-form route; check each of them separately."""
    for l_max in range(7):
        sph = oracle.compute(xyz, l_max, True, "values")[0]
        for l in range(l_max + 1):
            for m in range(-l, l + 1):
                assert np.allclose(sph[:, l * l + l + m], scipy_real_sph(xyz, l, m), rtol=1e-10, atol=1e-12)


def test_float32_follows_float64(oracle, xyz):
    got = oracle.compute(xyz.astype(np.float32), 10, True, "values")[0]
    want = oracle.compute(xyz.astype(np.float32).astype(np.float64), 10, True, "values")[0]
    assert np.allclose(got, want, rtol=0, atol=2e-5)


def test_unsold_sum_rule(oracle, xyz):
    r = np.linalg.norm(xyz, axis=1)
    sph = oracle.compute(xyz, L_MAX, True, "values")[0]
    solid = oracle.compute(xyz, L_MAX, False, "values")[0]
    for l in range(L_MAX + 1):
        block = slice(l * l, (l + 1) ** 2)
        assert np.allclose((sph[:, block] ** 2).sum(axis=1), (2 * l + 1) / (4 * pi), rtol=1e-11)
        assert np.allclose((solid[:, block] ** 2).sum(axis=1), (2 * l + 1) / (4 * pi) * r ** (2 * l), rtol=1e-11)


def test_z_axis(oracle):
    xyz = np.array([[0.0, 0.0, 2.5], [0.0, 0.0, -0.3]])
    for mode in ("values", "gradients", "hessians"):
        sph = oracle.compute(xyz, 12, True, mode)[0]
        for l in range(13):
            for m in range(-l, l + 1):
                k = l * l + l + m
                if m == 0:
                    want = sqrt((2 * l + 1) / (4 * pi)) * np.array([1.0, (-1.0) ** l])
                    assert np.allclose(sph[:, k], want, rtol=1e-13)
                else:
                    assert (sph[:, k] == 0).all()


def test_documented_constants(oracle):
    xyz = np.array([[0.3, -1.1, 0.7]])
    solid = oracle.compute(xyz, 2, False, "values")[0][0]
    x, y, z = xyz[0]
    assert solid[0] == pytest.approx(0.282094791773878, rel=1e-14)
    assert np.allclose(solid[1:4], 0.48860251190292 * np.array([y, z, x]), rtol=1e-14)
    c = sqrt(15 / (4 * pi))
    want = [c * x * y, c * y * z, sqrt(5 / (16 * pi)) * (2 * z * z - x * x - y * y), c * x * z, c / 2 * (x * x - y * y)]
    assert np.allclose(solid[4:9], want, rtol=1e-13)
