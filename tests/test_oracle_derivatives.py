"""The oracle's first and second derivatives against finite differences and identities.

Finite differences follow the reference's own derivative test
(sphericart/tests/test_derivatives.cpp:11-57,112-163: central differences,
delta = 1e-4, relative tolerance 1e-4, l_max = 0..14, both classes).
Identities: Euler's theorem for homogeneous polynomials (r . grad = l for solid,
0 for spherical harmonics), harmonicity (trace of the Hessian of a solid
harmonic vanishes), symmetry of the Hessian, Hessian . r = (l-1) grad.
"""

import numpy as np
import pytest

DELTA = 1e-4
TOL = 1e-4


@pytest.fixture(scope="module")
def xyz():
    # the reference's four fixed points (test_derivatives.cpp:171-177) plus random ones
    pts = [[0.01 * i - 0.3 * a * a for a in range(3)] for i in range(4)]
    rng = np.random.default_rng(5)
    return np.array(pts + list(rng.normal(size=(12, 3))))


def _close(analytic, numeric, scale):
    return np.abs(analytic - numeric) <= TOL * np.maximum(np.abs(numeric), scale)


@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("l_max", [0, 1, 2, 5, 6, 7, 10, 14])
@pytest.mark.parametrize("mode", ["gradients", "hessians"])
def test_gradient_finite_differences(oracle, xyz, normalized, l_max, mode):
    dsph = oracle.compute(xyz, l_max, normalized, mode)[1]
    scale = 1e-6 + np.abs(dsph).max()
    for a in range(3):
        step = np.zeros(3)
        step[a] = DELTA
        plus = oracle.compute(xyz + step, l_max, normalized, mode)[0]
        minus = oracle.compute(xyz - step, l_max, normalized, mode)[0]
        assert _close(dsph[:, a, :], (plus - minus) / (2 * DELTA), 1e-3 * scale).all()


@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("l_max", [0, 1, 2, 3, 6, 9, 14])
def test_hessian_finite_differences(oracle, xyz, normalized, l_max):
    ddsph = oracle.compute(xyz, l_max, normalized, "hessians")[2]
    scale = 1e-6 + np.abs(ddsph).max()
    for a in range(3):
        step = np.zeros(3)
        step[a] = DELTA
        plus = oracle.compute(xyz + step, l_max, normalized, "hessians")[1]
        minus = oracle.compute(xyz - step, l_max, normalized, "hessians")[1]
        numeric = (plus - minus) / (2 * DELTA)  # d/dx_a of grad_b
        assert _close(ddsph[:, a, :, :], numeric, 1e-3 * scale).all()


@pytest.mark.parametrize("mode", ["gradients", "hessians"])
def test_euler_homogeneity(oracle, xyz, mode):
    l_max = 12
    degree = np.concatenate([[l] * (2 * l + 1) for l in range(l_max + 1)])
    sph, dsph = oracle.compute(xyz, l_max, False, mode)[:2]
    radial = np.einsum("ia,iak->ik", xyz, dsph)
    assert np.allclose(radial, degree * sph, rtol=1e-10, atol=1e-10 * np.abs(sph).max())
    dsph = oracle.compute(xyz, l_max, True, mode)[1]
    radial = np.einsum("ia,iak->ik", xyz, dsph)
    assert np.abs(radial).max() < 1e-11 * max(1.0, np.abs(dsph).max())


def test_hessian_identities(oracle, xyz):
    l_max = 12
    degree = np.concatenate([[l] * (2 * l + 1) for l in range(l_max + 1)])
    for normalized in (True, False):
        _, dsph, ddsph = oracle.compute(xyz, l_max, normalized, "hessians")
        assert np.array_equal(ddsph, ddsph.transpose(0, 2, 1, 3))
        if not normalized:
            top = np.abs(ddsph).max()
            trace = ddsph[:, 0, 0] + ddsph[:, 1, 1] + ddsph[:, 2, 2]
            assert np.abs(trace).max() < 1e-11 * top
            along = np.einsum("ib,iabk->iak", xyz, ddsph)
            assert np.allclose(along, (degree - 1) * dsph, rtol=1e-9, atol=1e-11 * top)
