"""The checker's two contractions are dot products: pin them against einsum in extended precision."""

import numpy as np
import pytest


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-14), (np.float32, 2e-6)])
@pytest.mark.parametrize("n_total", [1, 4, 49, 289])
def test_backward_is_the_contraction_over_the_last_axis(oracle, dtype, tol, n_total):
    rng = np.random.default_rng(n_total)
    dsph = rng.standard_normal((13, 3, n_total)).astype(dtype)
    grad = rng.standard_normal((13, n_total)).astype(dtype)
    got = oracle.backward(dsph, grad)
    want = np.einsum("iak,ik->ia", dsph.astype(np.longdouble), grad.astype(np.longdouble))
    scale = np.einsum("iak,ik->ia", np.abs(dsph), np.abs(grad)).astype(np.longdouble) + 1
    assert got.dtype == dtype and got.shape == (13, 3)
    assert np.max(np.abs(got - want) / scale) < tol
    # one component at a time: a transposed operand or a wrong stride would show here
    one = np.zeros_like(grad)
    one[:, n_total // 2] = 1
    np.testing.assert_array_equal(oracle.backward(dsph, one), dsph[:, :, n_total // 2])


@pytest.mark.parametrize("dtype,tol", [(np.float64, 1e-14), (np.float32, 2e-6)])
@pytest.mark.parametrize("n_total", [1, 9, 49])
def test_backward_second_sums_over_the_first_derivative_axis(oracle, dtype, tol, n_total):
    rng = np.random.default_rng(100 + n_total)
    ddsph = rng.standard_normal((11, 3, 3, n_total)).astype(dtype)
    grad = rng.standard_normal((11, 3, n_total)).astype(dtype)
    got = oracle.backward_second(ddsph, grad)
    want = np.einsum("iabk,iak->ib", ddsph.astype(np.longdouble), grad.astype(np.longdouble))
    scale = np.einsum("iabk,iak->ib", np.abs(ddsph), np.abs(grad)).astype(np.longdouble) + 1
    assert np.max(np.abs(got - want) / scale) < tol
    # a non-symmetric ddsph tells the two derivative axes apart
    one = np.zeros_like(grad)
    one[:, 1, 0] = 1
    np.testing.assert_array_equal(oracle.backward_second(ddsph, one), ddsph[:, 1, :, 0])
