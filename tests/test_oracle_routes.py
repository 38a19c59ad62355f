"""Route consistency of the oracle, and the oracle against the compiled reference.

* closed forms up to l = 6 versus the recursion from l = 2
  (the reference's sphericart/tests/test_hardcoding.cpp:14,93-169, tolerance 1e-6);
* one point at a time versus many points (sphericart/tests/test_samples.cpp:18-122);
* bit-for-bit identity with the reference's own sphericart.cpp compiled with the
  same flags (oracle/_ref), when that library has been built.
"""

import numpy as np
import pytest

from helpers import MODES, same_numbers, special_points


@pytest.mark.parametrize("normalized", [True, False])
def test_closed_form_versus_recursion(oracle, normalized):
    rng = np.random.default_rng(3)
    xyz = rng.random((100, 3)) * 2 - 1
    for l_max in (2, 4, 6, 9):
        a = oracle.compute(xyz, l_max, normalized, "gradients")
        b = oracle.recursion_route(xyz, l_max, normalized, "gradients")
        for u, v in zip(a[:2], b):
            scale = np.abs(u).max()
            assert np.abs(u - v).max() < 1e-6 * scale


def test_hessian_route_returns_recursion_values(oracle):
    """With Hessians the values and gradients of l >= 2 come from the recursion
    (sphericart/src/sphericart.cpp:83-92), so they equal the recursion route exactly."""
    rng = np.random.default_rng(4)
    xyz = rng.normal(size=(50, 3))
    for normalized in (True, False):
        hess = oracle.compute(xyz, 8, normalized, "hessians")
        route = oracle.recursion_route(xyz, 8, normalized, "gradients")
        assert same_numbers(hess[0], route[0]).all()
        assert same_numbers(hess[1], route[1]).all()


def test_one_point_versus_many(oracle):
    xyz = np.array([[1.0, 2.0, 3.0]])
    many = np.repeat(xyz, 9, axis=0)
    for l_max in range(11):
        for mode in MODES:
            single = oracle.compute(xyz, l_max, True, mode)
            batch = oracle.compute(many, l_max, True, mode)
            for u, v in zip(single, batch):
                if u is not None:
                    assert same_numbers(np.broadcast_to(u, v.shape), v).all()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_bit_identical_to_compiled_reference(oracle, dtype):
    if not oracle.available("ref"):
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    rng = np.random.default_rng(11)
    for l_max in list(range(0, 13)) + [16, 20, 32]:
        assert same_numbers(oracle.prefactors(l_max, dtype), oracle.prefactors(l_max, dtype, "ref")).all()
        xyz = special_points(dtype, rng, 129)
        for normalized in (True, False):
            for mode in MODES:
                ours = oracle.compute(xyz, l_max, normalized, mode)
                theirs = oracle.compute(xyz, l_max, normalized, mode, "ref")
                for u, v in zip(ours, theirs):
                    if u is not None:
                        assert same_numbers(u, v).all(), (l_max, normalized, mode)
            if l_max >= 2:
                ours = oracle.recursion_route(xyz, l_max, normalized, "gradients")
                theirs = oracle.recursion_route(xyz, l_max, normalized, "gradients", "ref")
                for u, v in zip(ours, theirs):
                    assert same_numbers(u, v).all()


def test_fma_build_of_reference_stays_within_tolerance(oracle):
    """How far two builds of the same reference source drift apart (contraction on/off):
    the yardstick for the float32 tolerance. Informational bound, generous on purpose."""
    if not oracle.available("ref_fma"):
        pytest.skip("oracle/_ref not built (reference checkout absent)")
    rng = np.random.default_rng(12)
    xyz = rng.normal(size=(2000, 3)).astype(np.float32)
    strict = oracle.compute(xyz, 6, True, "gradients")
    fused = oracle.compute(xyz, 6, True, "gradients", "ref_fma")
    for u, v in zip(strict[:2], fused[:2]):
        assert np.abs(u - v).max() < 1e-4
