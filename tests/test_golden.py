"""The oracle reproduces the golden vectors (outputs of the compiled reference) bit for bit."""

import pytest

from golden_io import CONFIGS, config_case, degenerate_cases, edge_cases
from helpers import same_numbers


@pytest.mark.parametrize("name", CONFIGS)
def test_oracle_on_benchmark_configurations(oracle, name):
    xyz, l_max, normalized, mode, want = config_case(name)
    got = oracle.compute(xyz, l_max, normalized, mode)
    for g, w in zip(got, want):
        assert (g is None) == (w is None)
        if w is not None:
            assert g.shape == w.shape and g.dtype == w.dtype
            assert same_numbers(g, w).all()


@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_oracle_on_edge_cases(oracle, tag):
    count = 0
    for xyz, l_max, normalized, mode, want in edge_cases(tag):
        got = oracle.compute(xyz, l_max, normalized, mode)
        for g, w in zip(got, want):
            assert (g is None) == (w is None)
            if w is not None:
                assert same_numbers(g, w).all(), (l_max, normalized, mode)
        count += 1
    assert count == 36


@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_oracle_on_degenerate_points(oracle, tag):
    """The origin, NaN, infinite, denormal and overflowing coordinates: the restatement returns
    what the compiled reference returns, NaN for NaN, signed infinity for signed infinity, and the
    fixture does hold such numbers (the reference has no guard, templates.hpp:392-400)."""
    import numpy as np

    count = 0
    for xyz, where, l_max, normalized, mode, want in degenerate_cases(tag):
        with np.errstate(all="ignore"):
            got = oracle.compute(xyz, l_max, normalized, mode)
        for g, w in zip(got, want):
            assert (g is None) == (w is None)
            if w is not None:
                assert same_numbers(g, w).all(), (l_max, normalized, mode)
        ordinary = np.setdiff1d(np.arange(xyz.shape[0]), where)
        assert np.isfinite(want[0][ordinary]).all()
        if normalized:
            assert np.isnan(want[0][where[0], 1:]).all()  # the origin: 0 * inf
        count += 1
    assert count == 24


def test_cfg5_golden_holds_the_float_overflow(oracle):
    """In float the reference returns non-finite numbers for every l >= 29 (prefactor overflow);
    the fixture keeps that behaviour on record."""
    import numpy as np

    _, l_max, _, _, want = config_case("cfg5")
    sph = want[0]
    assert l_max == 32
    assert not np.isfinite(sph[:, 29 * 29 :]).any()
    assert np.isfinite(sph[:, : 20 * 20]).all()
