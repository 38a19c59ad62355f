"""Readers for the golden vectors of tests/golden (written by tests/golden/make_golden.py
from the compiled reference)."""

import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
CONFIGS = ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5")
EDGE_L_MAX = (0, 1, 2, 6, 7, 11)


def config_case(name):
    """(xyz, l_max, normalized, mode, (sph, dsph, ddsph)) of one benchmark configuration."""
    with np.load(os.path.join(GOLDEN, f"{name}.npz"), allow_pickle=False) as f:
        want = tuple(f[k] if k in f.files else None for k in ("sph", "dsph", "ddsph"))
        return f["xyz"], int(f["l_max"]), bool(f["normalized"]), str(f["mode"]), want


def edge_cases(tag):
    """Yield (xyz, l_max, normalized, mode, (sph, dsph, ddsph)) for every stored edge case of a precision."""
    with np.load(os.path.join(GOLDEN, f"edge_{tag}.npz"), allow_pickle=False) as f:
        xyz = f["xyz"]
        for l_max in EDGE_L_MAX:
            for normalized in (True, False):
                kind = "spherical" if normalized else "solid"
                for mode in ("values", "gradients", "hessians"):
                    want = tuple(
                        f[key] if (key := f"{kind}_l{l_max}_{mode}_{label}") in f.files else None
                        for label in ("sph", "dsph", "ddsph")
                    )
                    yield xyz, l_max, normalized, mode, want


DEGENERATE_L_MAX = (1, 6, 7, 11)


def degenerate_cases(tag):
    """Yield (xyz, degenerate_at, l_max, normalized, mode, (sph, dsph, ddsph)): points for which the
    reference returns infinities and NaN, between ordinary ones."""
    with np.load(os.path.join(GOLDEN, f"degenerate_{tag}.npz"), allow_pickle=False) as f:
        xyz, where = f["xyz"], f["degenerate_at"]
        for l_max in DEGENERATE_L_MAX:
            for normalized in (True, False):
                kind = "spherical" if normalized else "solid"
                for mode in ("values", "gradients", "hessians"):
                    want = tuple(
                        f[key] if (key := f"{kind}_l{l_max}_{mode}_{label}") in f.files else None
                        for label in ("sph", "dsph", "ddsph")
                    )
                    yield xyz, where, l_max, normalized, mode, want
