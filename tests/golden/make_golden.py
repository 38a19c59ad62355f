"""Write the golden vectors of tests/golden/*.npz.

Run in the development container, where the reference checkout is mounted:

    make -C oracle ref && python tests/golden/make_golden.py

Every expected output comes from the reference's own CPU implementation
(sphericart/src/sphericart.cpp and the headers it includes), compiled from where
it lies into oracle/_ref/libsphx_ref.so without FMA contraction -- not from this
repository's restatement. Inputs are the first points of the five benchmark
clouds (sphericart_amd/workloads.py) plus a small grid of edge cases and a set of
degenerate points (the origin, NaN, infinities, denormal and overflowing
coordinates); they are stored next to the outputs, so the files stand on their
own. `python tests/golden/make_golden.py degenerate` writes only the named group
(configs, edge, degenerate).
"""

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import oracle  # noqa: E402
from sphericart_amd.workloads import WORKLOADS  # noqa: E402

POINTS = {"cfg1": 64, "cfg2": 64, "cfg3": 200, "cfg4": 12, "cfg5": 400}
EDGE_L_MAX = (0, 1, 2, 6, 7, 11)
DEGENERATE_L_MAX = (1, 6, 7, 11)
TAKE = {"cfg5": slice(None, None, 25)}  # keep the file small but include the on-axis points 0, 200


def save(name, xyz, l_max, normalized, mode):
    sph, dsph, ddsph = oracle.compute(xyz, l_max, normalized, mode, flavour="ref")
    arrays = {
        "xyz": xyz,
        "l_max": np.int64(l_max),
        "normalized": np.bool_(normalized),
        "mode": np.str_(mode),
        "sph": sph,
    }
    if dsph is not None:
        arrays["dsph"] = dsph
    if ddsph is not None:
        arrays["ddsph"] = ddsph
    path = os.path.join(HERE, f"{name}.npz")
    np.savez_compressed(path, **arrays)
    print(f"{path}: {os.path.getsize(path) / 1024:.0f} KiB")


def degenerate_points(dtype):
    """70 points: inputs for which the reference returns infinities and NaN (it divides by
    sqrt(x^2 + y^2 + z^2) without a guard, sphericart/include/templates.hpp:392-400), each between
    ordinary points, so that a tile of 64 holds both kinds."""
    tiny, big = (1e-40, 1e20) if dtype == np.float32 else (1e-310, 1e160)
    nan, inf = float("nan"), float("inf")
    bad = [
        (0.0, 0.0, 0.0), (-0.0, 0.0, -0.0),
        (nan, 0.3, -0.2), (0.5, nan, 0.1), (0.1, 0.2, nan), (nan, nan, nan),
        (inf, 1.0, 2.0), (1.0, -inf, 2.0), (1.0, 2.0, inf), (-inf, inf, 0.0),
        (tiny, tiny, tiny), (tiny, 0.0, 0.0), (0.0, -tiny, 2 * tiny), (0.0, 0.0, tiny), (1.0, tiny, -tiny),
        (big, big, big), (big, 0.5, -0.25), (0.0, 0.0, big), (-big, 0.0, big), (0.0, 0.0, -big),
    ]
    rng = np.random.default_rng(4242)
    xyz = rng.normal(size=(70, 3))
    # bad points at 1, 4, 7, ... and, so that a tile boundary of every kernel sees one, at 63, 64
    where = [1 + 3 * i for i in range(len(bad) - 2)] + [63, 64]
    for at, point in zip(where, bad):
        xyz[at] = point
    with np.errstate(over="ignore", under="ignore"):
        return xyz.astype(dtype), np.array(where)


def write_degenerate():
    for dtype, tag in ((np.float32, "f32"), (np.float64, "f64")):
        xyz, where = degenerate_points(dtype)
        arrays = {"xyz": xyz, "degenerate_at": where}
        for l_max in DEGENERATE_L_MAX:
            for normalized in (True, False):
                for mode in ("values", "gradients", "hessians"):
                    kind = "spherical" if normalized else "solid"
                    with np.errstate(all="ignore"):
                        out = oracle.compute(xyz, l_max, normalized, mode, flavour="ref")
                    for label, array in zip(("sph", "dsph", "ddsph"), out):
                        if array is not None:
                            arrays[f"{kind}_l{l_max}_{mode}_{label}"] = array
        path = os.path.join(HERE, f"degenerate_{tag}.npz")
        np.savez_compressed(path, **arrays)
        print(f"{path}: {os.path.getsize(path) / 1024:.0f} KiB")


def main():
    if not oracle.available("ref"):
        raise SystemExit("oracle/_ref/libsphx_ref.so is missing: run `make -C oracle ref` first")
    groups = set(sys.argv[1:]) or {"configs", "edge", "degenerate"}
    if "degenerate" in groups:
        write_degenerate()
    if "configs" in groups:
        write_configs()
    if "edge" in groups:
        write_edge()


def write_configs():
    for name, w in WORKLOADS.items():
        if name not in POINTS:
            continue
        xyz = w.points(POINTS[name])[TAKE.get(name, slice(None))]
        save(name, xyz, w.l_max, w.normalized, w.derivatives)


def write_edge():
    # edge cases: both classes, all three call types, both precisions, l_max on either side of
    # the closed-form limits (1 with Hessians, 6 without)
    rng = np.random.default_rng(2024)
    pts = rng.normal(size=(24, 3))
    pts[0] = (0.0, 0.0, 1.5)
    pts[1] = (0.0, 0.0, -0.7)
    pts[2] = (1.0, 0.0, 0.0)
    pts[3] = (0.0, 2.0, 0.0)
    pts[4] = (1e-3, -2e-3, 5e-4)
    pts[5] = (30.0, -40.0, 25.0)
    for dtype, tag in ((np.float32, "f32"), (np.float64, "f64")):
        xyz = pts.astype(dtype)
        arrays = {"xyz": xyz}
        for l_max in EDGE_L_MAX:
            for normalized in (True, False):
                for mode in ("values", "gradients", "hessians"):
                    kind = "spherical" if normalized else "solid"
                    out = oracle.compute(xyz, l_max, normalized, mode, flavour="ref")
                    for label, array in zip(("sph", "dsph", "ddsph"), out):
                        if array is not None:
                            arrays[f"{kind}_l{l_max}_{mode}_{label}"] = array
        path = os.path.join(HERE, f"edge_{tag}.npz")
        np.savez_compressed(path, **arrays)
        print(f"{path}: {os.path.getsize(path) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
