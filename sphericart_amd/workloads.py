"""Seeded synthetic point clouds for the five benchmark / parity configurations.

Points are generated on the host in float64 from a counter-based generator
(SplitMix64 over the point index, so any slice of a cloud can be produced on its
own), rounded once to the working precision, and that one array is what both
the GPU path and any CPU checker are fed with. Only integer arithmetic, +, -, *,
/ and square roots are used, all of which IEEE 754 rounds correctly: no
function of the C library or of numpy's vector math is involved, so the clouds
are the same bits on every machine.
"""

from dataclasses import dataclass

import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)


def _splitmix64(x):
    """Vectorised SplitMix64 finaliser on uint64 arrays."""
    with np.errstate(over="ignore"):
        x = (x + np.uint64(0x9E3779B97F4A7C15)) & _MASK
        x = ((x ^ (x >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _MASK
        x = ((x ^ (x >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _MASK
        return x ^ (x >> np.uint64(31))


def uniform(seed, n, stream, first=0):
    """n doubles in (0, 1), stream-th sequence of the seed, starting at index `first`."""
    idx = np.arange(first, first + n, dtype=np.uint64)
    with np.errstate(over="ignore"):
        key = _splitmix64(np.uint64(seed) * np.uint64(0x100000001B3) + np.uint64(stream))
        bits = _splitmix64(idx * np.uint64(0xD1342543DE82EF95) + key)
    return ((bits >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, n, stream, first=0):
    """Deviates of mean 0 and variance 1: the sum of twelve uniform streams minus six
    (Irwin-Hall; bell-shaped within +-6, which is all the point clouds need)."""
    total = uniform(seed, n, 12 * stream, first)
    for j in range(1, 12):
        total = total + uniform(seed, n, 12 * stream + j, first)
    return total - 6.0


def _directions(seed, n, first):
    """Uniform directions after Marsaglia (1972): (a, b) uniform in the unit disk, s = a^2 + b^2,
    direction (2a sqrt(1-s), 2b sqrt(1-s), 1-2s). A point whose pair falls outside the disk takes
    the pair of the next attempt's streams, so every point still depends on its index alone."""
    a = np.zeros(n)
    b = np.zeros(n)
    s = np.full(n, 2.0)
    for attempt in range(64):
        todo = s >= 1.0
        if not todo.any():
            break
        ta = 2.0 * uniform(seed, n, 100 + 2 * attempt, first) - 1.0
        tb = 2.0 * uniform(seed, n, 101 + 2 * attempt, first) - 1.0
        a = np.where(todo, ta, a)
        b = np.where(todo, tb, b)
        s = np.where(todo, ta * ta + tb * tb, s)
    s = np.minimum(s, 1.0)  # (no point gets here unplaced: 0.215^64)
    root = np.sqrt(1.0 - s)
    return np.stack([2.0 * a * root, 2.0 * b * root, 1.0 - 2.0 * s], axis=1)


def _on_axis(xyz, radius, every, first):
    """Every `every`-th point (by global index) exactly on the z axis, sign alternating."""
    idx = np.arange(first, first + xyz.shape[0])
    hit = idx % every == 0
    sign = np.where((idx // every) % 2 == 0, 1.0, -1.0)
    xyz[hit, 0] = 0.0
    xyz[hit, 1] = 0.0
    xyz[hit, 2] = (sign * radius)[hit]
    return xyz


@dataclass(frozen=True)
class Workload:
    name: str
    description: str
    l_max: int
    dtype: str          # "f32" or "f64"
    normalized: bool    # spherical (True) or solid (False) harmonics
    derivatives: str    # "values", "gradients" or "hessians"
    n_samples: int
    seed: int

    @property
    def numpy_dtype(self):
        return np.float32 if self.dtype == "f32" else np.float64

    @property
    def n_components(self):
        return {"values": 1, "gradients": 4, "hessians": 13}[self.derivatives]

    @property
    def bytes_per_point(self):
        """Algorithmic traffic: 3 coordinates read, (l_max+1)^2 (1 + 3 + 9) numbers written."""
        size = 4 if self.dtype == "f32" else 8
        return size * (3 + (self.l_max + 1) ** 2 * self.n_components)

    def points(self, n=None, first=0):
        """`n` points of the cloud starting at global index `first` (default: all of it)."""
        n = self.n_samples if n is None else n
        return _GENERATORS[self.name](self.seed, n, first).astype(self.numpy_dtype)


def _cfg1(seed, n, first):
    return np.stack([normal(seed, n, a, first) for a in range(3)], axis=1)


def _shell(seed, n, first):
    radius = 0.5 + 4.5 * uniform(seed, n, 20, first)
    return _directions(seed, n, first) * radius[:, None], radius


def _cfg2(seed, n, first):
    return _shell(seed, n, first)[0]


def _cfg3(seed, n, first):
    xyz, radius = _shell(seed, n, first)
    return _on_axis(xyz, radius, 100, first)


def _cfg4(seed, n, first):
    return np.stack([-3.0 + 6.0 * uniform(seed, n, a, first) for a in range(3)], axis=1)


def _cfg5(seed, n, first):
    # radii from 1e-2 over thirteen octaves (to 82), the same share of the points in each:
    # 0.01 m 2^e with e uniform in 0 .. 12 and m uniform in [1, 2)
    octave = np.floor(13.0 * uniform(seed, n, 21, first))
    radius = 0.01 * np.ldexp(1.0 + uniform(seed, n, 20, first), octave.astype(np.int64))
    xyz = _directions(seed, n, first) * radius[:, None]
    return _on_axis(xyz, radius, 200, first)


_GENERATORS = {"cfg1": _cfg1, "cfg2": _cfg2, "cfg3": _cfg3, "cfg4": _cfg4, "cfg5": _cfg5, "val10": _cfg2, "val22": _cfg2,
               "val28": _cfg2, "grad10": _cfg3, "hess5": _cfg3}

WORKLOADS = {
    "cfg1": Workload(
        "cfg1", "spherical, l_max=8, f64, values+gradients, 10k points, xyz bell-shaped with variance 1",
        8, "f64", True, "gradients", 10_000, 1001,
    ),
    "cfg2": Workload(
        "cfg2", "spherical, l_max=3, f32, values, 1M points, uniform directions, r ~ U[0.5,5)",
        3, "f32", True, "values", 1_000_000, 1002,
    ),
    "cfg3": Workload(
        "cfg3",
        "spherical, l_max=6, f32, values+gradients, 1M points, uniform directions, r ~ U[0.5,5), "
        "1% of the points exactly on the +-z axis",
        6, "f32", True, "gradients", 1_000_000, 1003,
    ),
    "cfg4": Workload(
        "cfg4", "solid, l_max=16, f64, values+gradients+Hessians, 100k points, xyz ~ U[-3,3)^3",
        16, "f64", False, "hessians", 100_000, 1004,
    ),
    "cfg5": Workload(
        "cfg5",
        "spherical, l_max=32, f32, values+gradients, 200k points, uniform directions, "
        "r spread evenly over the 13 octaves of [1e-2, 82), 0.5% of the points on the +-z axis",
        32, "f32", True, "gradients", 200_000, 1005,
    ),
    # not one of the reference's configurations: values alone beyond the closed forms, the shape
    # the values kernel is profiled on
    "val10": Workload(
        "val10", "spherical, l_max=10, f32, values, 1M points, uniform directions, r ~ U[0.5,5)",
        10, "f32", True, "values", 1_000_000, 1010,
    ),
    # and at an l_max where 64 rows no longer fit in LDS (tiles of 32 points, two channels side by
    # side in a wave)
    "val22": Workload(
        "val22", "spherical, l_max=22, f32, values, 500k points, uniform directions, r ~ U[0.5,5)",
        22, "f32", True, "values", 500_000, 1013,
    ),
    # and where the rows of few points fill LDS (pairs_kernel)
    "val28": Workload(
        "val28", "spherical, l_max=28, f32, values, 350k points, uniform directions, r ~ U[0.5,5)",
        28, "f32", True, "values", 350_000, 1014,
    ),
    # likewise gradients at l_max just above the closed forms
    "grad10": Workload(
        "grad10",
        "spherical, l_max=10, f32, values+gradients, 1M points, uniform directions, r ~ U[0.5,5), "
        "1% of the points exactly on the +-z axis",
        10, "f32", True, "gradients", 1_000_000, 1011,
    ),
    # and second derivatives at small l_max
    "hess5": Workload(
        "hess5",
        "spherical, l_max=5, f32, values+gradients+Hessians, 500k points, uniform directions, r ~ U[0.5,5), "
        "1% of the points exactly on the +-z axis",
        5, "f32", True, "hessians", 500_000, 1012,
    ),
}
