"""The seeded point clouds: reproducible, sliceable, with the stated distributions."""

import hashlib

import numpy as np

from sphericart_amd.workloads import WORKLOADS, uniform


def test_generator_is_counter_based():
    a = uniform(7, 1000, 3)
    b = uniform(7, 400, 3, first=600)
    assert np.array_equal(a[600:], b)
    assert 0.0 < a.min() and a.max() < 1.0
    assert abs(a.mean() - 0.5) < 0.05


def test_slices_match_the_whole_cloud():
    for w in WORKLOADS.values():
        whole = w.points(3000)
        part = w.points(500, first=1700)
        assert whole.dtype == w.numpy_dtype and whole.shape == (3000, 3)
        assert np.array_equal(whole[1700:2200], part)


def test_distributions():
    p = WORKLOADS["cfg1"].points(20000)
    assert abs(p.mean()) < 0.03 and abs(p.std() - 1.0) < 0.03
    for name in ("cfg2", "cfg3"):
        r = np.linalg.norm(WORKLOADS[name].points(20000).astype(np.float64), axis=1)
        assert 0.5 - 1e-6 <= r.min() and r.max() <= 5.0 + 1e-6
    p = WORKLOADS["cfg3"].points(20000)
    on_axis = (p[:, 0] == 0) & (p[:, 1] == 0)
    assert on_axis.sum() == 200 and on_axis[::100].all()
    assert (p[0, 2] > 0) and (p[100, 2] < 0)
    p = WORKLOADS["cfg4"].points(20000)
    assert -3.0 <= p.min() and p.max() < 3.0
    p = WORKLOADS["cfg5"].points(20000).astype(np.float64)
    r = np.linalg.norm(p, axis=1)
    assert 0.99e-2 <= r.min() and r.max() <= 1.01e2
    assert ((p[:, 0] == 0) & (p[:, 1] == 0)).sum() == 100


def test_clouds_are_the_same_bits_everywhere():
    """The generator uses integer arithmetic, + - * /, ldexp and square roots only, all rounded
    correctly by IEEE 754: a slice of every cloud is pinned by its checksum."""
    want = {"cfg1": "3b8c626daaf7febe", "cfg2": "bc48309760e002a1", "cfg3": "b38668c24141b55b",
            "cfg4": "826d5a035d63f6ad", "cfg5": "aedd94e7b4e94cc1"}
    for name, digest in want.items():
        w = WORKLOADS[name]
        xyz = w.points(1000, first=12345 if w.n_samples > 20000 else 0)
        assert hashlib.sha256(xyz.tobytes()).hexdigest()[:16] == digest, name


def test_bytes_per_point():
    want = {"cfg1": 2616, "cfg2": 76, "cfg3": 796, "cfg4": 30080, "cfg5": 17436, "val10": 496, "val22": 2128, "val28": 3376, "grad10": 1948, "hess5": 1884}
    for name, w in WORKLOADS.items():
        assert w.bytes_per_point == want[name]
