"""A C++ program that uses the device classes the way the reference's examples/cuda/example.cu does
(examples/device_example.cpp, built beforehand by sphericart_amd/build.py) against the CPU checker."""

import os
import subprocess

import numpy as np
import pytest

from gpu_utils import announce
from helpers import same_numbers, special_points

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXAMPLE = os.path.join(ROOT, "sphericart_amd", "device_example")


@pytest.mark.gpu
@pytest.mark.parametrize("tag,dtype", [("f32", np.float32), ("f64", np.float64)])
@pytest.mark.parametrize("kind", ["spherical", "solid"])
@pytest.mark.parametrize("l_max", [1, 6, 10])
def test_cxx_classes_from_a_separate_program(oracle, tmp_path, tag, dtype, kind, l_max):
    announce("C++ example", tag, kind, l_max)
    assert os.path.exists(EXAMPLE), "build the example with `python -m sphericart_amd.build`"
    n, ny = 777, (l_max + 1) ** 2
    xyz = special_points(dtype, np.random.default_rng(l_max), n)
    xyz.tofile(tmp_path / "xyz.bin")
    done = subprocess.run(
        [EXAMPLE, tag, kind, str(l_max), str(n), str(tmp_path / "xyz.bin"), str(tmp_path / "out.bin")],
        capture_output=True, text=True, timeout=100,
    )
    assert done.returncode == 0, done.stderr
    assert "device_example: ok" in done.stdout
    out = np.fromfile(tmp_path / "out.bin", dtype=dtype)
    got = (out[: n * ny].reshape(n, ny), out[n * ny : 4 * n * ny].reshape(n, 3, ny),
           out[4 * n * ny :].reshape(n, 3, 3, ny))
    want = oracle.compute(xyz, l_max, kind == "spherical", "hessians")
    for g, w in zip(got, want):
        assert same_numbers(g, w).all()
