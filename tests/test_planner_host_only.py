"""The planner is plain host C++: sphx_plan.cpp compiles with g++ alone (no HIP header, no device) into a small
program, whose plans for a spread of shapes are those the library reports through sphx_describe_plan, word for
word, and name the kernels the shapes are meant to get."""

import ctypes
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "sphericart_amd", "csrc")

SHAPES = [
    # n_samples, l_max, mode, is_f64, normalized, the kernel it is meant to get
    (1_000_000, 6, 1, 0, 1, "gradients_lanes_kernel<float, true>"),
    (1_000_000, 3, 0, 0, 1, "closed_form_kernel<float, 0, true, 3, false>"),
    (10_000, 8, 1, 1, 1, "gradients_lanes_kernel<double, true>"),
    (100_000, 16, 2, 1, 0, "recursion_kernel<double, 2, false, true, true, false, true>"),
    (200_000, 32, 1, 0, 1, "pairs_kernel<float, 1, true>"),
    (200_000, 32, 0, 0, 1, "pairs_kernel<float, 0, true>"),
    (200_000, 20, 0, 1, 0, "pairs_kernel<double, 0, false>"),
    (1_000_000, 10, 0, 0, 1, "values_kernel<float, true, 1>"),
    (1_000_000, 22, 0, 0, 1, "values_kernel<float, true, 2>"),
    (500_000, 5, 2, 0, 1, "recursion_kernel<float, 2, true, true, false, false, true>"),
    (500_000, 3, 2, 0, 1, "hessians_lanes_kernel<float, true>"),
    (1_000_000, 10, 1, 0, 1, "recursion_kernel<float, 1, true, true, false, false, true>"),
    (50_000, 20, 2, 1, 1, "pairs_kernel<double, 2, true>"),
    (2_000, 32, 1, 0, 1, "recursion_kernel<float, 1, true, true, false, false, true>"),
    (2_000, 40, 1, 1, 1, "recursion_kernel<double, 1, true, false, false, false, false>"),
    (5, 24, 2, 1, 1, "recursion_kernel<double, 2, true, true, false, false, false>"),
    (1, 0, 0, 0, 1, "closed_form_kernel<float, 0, true, 0, false>"),
    # the flush at raised priority: by the table of shapes, and only with many tiles per workgroup
    (200_000, 33, 1, 0, 0, "pairs_kernel<float, 1, false>"),
    (40_000, 33, 1, 0, 0, "pairs_kernel<float, 1, false>"),
    (300_000, 10, 2, 0, 0, "recursion_kernel<float, 2, false, true, false, false, true>"),
    (300_000, 9, 2, 0, 0, "recursion_kernel<float, 2, false, true, false, false, true>"),
]
PRIORITY = {(200_000, 33): True, (40_000, 33): False, (300_000, 10): True, (300_000, 9): False}


@pytest.fixture(scope="module")
def probe(tmp_path_factory):
    binary = tmp_path_factory.mktemp("planner") / "planner_probe"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", os.path.join(ROOT, "tests", "planner_probe.cpp"),
                    os.path.join(CSRC, "sphx_plan.cpp"), "-o", str(binary)], check=True)
    return str(binary)


def test_plans_without_a_device_match_the_library_and_name_the_intended_kernels(probe, library):
    args = [str(v) for shape in SHAPES for v in shape[:5]]
    lines = subprocess.run([probe] + args, capture_output=True, text=True, check=True).stdout.splitlines()
    assert len(lines) == len(SHAPES)
    library.sphx_reset_switches()
    for (n, l_max, mode, is_f64, normalized, kernel), line in zip(SHAPES, lines):
        text = ctypes.create_string_buffer(1024)
        assert library.sphx_describe_plan(n, l_max, mode, is_f64, normalized, text, len(text)) == 0
        assert line == text.value.decode(), (n, l_max, mode, is_f64, normalized)
        assert line.split(" + ")[-1].startswith(kernel + " ["), (line, kernel)
        assert line.endswith("(flush at raised priority)") == PRIORITY.get((n, l_max), False), line


def test_shapes_beyond_the_tables_or_lds_are_refused_with_a_message(probe):
    out = subprocess.run([probe, "10", "65", "0", "0", "1", "10", "64", "2", "1", "1"], capture_output=True, text=True,
                         check=True).stdout.splitlines()
    assert out[0].startswith("status 2:") and "prefactor tables" in out[0]
    assert out[1].startswith("status 2:") and "LDS" in out[1]
