"""Host-side checks that need no GPU: the shared library loads, exports every symbol the headers
declare, plans launches sensibly, and the Python calculators validate their input."""

import ctypes
import os
import re
import subprocess
import sys

import numpy as np
import pytest
import torch

import sphericart_amd
from sphericart_amd import _c_lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sphx_[a-z0-9_]+|sphericart_cuda_[a-z_]+harmonics_[a-z_]+?(?:_f)?)\s*\(", text)))


def test_every_declared_symbol_is_exported(library):
    c_api = [s for s in _declared("sphericart.h") if not s.endswith("_t")]
    launch = _declared("sphx_launch.h")
    assert sorted(c_api) == sorted(_c_lib.C_API_SYMBOLS)
    assert len(c_api) == 20
    for name in c_api + launch:
        assert hasattr(library, name), name
    assert set(_c_lib.LAUNCH_SYMBOLS) <= set(launch)


def test_cxx_classes_are_exported(library):
    out = subprocess.run(["nm", "-DC", _c_lib.LIBRARY_PATH], capture_output=True, text=True, check=True).stdout
    for cls in ("SphericalHarmonics", "SolidHarmonics"):
        for t in ("float", "double"):
            assert f"sphericart::cuda::{cls}<{t}>::{cls}(unsigned long)" in out
    for method in ("compute", "compute_with_gradients", "compute_with_hessians"):
        assert f"sphericart::cuda::SphericalHarmonics<double>::{method}(" in out


def test_cxx_example_is_built_and_linked_against_the_library():
    example = os.path.join(ROOT, "sphericart_amd", "device_example")
    assert os.path.exists(example), "python -m sphericart_amd.build builds it next to the library"
    needed = subprocess.run(["ldd", example], capture_output=True, text=True, check=True).stdout
    assert "libsphericart_amd.so" in needed


def test_header_compiles_as_c_and_cxx(tmp_path):
    """include/sphericart.h is a C header and a C++ header; sphx_launch.h is plain C."""
    c_file = tmp_path / "probe.c"
    c_file.write_text('#include "sphericart.h"\n#include "sphx_launch.h"\nint main(void) { return 0; }\n')
    subprocess.run(["gcc", "-std=c99", "-fsyntax-only", f"-I{ROOT}/include", str(c_file)], check=True)
    cxx_file = tmp_path / "probe.cpp"
    cxx_file.write_text(
        '#include "sphericart.h"\n#include "sphericart_cuda.hpp"\n'
        "int main() { sphericart::cuda::SolidHarmonics<float>* p = nullptr; (void)p; return 0; }\n"
    )
    subprocess.run(["g++", "-std=c++17", "-fsyntax-only", f"-I{ROOT}/include", str(cxx_file)], check=True)


def _plan(library, n, l_max, mode, f64):
    out = [ctypes.c_int() for _ in range(4)]
    status = library.sphx_plan(n, l_max, mode, int(f64), *[ctypes.byref(v) for v in out])
    return status, [v.value for v in out]


def test_launch_plans(library):
    # gradients at l_max = 6: the closed forms in slices for eight waves, 32 points per workgroup
    status, (tile, threads, lds, groups) = _plan(library, 1_000_000, 6, 1, False)
    assert status == 0 and tile == 32 and threads == 512
    assert lds == 32 * 4 * 49 * 4 and groups == 31256  # 8 XCD stretches of 3907 tiles
    # values at l_max = 6: one wave per 64 points
    status, (tile, threads, lds, groups) = _plan(library, 1_000_000, 6, 0, False)
    assert status == 0 and tile == 64 and threads == 64
    assert lds == 64 * 49 * 4 and groups == 15632  # 8 XCD stretches of 1954 tiles
    for n, l_max, mode, f64 in ((10_000, 8, 1, True), (100_000, 16, 2, True), (200_000, 32, 1, False), (5, 20, 2, False)):
        status, (tile, threads, lds, groups) = _plan(library, n, l_max, mode, f64)
        assert status == 0
        assert 1 <= tile <= 64 and threads % 64 == 0 and 256 <= threads <= 1024 and lds <= 160 * 1024
        assert groups % 8 == 0 and groups >= 8
    # cfg5: pairs_kernel, one workgroup per CU with nearly all of its LDS, five points per tile (three prep
    # waves, four sequence waves, eight entry waves for the 507 pairs of a point);
    # the same shape with few points: recursion_kernel in workgroups of 512 threads
    status, (tile, threads, lds, groups) = _plan(library, 200_000, 32, 1, False)
    assert status == 0 and (tile, threads, groups) == (5, 960, 256) and 140_000 < lds <= 160 * 1024
    status, (tile, threads, lds, groups) = _plan(library, 2_000, 32, 1, False)
    assert status == 0 and threads == 512 and lds <= 80 * 1024
    # second derivatives in float64 keep 512 threads (more than 128 registers per lane); solid harmonics, whose
    # entries (l, +m) and (l, -m) fit 128 registers as two jobs, take 1024 (cfg4)
    assert _plan(library, 100_000, 16, 2, True)[1][1] == 512
    text = ctypes.create_string_buffer(512)
    assert library.sphx_describe_plan(100_000, 16, 2, 1, 0, text, 512) == 0
    assert text.value.decode().startswith("recursion_kernel<double, 2, false, true, true, false, true> [4 points per tile, 1024 threads")
    assert library.sphx_describe_plan(100_000, 16, 2, 1, 1, text, 512) == 0
    assert "512 threads" in text.value.decode()
    # values: as many points per workgroup as fit in half a CU's LDS, in steps of four; in float32
    # one workgroup with all of LDS while 40 points fit; from l_max = 24 (float64: 19) pairs_kernel with as
    # many points per tile as fit (and the lanes kernel again where there are few points)
    status, (tile, threads, lds, groups) = _plan(library, 1_000_000, 16, 0, False)
    assert status == 0 and (tile, threads) == (60, 512) and lds == 60 * (289 + 51) * 4
    status, (tile, threads, lds, groups) = _plan(library, 1_000_000, 28, 0, False)
    assert status == 0 and (tile, threads, groups) == (25, 1024, 256) and 150_000 < lds <= 160 * 1024
    status, (tile, threads, lds, groups) = _plan(library, 20_000, 28, 0, False)
    assert status == 0 and (tile, threads) == (44, 768) and 80 * 1024 < lds <= 160 * 1024
    # tiles of 32 and 16 points: two and four channels side by side in a wave
    assert _plan(library, 1_000_000, 22, 0, False)[1][:2] == [32, 512]
    assert _plan(library, 20_000, 26, 0, False)[1][:2] == [16, 320]
    assert _plan(library, 20_000, 32, 0, False)[1][:2] == [32, 832]
    assert _plan(library, 20_000, 34, 0, False)[1][1] == 1024
    assert _plan(library, 20_000, 22, 0, True)[1][:2] == [32, 1024]
    assert _plan(library, 20_000, 23, 0, True)[1][1] == 1024
    assert _plan(library, 1_000_000, 32, 0, False)[1][:2] == [20, 1024]
    assert _plan(library, 1_000_000, 24, 0, True)[1][0] == 16
    assert _plan(library, 10, 65, 0, False)[0] == 2       # beyond the tables
    assert _plan(library, 10, 64, 2, True)[0] == 2        # one point's rows no longer fit in LDS
    assert b"LDS" in library.sphx_last_error()
    assert _plan(library, 10, -1, 0, False)[0] == 1
    assert _plan(library, 10, 3, 7, False)[0] == 1


def test_planner_overrides(library, switches):
    """sphx_set_switch changes what the next call plans; sphx_reset_switches restores the default;
    unknown names are refused. Environment variables alone change nothing."""
    default = _plan(library, 50_000, 14, 1, False)
    os.environ["SPHX_TILE"] = "3"
    try:
        assert _plan(library, 50_000, 14, 1, False) == default
    finally:
        del os.environ["SPHX_TILE"]
    switches("SPHX_TILE", 3)
    status, (tile, _, _, _) = _plan(library, 50_000, 14, 1, False)
    assert status == 0 and tile == 3 and default[1][0] != 3
    library.sphx_reset_switches()
    assert _plan(library, 50_000, 14, 1, False) == default
    # the same for pairs_kernel, which takes values and gradients from l_max = 20 on in float32
    default = _plan(library, 50_000, 20, 1, False)
    switches("SPHX_PAIRS_TILE", 3)
    status, (tile, _, _, _) = _plan(library, 50_000, 20, 1, False)
    assert status == 0 and tile == 3 and default[1][0] != 3
    switches("SPHX_PAIRS", 0)
    assert _plan(library, 50_000, 20, 1, False)[1][1] in (512, 1024)  # recursion_kernel again
    library.sphx_reset_switches()
    assert _plan(library, 50_000, 20, 1, False) == default
    # four channels side by side in a wave: that kernel exists for up to eight waves, whatever the shape asks
    switches("SPHX_VALUES_PACK", 4)
    switches("SPHX_PAIRS", 0)
    for l_max in (25, 33, 39, 40):
        status, (tile, threads, _, _) = _plan(library, 100_000, l_max, 0, False)
        assert status == 0 and threads <= 512, (l_max, tile, threads)
    library.sphx_reset_switches()
    assert library.sphx_set_switch(b"SPHX_NO_SUCH_SWITCH", 1) == 1
    assert b"unknown switch" in library.sphx_last_error()
    assert library.sphx_set_switch(None, 1) == 1


def test_asking_for_plans_keeps_the_plans_of_recent_calls_and_set_switch_wins_over_the_environment():
    """A process of its own with SPHX_DEBUG_SWITCHES: a switch set by the program before anything else still holds
    after the environment has been read."""
    code = (
        "import sys, ctypes; sys.path.insert(0, %r)\n"
        "from sphericart_amd import _c_lib\n"
        "lib = _c_lib.get_library()\n"
        "assert lib.sphx_set_switch(b'SPHX_TILE', 3) == 0\n"
        "out = [ctypes.c_int() for _ in range(4)]\n"
        "assert lib.sphx_plan(50000, 14, 1, 0, *[ctypes.byref(v) for v in out]) == 0\n"
        "print(out[0].value)\n"
    ) % ROOT
    env = dict(os.environ, SPHX_DEBUG_SWITCHES="1", SPHX_TILE="5")
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, check=True, env=env).stdout
    assert out.strip() == "3"
    del env["SPHX_TILE"]
    env["SPHX_SEQUENCE_WAVES"] = "1"  # (another switch from the environment is still read)
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, check=True, env=env).stdout
    assert out.strip() == "3"


def test_static_scratch_capacity(library):
    # 32 MiB / (8 * (3 + (l_max + 1)^2 * {1, 4, 13}))
    assert library.sphx_forward_f32_via_f64_static_capacity(6, 1) == (32 << 20) // (8 * (3 + 49 * 4))
    assert library.sphx_forward_f32_via_f64_static_capacity(32, 2) == (32 << 20) // (8 * (3 + 1089 * 13))
    assert library.sphx_forward_f32_via_f64_static_capacity(-1, 0) == 0
    assert library.sphx_forward_f32_via_f64_static_capacity(4, 3) == 0
    # zero points: nothing is looked at
    assert library.sphx_forward_f32_via_f64_static(None, 0, 4, 1, 1, None, None, None, None) == 0
    assert library.sphx_forward_f32_via_f64_static(None, 5, 4, 1, 0, None, None, None, None) == 1


def test_zero_samples_is_a_no_op(library):
    # returns before touching pointers or the GPU (reference: sphericart_cuda.cpp:85-89)
    assert library.sphx_forward_f32(None, 0, 4, 1, 2, None, None, None, None) == 0
    assert library.sphx_forward_f64(None, 0, 4, 0, 0, None, None, None, None) == 0


def test_null_pointers_are_rejected(library):
    assert library.sphx_forward_f32(None, 3, 4, 1, 0, None, None, None, None) == 1
    assert b"null" in library.sphx_last_error()


def test_python_calculators_validate_input():
    calc = sphericart_amd.SphericalHarmonics(4)
    with pytest.raises(TypeError):
        calc.compute(np.zeros((3, 3)))
    with pytest.raises(TypeError):
        calc.compute(torch.zeros((3, 3), dtype=torch.float16))
    with pytest.raises(ValueError):
        calc.compute(torch.zeros((3, 4)))
    with pytest.raises(ValueError, match="no CPU evaluation path"):
        calc.compute(torch.zeros((3, 3)))
    with pytest.raises(ValueError):
        sphericart_amd.SolidHarmonics(-1)


def test_missing_library_fails_loudly(tmp_path):
    """Without the built library there is nothing to fall back to."""
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "from sphericart_amd import _c_lib\n"
        "_c_lib.LIBRARY_PATH = %r\n"
        "try:\n    _c_lib.get_library()\nexcept RuntimeError as e:\n    print('RuntimeError', e)\n"
    ) % (ROOT, str(tmp_path / "absent.so"))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, check=True).stdout
    assert "RuntimeError" in out and "no CPU or pure-Python evaluation path" in out


@pytest.mark.skipif(torch.cuda.is_available(), reason="only meaningful without a GPU")
def test_no_gpu_means_no_calculator(library):
    """`new` maps the constructor's exception to NULL (reference: sphericart-capi.cpp:637-643)."""
    assert library.sphericart_cuda_spherical_harmonics_new(3) is None
    assert library.sphericart_cuda_solid_harmonics_new_f(3) is None
