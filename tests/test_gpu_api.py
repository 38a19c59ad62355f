"""Behaviour of the boundary on a real GPU: sizes, alignment, streams, error conventions."""

import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import sphericart_amd
from gpu_utils import announce, run_calculator, run_launch_layer
from helpers import MODES, same_numbers, special_points

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("l_max,mode", [(3, "values"), (6, "gradients"), (1, "hessians"), (9, "gradients"), (5, "hessians"),
                                        (7, "values"), (12, "values"), (24, "values")])
def test_ragged_sizes(oracle, l_max, mode):
    """Point counts around the tile sizes, including a single point (tail tiles are partial)."""
    rng = np.random.default_rng(0)
    for n in (1, 2, 3, 7, 63, 64, 65, 127, 129, 255, 1000, 4099):
        for dtype in (np.float32, np.float64):
            announce("ragged", l_max, mode, n, np.dtype(dtype).name)
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, True, mode)
            got = run_calculator(xyz, l_max, True, mode)
            for g, w in zip(got, want):
                if w is not None:
                    assert same_numbers(g, w).all(), (n, dtype)


def test_zero_points():
    """Reference: python/tests/test_corner_cases.py:7-32 and
    sphericart-torch/python/tests/test_no_points.py:32-45."""
    for l_max in (0, 3, 7, 10, 20, 50):
        for cls in (sphericart_amd.SphericalHarmonics, sphericart_amd.SolidHarmonics):
            calc = cls(l_max)
            for dtype in (torch.float32, torch.float64):
                xyz = torch.empty((0, 3), dtype=dtype, device="cuda")
                sph, dsph, ddsph = calc.compute_with_hessians(xyz)
                assert sph.shape == (0, (l_max + 1) ** 2)
                assert dsph.shape == (0, 3, (l_max + 1) ** 2)
                assert ddsph.shape == (0, 3, 3, (l_max + 1) ** 2)
            del calc  # double delete must be harmless
    calc = sphericart_amd.SphericalHarmonics(2)
    calc._ensure_cuda_calculators()
    calc.__del__()
    calc.__del__()


def test_unaligned_outputs_take_the_narrow_store_path(oracle, library):
    """Output pointers that are not 16-byte aligned still give the same numbers."""
    rng = np.random.default_rng(1)
    for dtype, tdtype in ((np.float32, torch.float32), (np.float64, torch.float64)):
        for l_max, mode in ((6, "gradients"), (7, "gradients"), (3, "hessians"), (3, "values"), (7, "values"),
                            (8, "values"), (11, "values"), (24, "values")):
            announce("unaligned", np.dtype(dtype).name, l_max, mode)
            n, ny = 333, (l_max + 1) ** 2
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, True, mode)
            sizes = (n * ny, 3 * n * ny, 9 * n * ny)
            shapes = ((n, ny), (n, 3, ny), (n, 3, 3, ny))
            raw = [torch.zeros(s + 1, dtype=tdtype, device="cuda") for s in sizes]
            out = tuple(raw[i][1:].view(shapes[i]) if w is not None else None for i, w in enumerate(want))
            assert out[0].data_ptr() % 16 != 0
            status, _ = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, True, mode, out=out)
            assert status == 0, library.sphx_last_error()
            torch.cuda.synchronize()
            for o, w in zip(out, want):
                if w is not None:
                    assert same_numbers(o.cpu().numpy(), w).all()


@pytest.mark.parametrize("shift", [0, 1, 5])
def test_many_tiles_per_workgroup_with_shifted_outputs(oracle, library, shift):
    """Enough points that every workgroup of the recursion kernel walks several chunks of tiles,
    with outputs that start `shift` elements into a 128-byte line: the lines that consecutive
    tiles share are carried from one tile to the next and must come out complete."""
    rng = np.random.default_rng(7 + shift)
    cases = ((np.float32, torch.float32, 7, "gradients"), (np.float64, torch.float64, 10, "gradients"),
             (np.float32, torch.float32, 3, "hessians"), (np.float64, torch.float64, 12, "hessians"),
             (np.float32, torch.float32, 9, "values"))
    for dtype, tdtype, l_max, mode in cases:
        announce("many tiles", np.dtype(dtype).name, l_max, mode, "shift", shift)
        n, ny = 40_003, (l_max + 1) ** 2
        xyz = special_points(dtype, rng, n)
        want = oracle.compute(xyz, l_max, False, mode)
        sizes = (n * ny, 3 * n * ny, 9 * n * ny)
        shapes = ((n, ny), (n, 3, ny), (n, 3, 3, ny))
        raw = [torch.full((s + 64,), float("nan"), dtype=tdtype, device="cuda") for s in sizes]
        out = tuple(raw[i][shift:shift + sizes[i]].view(shapes[i]) if w is not None else None
                    for i, w in enumerate(want))
        status, _ = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, False, mode, out=out)
        assert status == 0, library.sphx_last_error()
        torch.cuda.synchronize()
        for i, (o, w) in enumerate(zip(out, want)):
            if w is not None:
                assert same_numbers(o.cpu().numpy(), w).all()
                # nothing written outside the arrays
                assert torch.isnan(raw[i][:shift]).all() and torch.isnan(raw[i][shift + sizes[i]:]).all()


@pytest.mark.parametrize("route", ["lanes", "recursion"])
@pytest.mark.parametrize("dtype,tdtype", [(np.float32, torch.float32), (np.float64, torch.float64)])
def test_second_derivatives_at_small_l_max_by_both_kernels(oracle, library, route, dtype, tdtype, switches):
    """l_max 2 ... 8 with Hessians through the one-point-per-lane kernel wherever its rows fit and
    through the recursion kernel (the library picks per l_max by itself; the switch is set
    for this test), sizes around a tile, shifted outputs with guard elements."""
    switches("SPHX_HESSIAN_LANES", "2" if route == "lanes" else "0")
    rng = np.random.default_rng(17)
    for l_max in range(2, 9):
        for n, shift in ((1, 0), (31, 1), (64, 0), (65, 2), (2049, 0), (4133, 3)):
            normalized = bool((l_max + n) & 1)
            announce("small l_max hessians", route, np.dtype(dtype).name, l_max, n, shift, normalized)
            ny = (l_max + 1) ** 2
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, "hessians")
            sizes = (n * ny, 3 * n * ny, 9 * n * ny)
            shapes = ((n, ny), (n, 3, ny), (n, 3, 3, ny))
            raw = [torch.full((s + 16,), float("nan"), dtype=tdtype, device="cuda") for s in sizes]
            out = tuple(raw[i][shift:shift + sizes[i]].view(shapes[i]) for i in range(3))
            status, _ = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, normalized, "hessians",
                                         out=out)
            assert status == 0, library.sphx_last_error()
            torch.cuda.synchronize()
            for i, (o, w) in enumerate(zip(out, want)):
                assert same_numbers(o.cpu().numpy(), w).all(), (l_max, n, i)
                assert torch.isnan(raw[i][:shift]).all() and torch.isnan(raw[i][shift + sizes[i]:]).all()


@pytest.mark.parametrize("launches", ["one", "two"])
def test_rows_cut_at_l7_by_one_launch_and_by_two(oracle, library, launches, switches):
    """Few points per tile: the recursion kernel stages l >= 7 and l <= 6 comes either from its
    wave 0 (the default) or from a launch of the closed-form kernel before it (switch set for this
    test). Sizes around the batches of 64 points, workgroups without tiles included."""
    switches("SPHX_PREFIX_INSIDE", "1" if launches == "one" else "0")
    rng = np.random.default_rng(23)
    cases = ((np.float32, torch.float32, 20, "gradients"), (np.float32, torch.float32, 32, "gradients"),
             (np.float64, torch.float64, 14, "gradients"), (np.float32, torch.float32, 36, "values"),
             (np.float64, torch.float64, 26, "values"))
    for dtype, tdtype, l_max, mode in cases:
        for n, shift in ((1, 0), (63, 1), (65, 0), (1000, 3), (4133, 0)):
            normalized = bool((l_max + n) & 1)
            announce("rows cut", launches, np.dtype(dtype).name, l_max, mode, n, shift, normalized)
            ny = (l_max + 1) ** 2
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, mode)
            sizes = (n * ny, 3 * n * ny)
            shapes = ((n, ny), (n, 3, ny))
            raw = [torch.full((s + 16,), float("nan"), dtype=tdtype, device="cuda") for s in sizes]
            out = tuple(raw[i][shift:shift + sizes[i]].view(shapes[i]) if want[i] is not None else None
                        for i in range(2)) + (None,)
            status, _ = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, normalized, mode, out=out)
            assert status == 0, library.sphx_last_error()
            torch.cuda.synchronize()
            for i in range(2):
                if want[i] is not None:
                    assert same_numbers(out[i].cpu().numpy(), want[i]).all(), (l_max, n, i)
                    assert torch.isnan(raw[i][:shift]).all() and torch.isnan(raw[i][shift + sizes[i]:]).all()


@pytest.mark.parametrize("tile", [3, 5, 7])
def test_recursion_kernel_with_tiles_that_are_no_power_of_two(oracle, library, tile, switches):
    """The planner takes as many points per tile as fit; here sizes it would not pick are forced
    (switches set for this test), with the lane kernels off so that the recursion kernel
    runs at every l_max."""
    switches("SPHX_TILE", str(tile))
    switches("SPHX_GRADIENT_LANES", "0")
    switches("SPHX_HESSIAN_LANES", "0")
    switches("SPHX_VALUES_LDS", "1")
    rng = np.random.default_rng(29 + tile)
    cases = ((np.float32, 9, "hessians"), (np.float64, 8, "hessians"), (np.float32, 12, "gradients"),
             (np.float64, 13, "gradients"), (np.float32, 20, "gradients"), (np.float64, 10, "values"))
    for dtype, l_max, mode in cases:
        for n in (1, tile, 8 * tile + 1, 3001):
            announce("odd tiles", tile, np.dtype(dtype).name, l_max, mode, n)
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, True, mode)
            status, out = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, True, mode)
            assert status == 0, library.sphx_last_error()
            torch.cuda.synchronize()
            for o, w in zip(out, want):
                if w is not None:
                    assert same_numbers(o.cpu().numpy().reshape(w.shape), w).all(), (l_max, mode, n)


@pytest.mark.parametrize("order", ["list", "points"])
def test_entry_jobs_as_one_list_and_point_by_point(oracle, library, order, switches):
    """The two variants of the recursion kernel's entry stage (the jobs of a tile as one list
    over the lanes, or whole points side by side; the planner picks per shape, the switch forces
    one wherever the other would save nothing), with enough points for full tiles."""
    switches("SPHX_JOB_LIST", "1" if order == "list" else "0")
    switches("SPHX_GRADIENT_LANES", "0")
    switches("SPHX_HESSIAN_LANES", "0")
    switches("SPHX_VALUES_LDS", "1")
    rng = np.random.default_rng(31)
    cases = ((np.float32, 17, "gradients"), (np.float32, 20, "gradients"), (np.float64, 16, "gradients"),
             (np.float32, 14, "hessians"), (np.float64, 14, "hessians"), (np.float32, 34, "values"),
             (np.float64, 9, "gradients"), (np.float32, 8, "hessians"))
    for dtype, l_max, mode in cases:
        n = 6007
        normalized = bool(l_max & 1)
        announce("entry jobs", order, np.dtype(dtype).name, l_max, mode, normalized)
        xyz = special_points(dtype, rng, n)
        want = oracle.compute(xyz, l_max, normalized, mode)
        status, out = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, normalized, mode)
        assert status == 0, library.sphx_last_error()
        torch.cuda.synchronize()
        for o, w in zip(out, want):
            if w is not None:
                assert same_numbers(o.cpu().numpy().reshape(w.shape), w).all(), (l_max, mode)


def test_lds_size_alternates_between_launches(oracle):
    """One kernel, launches that need more, then less, then more LDS again (all above 64 KB)."""
    rng = np.random.default_rng(21)
    xyz = special_points(np.float32, rng, 2000)
    for l_max in (8, 10, 8, 12, 9, 8):
        announce("alternating LDS", l_max)
        want = oracle.compute(xyz, l_max, True, "gradients")
        got = run_calculator(xyz, l_max, True, "gradients")
        for g, w in zip(got, want):
            if w is not None:
                assert same_numbers(g, w).all(), l_max


def test_calls_from_several_host_threads(oracle, library):
    """Four host threads, each on a stream of its own, shapes that need different kernels and
    LDS sizes, started together on a fresh set of shapes (the per-kernel facts are cached under a
    lock, the last error is per thread)."""
    import threading

    rng = np.random.default_rng(33)
    shapes = [(13, "values", np.float32), (9, "gradients", np.float64), (4, "hessians", np.float32),
              (14, "gradients", np.float32)]
    clouds = [special_points(dtype, rng, 1500) for _, _, dtype in shapes]
    wanted = [oracle.compute(xyz, l_max, True, mode) for xyz, (l_max, mode, _) in zip(clouds, shapes)]
    results, errors = [None] * len(shapes), []
    gate = threading.Barrier(len(shapes))

    def work(i):
        try:
            l_max, mode, _ = shapes[i]
            stream = torch.cuda.Stream()
            d_xyz = torch.from_numpy(clouds[i]).cuda()
            torch.cuda.synchronize()
            gate.wait()
            for _ in range(20):
                status, out = run_launch_layer(library, d_xyz, l_max, True, mode, stream=stream.cuda_stream)
                if status != 0:
                    raise RuntimeError(library.sphx_last_error())
            stream.synchronize()
            results[i] = [o.cpu().numpy() if o is not None else None for o in out]
        except Exception as exc:  # reported by the main thread
            errors.append((i, repr(exc)))

    announce("host threads", shapes)
    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(shapes))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    for got, want in zip(results, wanted):
        for g, w in zip(got, want):
            if w is not None:
                assert same_numbers(g, w).all()


def test_non_contiguous_input(oracle):
    """Reference: sphericart-torch/python/tests/test_autograd.py:88-124 (inputs are made contiguous)."""
    rng = np.random.default_rng(2)
    wide = torch.from_numpy(rng.normal(size=(100, 6))).cuda()
    xyz = wide[:, ::2]
    assert not xyz.is_contiguous()
    calc = sphericart_amd.SolidHarmonics(5)
    sph, dsph = calc.compute_with_gradients(xyz)
    want = oracle.compute(xyz.cpu().numpy().copy(), 5, False, "gradients")
    assert same_numbers(sph.cpu().numpy(), want[0]).all()
    assert same_numbers(dsph.cpu().numpy(), want[1]).all()


def test_user_streams(oracle):
    """Work goes to the caller's stream; two streams give the same numbers
    (reference: sphericart-torch/python/tests/test_cuda_stream.py:15-29)."""
    rng = np.random.default_rng(3)
    xyz_host = rng.normal(size=(5000, 3)).astype(np.float32)
    want = oracle.compute(xyz_host, 8, True, "gradients")
    calc = sphericart_amd.SphericalHarmonics(8)
    results = []
    for _ in range(2):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            xyz = torch.from_numpy(xyz_host).cuda()
            sph, dsph = calc.compute_with_gradients(xyz)
        stream.synchronize()
        results.append((sph.cpu().numpy(), dsph.cpu().numpy()))
    for sph, dsph in results:
        assert same_numbers(sph, want[0]).all() and same_numbers(dsph, want[1]).all()


def test_offsets_beyond_32_bits(oracle, library):
    """Element offsets past 2^31 (the reference's device kernel indexes with int,
    sphericart/src/sphericart_impl.cu:159,195): check the last rows of a 2.4e9-element dsph."""
    l_max, n = 32, 740_000
    ny = (l_max + 1) ** 2
    assert 3 * n * ny > 2**31
    announce("large offsets", n, l_max)
    rng = np.random.default_rng(4)
    tail = rng.normal(size=(2000, 3)).astype(np.float32)
    xyz = torch.ones((n, 3), dtype=torch.float32, device="cuda")
    xyz[-2000:] = torch.from_numpy(tail).cuda()
    status, (sph, dsph, _) = run_launch_layer(library, xyz, l_max, True, "gradients")
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    want = oracle.compute(tail, l_max, True, "gradients")
    assert same_numbers(sph[-2000:].cpu().numpy(), want[0]).all()
    assert same_numbers(dsph[-2000:].cpu().numpy(), want[1]).all()
    first = oracle.compute(np.ones((1, 3), dtype=np.float32), l_max, True, "gradients")
    assert same_numbers(dsph[:1].cpu().numpy(), first[1]).all()


def test_unsupported_l_max():
    calc = sphericart_amd.SphericalHarmonics(65)
    with pytest.raises(RuntimeError, match="failed to initialize"):
        calc.compute(torch.zeros((4, 3), device="cuda"))


def test_rows_too_large_for_lds_are_reported(library):
    xyz = torch.ones((4, 3), dtype=torch.float64, device="cuda")
    status, _ = run_launch_layer(library, xyz, 60, True, "hessians")
    assert status == 2
    assert b"LDS" in library.sphx_last_error()


def test_c_api_aborts_on_null_output():
    """compute_* print `fatal error: ...` and abort (reference: sphericart-capi.cpp:653-666).
    The check happens on the host before any device work, so the child needs no device memory:
    non-null integers stand in for `xyz` and `sph` and nothing ever looks at them."""
    code = (
        "import sys; sys.path.insert(0, %r)\n"
        "import sphericart_amd\n"
        "lib = sphericart_amd.get_library()\n"
        "calc = lib.sphericart_cuda_spherical_harmonics_new_f(3)\n"
        "assert calc\n"
        "print('before', flush=True)\n"
        "lib.sphericart_cuda_spherical_harmonics_compute_array_with_gradients_f(calc, 4096, 4, 8192, None, None)\n"
        "print('after', flush=True)\n"
    ) % ROOT
    done = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert done.returncode == -6, (done.returncode, done.stdout, done.stderr)
    assert "before" in done.stdout and "after" not in done.stdout
    assert "fatal error:" in done.stdout and "dsph != nullptr" in done.stdout
