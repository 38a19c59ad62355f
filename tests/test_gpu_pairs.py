"""pairs_kernel (every entry lane bound to one (l, m) pair) against the oracle, number for number.

The planner gives it values alone in float32 from l_max = 23 and in float64 from l_max = 20, gradients in float32
from l_max = 20 and in float64 from l_max = 16, and second derivatives in float64 from l_max = 20, when a call
has 32 768 points or more; here SPHX_PAIRS = 2 sends every shape it can hold through it, with the tile, batch and wave counts
the planner would pick and with forced ones, so that every path of the kernel runs at sizes the oracle
finishes in seconds: partial last tiles, fewer tiles than workgroups, several points side by side in the
entry waves, several rounds of recursions per tile, outputs that start anywhere inside a 128-byte line.
"""

import ctypes

import numpy as np
import pytest
import torch

from gpu_utils import announce
from helpers import same_numbers, special_points

pytestmark = pytest.mark.gpu


def _evaluate(library, xyz, l_max, normalized, shift=0, mode=1):
    """sphx_forward_* with derivatives into buffers with NaN guard bands; returns (sph, dsph[, ddsph], guards intact)."""
    n = xyz.shape[0]
    ny = (l_max + 1) ** 2
    tdtype = torch.float32 if xyz.dtype == np.float32 else torch.float64
    sizes = (n * ny, 3 * n * ny, 9 * n * ny)[:mode + 1]
    shapes = ((n, ny), (n, 3, ny), (n, 3, 3, ny))
    raw = [torch.full((size + 64,), float("nan"), dtype=tdtype, device="cuda") for size in sizes]
    out = [raw[i][shift:shift + sizes[i]].view(shapes[i]) for i in range(mode + 1)]
    forward = library.sphx_forward_f32 if xyz.dtype == np.float32 else library.sphx_forward_f64
    xyz_dev = torch.from_numpy(xyz).cuda()
    status = forward(xyz_dev.data_ptr(), n, l_max, int(normalized), mode, out[0].data_ptr(),
                     out[1].data_ptr() if mode >= 1 else None, out[2].data_ptr() if mode == 2 else None,
                     torch.cuda.current_stream().cuda_stream)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    guards = all(bool(torch.isnan(raw[i][:shift]).all() and torch.isnan(raw[i][shift + sizes[i]:]).all())
                 for i in range(mode + 1))
    return tuple(o.cpu().numpy() for o in out) + (guards,)


def _plan_text(library, n, l_max, f64, normalized, mode=1):
    text = ctypes.create_string_buffer(512)
    assert library.sphx_describe_plan(n, l_max, mode, int(f64), int(normalized), text, 512) == 0
    return text.value.decode()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
def test_every_l_max_it_holds(oracle, library, switches, dtype, normalized):
    """l_max 7 .. 40 at a ragged number of points (a partial last tile, tiles of up to twelve points)."""
    rng = np.random.default_rng(7)
    switches("SPHX_PAIRS", 2)
    ran = 0
    for l_max in (7, 8, 9, 13, 16, 19, 20, 23, 24, 27, 31, 32, 33, 36, 40):
        n = 389 if l_max < 30 else 167
        text = _plan_text(library, n, l_max, dtype == np.float64, normalized)
        announce("pairs", np.dtype(dtype).name, "normalized", normalized, "l_max", l_max, "n", n, text)
        if not text.startswith("pairs_kernel"):
            continue  # more pairs than the entry waves have lanes, or rows too long for LDS
        ran += 1
        xyz = special_points(dtype, rng, n)
        want = oracle.compute(xyz, l_max, normalized, "gradients")
        sph, dsph, guards = _evaluate(library, xyz, l_max, normalized)
        assert same_numbers(sph, want[0]).all(), (l_max, "values")
        assert same_numbers(dsph, want[1]).all(), (l_max, "gradients")
        assert guards
    assert ran >= 10


def test_forced_tiles_batches_and_waves(oracle, library, switches):
    """Plans the planner would not make: every tile size, small and large batches, one to four sequence
    waves (several rounds of recursions per tile), one to three prep waves, chunks of one to eight tiles."""
    rng = np.random.default_rng(11)
    cases = [
        (np.float32, 32, {"SPHX_PAIRS_TILE": 1}),
        (np.float32, 32, {"SPHX_PAIRS_TILE": 2, "SPHX_PAIRS_SEQUENCE_WAVES": 1}),
        (np.float32, 32, {"SPHX_PAIRS_TILE": 3, "SPHX_PAIRS_BATCH": 3, "SPHX_PAIRS_PREP_WAVES": 3}),
        (np.float32, 32, {"SPHX_PAIRS_TILE": 4, "SPHX_PAIRS_CHUNK": 3}),
        (np.float32, 24, {"SPHX_PAIRS_TILE": 7, "SPHX_PAIRS_SEQUENCE_WAVES": 2}),
        (np.float32, 20, {"SPHX_PAIRS_TILE": 12, "SPHX_PAIRS_BATCH": 4}),
        (np.float32, 12, {"SPHX_PAIRS_TILE": 16, "SPHX_PAIRS_PREP_WAVES": 1}),
        (np.float32, 9, {"SPHX_PAIRS_TILE": 5, "SPHX_PAIRS_CHUNK": 0}),
        (np.float64, 28, {"SPHX_PAIRS_TILE": 1, "SPHX_PAIRS_CHUNK": 2}),
        (np.float64, 24, {"SPHX_PAIRS_TILE": 3, "SPHX_PAIRS_SEQUENCE_WAVES": 4}),
        (np.float64, 16, {"SPHX_PAIRS_TILE": 6, "SPHX_PAIRS_BATCH": 10}),
        (np.float64, 10, {"SPHX_PAIRS_TILE": 9, "SPHX_PAIRS_PREP_WAVES": 2, "SPHX_PAIRS_SEQUENCE_WAVES": 1}),
    ]
    for dtype, l_max, overrides in cases:
        library.sphx_reset_switches()
        switches("SPHX_PAIRS", 2)
        for name, value in overrides.items():
            switches(name, value)
        for n, normalized in ((1201, True), (77, False)):
            text = _plan_text(library, n, l_max, dtype == np.float64, normalized)
            announce("pairs forced", np.dtype(dtype).name, "l_max", l_max, overrides, "n", n, text)
            assert text.startswith("pairs_kernel"), text
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, "gradients")
            sph, dsph, guards = _evaluate(library, xyz, l_max, normalized, shift=int(rng.integers(0, 33)))
            assert same_numbers(sph, want[0]).all(), (l_max, overrides, n, "values")
            assert same_numbers(dsph, want[1]).all(), (l_max, overrides, n, "gradients")
            assert guards, (l_max, overrides, n)


def test_few_points_and_shifted_outputs(oracle, library, switches):
    """One point to a few tiles (most workgroups have no tile), outputs shifted by 0 .. 33 elements."""
    rng = np.random.default_rng(13)
    switches("SPHX_PAIRS", 2)
    for dtype, l_max in ((np.float32, 21), (np.float64, 17)):
        for n in (1, 2, 3, 4, 5, 11, 12, 13, 25, 64, 100):
            shift = int(rng.integers(0, 34))
            announce("pairs few points", np.dtype(dtype).name, "l_max", l_max, "n", n, "shift", shift)
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, True, "gradients")
            sph, dsph, guards = _evaluate(library, xyz, l_max, True, shift=shift)
            assert same_numbers(sph, want[0]).all(), (l_max, n, "values")
            assert same_numbers(dsph, want[1]).all(), (l_max, n, "gradients")
            assert guards, (l_max, n)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
def test_second_derivatives(oracle, library, switches, dtype, normalized):
    """The same kernel with second derivatives (closed forms only to l = 1, three recursions per l, thirteen rows
    per point, the lane table ordered by kind): l_max 2 .. 24, planned and forced tiles."""
    rng = np.random.default_rng(17)
    ran = 0
    for l_max, overrides in ((2, {}), (3, {"SPHX_PAIRS_TILE": 1}), (4, {}), (5, {"SPHX_PAIRS_TILE": 7}), (8, {}),
                             (9, {"SPHX_PAIRS_SEQUENCE_WAVES": 1, "SPHX_PAIRS_TILE": 5}), (12, {}),
                             (16, {"SPHX_PAIRS_TILE": 2, "SPHX_PAIRS_CHUNK": 0}), (16, {}), (20, {}),
                             (24, {"SPHX_PAIRS_BATCH": 9})):
        library.sphx_reset_switches()
        switches("SPHX_PAIRS", 2)
        switches("SPHX_HESSIAN_LANES", 0)
        for name, value in overrides.items():
            switches(name, value)
        n = 301 if l_max <= 12 else 83
        text = _plan_text(library, n, l_max, dtype == np.float64, normalized, mode=2)
        announce("pairs second derivatives", np.dtype(dtype).name, "normalized", normalized, "l_max", l_max, overrides,
                 "n", n, text)
        if not text.startswith("pairs_kernel"):
            continue
        ran += 1
        xyz = special_points(dtype, rng, n)
        want = oracle.compute(xyz, l_max, normalized, "hessians")
        sph, dsph, ddsph, guards = _evaluate(library, xyz, l_max, normalized, shift=int(rng.integers(0, 17)), mode=2)
        assert same_numbers(sph, want[0]).all(), (l_max, "values")
        assert same_numbers(dsph, want[1]).all(), (l_max, "gradients")
        assert same_numbers(ddsph, want[2]).all(), (l_max, "second derivatives")
        assert guards
    assert ran >= 8


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
def test_values_alone(oracle, library, switches, dtype, normalized):
    """The same kernel without derivatives (one row per point, a batch is a single tile of up to 64 points, the
    entry lanes take four points per turn): l_max 7 .. 36, planned and forced tiles, batches of several tiles,
    few points, outputs that start anywhere inside a line."""
    rng = np.random.default_rng(19)
    ran = 0
    for l_max, overrides in ((7, {}), (8, {"SPHX_PAIRS_TILE": 1}), (9, {"SPHX_PAIRS_TILE": 3, "SPHX_PAIRS_BATCH": 3}),
                             (12, {}), (16, {"SPHX_PAIRS_TILE": 5, "SPHX_PAIRS_SEQUENCE_WAVES": 1}), (20, {}),
                             (23, {"SPHX_PAIRS_TILE": 6, "SPHX_PAIRS_BATCH": 2, "SPHX_PAIRS_PREP_WAVES": 1}), (24, {}),
                             (27, {"SPHX_PAIRS_SEQUENCE_WAVES": 8}), (28, {}), (31, {"SPHX_PAIRS_TILE": 7}), (32, {}),
                             (33, {"SPHX_PAIRS_CHUNK": 2, "SPHX_PAIRS_TILE": 2}), (36, {})):
        library.sphx_reset_switches()
        switches("SPHX_PAIRS", 2)
        for name, value in overrides.items():
            switches(name, value)
        for n in (1, 5, 70, 333):
            text = _plan_text(library, n, l_max, dtype == np.float64, normalized, mode=0)
            announce("pairs values", np.dtype(dtype).name, "normalized", normalized, "l_max", l_max, overrides, "n", n, text)
            if not text.startswith("pairs_kernel"):
                continue
            ran += 1
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, "values")
            (sph, guards) = _evaluate(library, xyz, l_max, normalized, shift=int(rng.integers(0, 33)), mode=0)
            assert same_numbers(sph, want[0]).all(), (l_max, overrides, n, "values")
            assert guards, (l_max, overrides, n)
    assert ran >= 40


def test_planned_by_shape(library):
    """What the planner picks without overrides."""
    assert _plan_text(library, 200_000, 32, False, True).startswith("pairs_kernel<float, 1, true>")
    assert _plan_text(library, 100_000, 20, False, False).startswith("pairs_kernel<float, 1, false>")
    assert _plan_text(library, 100_000, 17, True, True).startswith("pairs_kernel<double, 1, true>")
    assert _plan_text(library, 50_000, 20, True, True, mode=2).startswith("pairs_kernel<double, 2, true>")
    assert _plan_text(library, 100_000, 16, True, False, mode=2).startswith("recursion_kernel")  # cfg4
    assert _plan_text(library, 100_000, 19, False, True).startswith("recursion_kernel")
    assert _plan_text(library, 100_000, 16, True, True).startswith("recursion_kernel")
    assert _plan_text(library, 50_000, 22, True, True, mode=2).startswith("recursion_kernel")
    assert _plan_text(library, 20_000, 32, False, True).startswith("recursion_kernel")  # few points
    assert _plan_text(library, 200_000, 32, False, True, mode=0).startswith("pairs_kernel<float, 0, true>")
    assert _plan_text(library, 200_000, 20, True, False, mode=0).startswith("pairs_kernel<double, 0, false>")
    assert _plan_text(library, 200_000, 22, False, True, mode=0).startswith("values_kernel")
    assert _plan_text(library, 200_000, 18, True, True, mode=0).startswith("values_kernel")
    assert _plan_text(library, 200_000, 23, False, True, mode=0).startswith("values_kernel")
    assert _plan_text(library, 20_000, 32, False, True, mode=0).startswith("values_kernel")  # few points
    # second derivatives in float32 stay where they were
    assert not _plan_text(library, 200_000, 24, False, True, mode=2).startswith("pairs")
