"""GPU results against the CPU oracle and the golden vectors, through the C entry points.

Bar (reference: python/tests/test_cupy.py:22-49): |gpu - cpu| <= 1e-5 max(1, |cpu|) in float32,
1e-12 max(1, |cpu|) in float64, and non-finite exactly where the reference is non-finite
(float32 prefactors overflow from l = 29). Because library and oracle are both built without
FMA contraction and follow the same operation order, the tests also demand the stronger
property that every number is identical.
"""

import numpy as np
import pytest
import torch

from golden_io import CONFIGS, config_case, degenerate_cases, edge_cases
from gpu_utils import announce, run_calculator, run_launch_layer
from helpers import MODES, same_numbers, special_points, within_tolerance
from sphericart_amd.workloads import WORKLOADS

pytestmark = pytest.mark.gpu

L_MAX_SWEEP = [0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 15, 16, 20, 23, 24, 25, 32]


def check(got, want, what):
    for g, w, label in zip(got, want, ("sph", "dsph", "ddsph")):
        assert (g is None) == (w is None), (what, label)
        if w is None:
            continue
        assert g.shape == w.shape and g.dtype == w.dtype, (what, label)
        ok = within_tolerance(g, w)
        assert ok.all(), (what, label, "outside tolerance:", int((~ok).sum()))
        same = same_numbers(g, w)
        assert same.all(), (what, label, "not identical:", int((~same).sum()))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
@pytest.mark.parametrize("mode", MODES)
def test_sweep_against_oracle(oracle, dtype, normalized, mode):
    rng = np.random.default_rng(42)
    for l_max in L_MAX_SWEEP:
        announce("sweep", np.dtype(dtype).name, "normalized" if normalized else "solid", mode, "l_max", l_max)
        xyz = special_points(dtype, rng, 777)
        want = oracle.compute(xyz, l_max, normalized, mode)
        got = run_calculator(xyz, l_max, normalized, mode)
        check(got, want, (l_max, normalized, mode))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
def test_closed_form_gradients_by_both_kernels(oracle, library, switches, dtype, normalized):
    """Gradients at l_max <= 6 have two kernels: one wave per 64 points, or the closed forms in
    slices for the waves of a workgroup (the planner's choice at l_max = 4-6). Both against the
    oracle, for every l_max, at sizes that leave tiles of 32, 64 and N / CUs points ragged."""
    rng = np.random.default_rng(7)
    for l_max in range(1, 7):
        for n in (1, 33, 777, 20001):
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, "gradients")
            xyz_dev = torch.from_numpy(xyz).cuda()
            for lanes in (1, 0):
                switches("SPHX_GRADIENT_LANES", lanes)
                announce("closed-form gradients", np.dtype(dtype).name, normalized, l_max, n, "lanes", lanes)
                status, got = run_launch_layer(library, xyz_dev, l_max, normalized, "gradients")
                torch.cuda.synchronize()
                assert status == 0, library.sphx_last_error()
                got = tuple(None if g is None else g.cpu().numpy() for g in got)
                check(got, want, (l_max, normalized, n, lanes))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
def test_second_derivative_lanes_with_shared_channels(oracle, library, switches, dtype, normalized):
    """The one-point-per-lane kernel for second derivatives at l_max 2-5, with one, two and four
    waves per l channel (each wave a part of the channel's m), against the oracle."""
    rng = np.random.default_rng(9)
    for l_max in range(2, 6):
        for n in (3, 100, 4097):
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, "hessians")
            xyz_dev = torch.from_numpy(xyz).cuda()
            for parts in (1, 2, 4):
                switches("SPHX_HESSIAN_LANES", 2)
                switches("SPHX_HESSIAN_LANES_PARTS", parts)
                announce("second derivatives, lanes", np.dtype(dtype).name, normalized, l_max, n, "parts", parts)
                status, got = run_launch_layer(library, xyz_dev, l_max, normalized, "hessians")
                torch.cuda.synchronize()
                assert status == 0, library.sphx_last_error()
                got = tuple(None if g is None else g.cpu().numpy() for g in got)
                check(got, want, (l_max, normalized, n, parts))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("normalized", [True, False])
def test_gradient_lanes_with_shared_channels(oracle, library, switches, dtype, normalized):
    """The one-point-per-lane kernel for gradients above the closed forms, with one and two waves
    per l channel (each wave half of the channel's m), in workgroups of eight, twelve and sixteen
    waves, few points (where the planner picks two waves per channel while waves are left for the
    closed forms) and many, against the oracle."""
    rng = np.random.default_rng(21)
    for l_max in (7, 8, 9, 10, 12):
        for n in (1, 50, 3000, 10000, 40000):
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, "gradients")
            xyz_dev = torch.from_numpy(xyz).cuda()
            for parts, waves in ((1, 8), (2, 8), (1, 16), (2, 16), (2, 12)):
                switches("SPHX_GRADIENT_LANES", 2)
                switches("SPHX_GRADIENT_LANES_WAVES", waves)
                switches("SPHX_GRADIENT_LANES_PARTS", parts)
                announce("gradients, lanes", np.dtype(dtype).name, normalized, l_max, n, "parts", parts, "waves", waves)
                status, got = run_launch_layer(library, xyz_dev, l_max, normalized, "gradients")
                torch.cuda.synchronize()
                assert status == 0, library.sphx_last_error()
                got = tuple(None if g is None else g.cpu().numpy() for g in got)
                check(got, want, (l_max, normalized, n, parts, waves))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_values_kernel_with_tiles_of_any_size(oracle, library, switches, dtype):
    """values_kernel takes as many points per workgroup as fit in LDS, in steps of four: tiles
    of 60, 44, 28 points and others, a last tile that is not full, two workgroups per CU and
    one with all of LDS, steps of one and halving; and tiles of 32 and 16 points with two and
    four channels side by side in a wave (channels that do not fill the last bundle, l_max =
    7-9, included). All against the oracle."""
    rng = np.random.default_rng(47)
    for l_max in (7, 8, 9, 11, 16, 19, 22, 23, 24, 26, 28, 32):
        for normalized in (True, False):
            for n in (1, 59, 1201):
                xyz = special_points(dtype, rng, n)
                want = oracle.compute(xyz, l_max, normalized, "values")
                xyz_dev = torch.from_numpy(xyz).cuda()
                for step, least, pack, alone in ((None, None, None, None), (1, 8, 1, 0), (0, 32, 1, 0), (4, 8, 1, 1),
                                                 (4, 8, 2, 0), (4, 8, 4, 0), (4, 8, 2, 1)):
                    library.sphx_reset_switches()
                    if step is not None:
                        switches("SPHX_VALUES_TILE_STEP", step)
                        switches("SPHX_VALUES_MIN_TILE", least)
                        switches("SPHX_VALUES_PACK", pack)
                        switches("SPHX_VALUES_ALONE", alone)
                    announce("values, tiles", np.dtype(dtype).name, normalized, l_max, n, "step", step, "pack", pack, "alone", alone)
                    status, got = run_launch_layer(library, xyz_dev, l_max, normalized, "values")
                    torch.cuda.synchronize()
                    assert status == 0, library.sphx_last_error()
                    got = tuple(None if g is None else g.cpu().numpy() for g in got)
                    check(got, want, (l_max, normalized, n, step, pack, alone))
    library.sphx_reset_switches()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("mode", ["values", "gradients", "hessians"])
def test_workgroups_of_512_and_1024_threads(oracle, library, switches, dtype, mode):
    """The recursion kernel in workgroups of 512 threads (two to a CU) and of 1024 (one, with all of
    its LDS, larger tiles, waves of their own for the closed forms, kinds of jobs at wave
    boundaries), many points and few, against the oracle. Second derivatives in float64 exist
    with 512 threads only; the switch is then ignored."""
    rng = np.random.default_rng(31)
    l_values = {"values": (9, 23, 31, 46), "gradients": (9, 12, 21, 32, 44), "hessians": (4, 7, 13, 22)}[mode]
    for l_max in l_values:
        for normalized in (True, False):
            n = 3001 if l_max < 30 else 1201
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, mode)
            xyz_dev = torch.from_numpy(xyz).cuda()
            for threads, extra in ((512, {}), (1024, {}), (1024, {"SPHX_SLICE_WAVES": 3, "SPHX_SEQUENCE_WAVES": 4}),
                                   (1024, {"SPHX_SLICE_WAVES": 0, "SPHX_SPREAD_KINDS": 0, "SPHX_JOB_LIST": 0})):
                library.sphx_reset_switches()
                switches("SPHX_GRADIENT_LANES", 0)
                switches("SPHX_HESSIAN_LANES", 0)
                switches("SPHX_VALUES_LDS", 1)
                switches("SPHX_GROUP_THREADS", threads)
                for name, value in extra.items():
                    switches(name, value)
                announce("workgroup size", np.dtype(dtype).name, mode, normalized, l_max, threads, extra)
                status, got = run_launch_layer(library, xyz_dev, l_max, normalized, mode)
                torch.cuda.synchronize()
                assert status == 0, library.sphx_last_error()
                got = tuple(None if g is None else g.cpu().numpy() for g in got)
                check(got, want, (l_max, normalized, threads, extra))
    library.sphx_reset_switches()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("mode", ["gradients", "hessians"])
def test_job_list_by_kind_and_points_side_by_side(oracle, library, switches, dtype, mode):
    """The recursion kernel deals the entry jobs of a tile either point by point, side by side,
    or as one list ordered by kind of job. Both, with tiles of one to many points (single jobs
    per kind at l_max = 2 and 3 included), against the oracle."""
    rng = np.random.default_rng(13)
    shapes = [(2, 0), (3, 0), (4, 3), (7, 0), (9, 5), (13, 0), (18, 2)] if mode == "hessians" else \
        [(7, 0), (8, 3), (12, 0), (17, 0), (21, 4), (26, 0), (33, 1)]
    for l_max, tile in shapes:
        for normalized in (True, False):
            n = 1500
            xyz = special_points(dtype, rng, n)
            want = oracle.compute(xyz, l_max, normalized, mode)
            xyz_dev = torch.from_numpy(xyz).cuda()
            for job_list in (2, 0):
                switches("SPHX_GRADIENT_LANES", 0)
                switches("SPHX_HESSIAN_LANES", 0)
                switches("SPHX_JOB_LIST", job_list)
                if tile:
                    switches("SPHX_TILE", tile)
                announce("job list", np.dtype(dtype).name, mode, normalized, l_max, "tile", tile, "list", job_list)
                status, got = run_launch_layer(library, xyz_dev, l_max, normalized, mode)
                torch.cuda.synchronize()
                assert status == 0, library.sphx_last_error()
                got = tuple(None if g is None else g.cpu().numpy() for g in got)
                check(got, want, (l_max, normalized, tile, job_list))
            library.sphx_reset_switches()


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_wave_priorities_change_no_number(oracle, library, switches, dtype):
    """The waves that flush a tile, or the ones that prepare the next, may run at raised priority in the two
    persistent kernels (the planner's choice by shape, SPHX_WAVE_PRIORITIES here): every setting against the
    oracle, on shapes of the recursion kernel and of pairs_kernel, many tiles per workgroup."""
    rng = np.random.default_rng(29)
    for mode, l_max, normalized, n, pairs in (("gradients", 12, False, 40000, 0), ("hessians", 10, False, 30000, 0),
                                              ("gradients", 21, True, 6000, 2), ("hessians", 20, False, 3000, 2)):
        xyz = special_points(dtype, rng, n)
        want = oracle.compute(xyz, l_max, normalized, mode)
        xyz_dev = torch.from_numpy(xyz).cuda()
        for priorities in (0, 1, 2, 3):
            switches("SPHX_PAIRS", pairs)
            switches("SPHX_WAVE_PRIORITIES", priorities)
            announce("wave priorities", np.dtype(dtype).name, mode, normalized, l_max, n, priorities)
            status, got = run_launch_layer(library, xyz_dev, l_max, normalized, mode)
            torch.cuda.synchronize()
            assert status == 0, library.sphx_last_error()
            got = tuple(None if g is None else g.cpu().numpy() for g in got)
            check(got, want, (l_max, normalized, mode, priorities))
        library.sphx_reset_switches()


@pytest.mark.parametrize("name", CONFIGS)
def test_golden_benchmark_configurations(name):
    xyz, l_max, normalized, mode, want = config_case(name)
    announce("golden", name)
    check(run_calculator(xyz, l_max, normalized, mode), want, name)


@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_golden_edge_cases(tag):
    for xyz, l_max, normalized, mode, want in edge_cases(tag):
        announce("golden edge", tag, l_max, normalized, mode)
        check(run_calculator(xyz, l_max, normalized, mode), want, (tag, l_max, normalized, mode))


@pytest.mark.parametrize("tag", ["f32", "f64"])
def test_golden_degenerate_points(tag):
    """The origin, NaN, infinite, denormal and overflowing coordinates, each between ordinary
    points of the same tile: what the compiled reference returns (it has no guard around
    1 / sqrt(x^2 + y^2 + z^2), sphericart/include/templates.hpp:392-400), number for number, NaN
    for NaN and signed infinity for signed infinity; the ordinary neighbours are unaffected."""
    for xyz, where, l_max, normalized, mode, want in degenerate_cases(tag):
        announce("golden degenerate", tag, l_max, normalized, mode)
        got = run_calculator(xyz, l_max, normalized, mode)
        for g, w, label in zip(got, want, ("sph", "dsph", "ddsph")):
            assert (g is None) == (w is None)
            if w is not None:
                same = same_numbers(g, w)
                bad_points = np.unique(np.nonzero(~same)[0])
                assert same.all(), (tag, l_max, normalized, mode, label, "points", bad_points[:10],
                                    "of which degenerate", np.intersect1d(bad_points, where)[:10])


@pytest.mark.parametrize("name", CONFIGS)
def test_benchmark_configurations_at_full_size(oracle, library, name):
    """The five configurations at their real sizes: every number against the oracle, in slabs."""
    w = WORKLOADS[name]
    announce("full size", name, w.description)
    xyz = w.points()
    xyz_dev = torch.from_numpy(xyz).cuda()
    status, out = run_launch_layer(library, xyz_dev, w.l_max, w.normalized, w.derivatives)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    slab = max(1, min(w.n_samples, (256 << 20) // w.bytes_per_point))
    for first in range(0, w.n_samples, slab):
        last = min(w.n_samples, first + slab)
        want = oracle.compute(xyz[first:last], w.l_max, w.normalized, w.derivatives)
        got = tuple(o[first:last].cpu().numpy() if o is not None else None for o in out)
        check(got, want, (name, first))


def test_literal_clouds_of_the_reference_at_full_size(oracle, library):
    """The first and the last benchmark configuration with their clouds drawn the way the reference's own scripts
    draw them, at full size: cfg1 as i.i.d. N(0, 1) components from numpy's generator, cfg5 with radii exp(u), u
    uniform in [ln 1e-2, ln 1e2), on directions uniform on the sphere (normalised normal deviates), 0.5 % of the
    points put on the +-z axis. The array is drawn here and handed to the GPU and to the oracle alike, so the
    C library's exp and numpy's generator need not agree between machines. (The seeded clouds of
    sphericart_amd.workloads stay the fixtures' and the benchmark's: those are the same bits everywhere.)"""
    rng = np.random.default_rng(20240521)
    clouds = {"cfg1": rng.standard_normal((10_000, 3))}
    n = 200_000
    directions = rng.standard_normal((n, 3))
    directions /= np.linalg.norm(directions, axis=1, keepdims=True)
    radii = np.exp(rng.uniform(np.log(1e-2), np.log(1e2), size=n))
    cloud = directions * radii[:, None]
    on_axis = np.arange(n) % 200 == 0
    cloud[on_axis, 0] = 0.0
    cloud[on_axis, 1] = 0.0
    cloud[on_axis, 2] = np.where(np.arange(n)[on_axis] % 400 == 0, 1.0, -1.0) * radii[on_axis]
    clouds["cfg5"] = cloud
    for name, xyz in clouds.items():
        w = WORKLOADS[name]
        xyz = np.ascontiguousarray(xyz.astype(w.numpy_dtype))
        assert xyz.shape == (w.n_samples, 3)
        announce("literal cloud", name, w.description)
        xyz_dev = torch.from_numpy(xyz).cuda()
        status, out = run_launch_layer(library, xyz_dev, w.l_max, w.normalized, w.derivatives)
        assert status == 0, library.sphx_last_error()
        torch.cuda.synchronize()
        slab = max(1, min(w.n_samples, (256 << 20) // w.bytes_per_point))
        for first in range(0, w.n_samples, slab):
            last = min(w.n_samples, first + slab)
            want = oracle.compute(xyz[first:last], w.l_max, w.normalized, w.derivatives)
            got = tuple(o[first:last].cpu().numpy() if o is not None else None for o in out)
            check(got, want, (name, first))


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_values_with_fewer_points_than_a_channel_has_prefactors(oracle, library, dtype):
    """values_kernel hands a channel's prefactors from lane to lane: with one, two or five points in a tile (or a
    last tile that holds so few) most of the lanes that hold a prefactor have no point. Every l_max the kernel
    takes, to the largest of the tables."""
    rng = np.random.default_rng(53)
    for l_max in (7, 10, 20, 33, 40, 63):
        for n in (1, 2, 5, 25, 45, 64 + 3):
            for normalized in (True, False):
                announce("values, few points", np.dtype(dtype).name, normalized, l_max, n)
                xyz = special_points(dtype, rng, n)
                want = oracle.compute(xyz, l_max, normalized, "values")
                status, got = run_launch_layer(library, torch.from_numpy(xyz).cuda(), l_max, normalized, "values")
                torch.cuda.synchronize()
                assert status == 0, library.sphx_last_error()
                got = tuple(None if g is None else g.cpu().numpy() for g in got)
                check(got, want, (l_max, normalized, n))


@pytest.mark.parametrize("name", ["cfg3", "cfg4", "cfg5"])
def test_size_independent_properties_at_full_size(library, name):
    """Identities that need no reference at all, evaluated on the device over the whole output:
    Unsold's sum rule, Euler homogeneity, harmonicity and symmetry of the Hessian."""
    w = WORKLOADS[name]
    announce("properties", name)
    xyz = torch.from_numpy(w.points()).cuda()
    status, (sph, dsph, ddsph) = run_launch_layer(library, xyz, w.l_max, w.normalized, w.derivatives)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    l_top = min(w.l_max, 16)  # float32 loses the high-|m| prefactors beyond l ~ 18
    r = xyz.double().norm(dim=1)
    eps = 3e-4 if w.dtype == "f32" else 1e-10
    for l in range(l_top + 1):
        block = slice(l * l, (l + 1) ** 2)
        total = (sph[:, block].double() ** 2).sum(dim=1)
        want = (2 * l + 1) / (4 * np.pi) * (torch.ones_like(r) if w.normalized else r ** (2 * l))
        assert torch.allclose(total, want, rtol=eps * (l + 1), atol=0), (name, "sum rule", l)
        radial = torch.einsum("ia,iak->ik", xyz.double(), dsph[:, :, block].double())
        scale = (dsph[:, :, block].double().abs().amax(dim=(1, 2)) * r).clamp_min(1e-30)
        if w.normalized:
            assert ((radial.abs().amax(dim=1) / scale) < eps * (l + 1)).all(), (name, "r.grad = 0", l)
        else:
            diff = (radial - l * sph[:, block].double()).abs().amax(dim=1)
            assert ((diff / scale) < eps * (l + 1)).all(), (name, "r.grad = l", l)
    if ddsph is not None:
        assert torch.equal(ddsph, ddsph.transpose(1, 2))
        if not w.normalized:
            trace = (ddsph[:, 0, 0] + ddsph[:, 1, 1] + ddsph[:, 2, 2]).abs().amax(dim=1)
            top = ddsph.abs().amax(dim=(1, 2, 3))
            assert (trace <= 1e-9 * top).all(), (name, "harmonicity")


def test_finite_differences_through_the_device():
    """Same pattern as the reference's device-side derivative test
    (sphericart/tests/test_derivatives_sycl.cpp:262-312): analytic gradients and Hessians from the
    device against central differences of device values, float64, delta = 1e-4, tolerance 1e-4."""
    delta, tol = 1e-4, 1e-4
    rng = np.random.default_rng(8)
    xyz = rng.normal(size=(16, 3))
    xyz *= (rng.uniform(0.8, 1.5, size=16) / np.linalg.norm(xyz, axis=1))[:, None]
    for normalized in (True, False):
        for l_max in (1, 4, 6, 9, 14):
            announce("finite differences", normalized, l_max)
            _, dsph, ddsph = run_calculator(xyz, l_max, normalized, "hessians")
            gscale = 1e-2 * np.abs(dsph).max()
            hscale = 1e-2 * np.abs(ddsph).max() + 1e-9
            for a in range(3):
                step = np.zeros(3)
                step[a] = delta
                plus = run_calculator(xyz + step, l_max, normalized, "hessians")
                minus = run_calculator(xyz - step, l_max, normalized, "hessians")
                fd1 = (plus[0] - minus[0]) / (2 * delta)
                fd2 = (plus[1] - minus[1]) / (2 * delta)
                assert (np.abs(dsph[:, a] - fd1) <= tol * np.maximum(np.abs(fd1), gscale)).all()
                assert (np.abs(ddsph[:, a] - fd2) <= tol * np.maximum(np.abs(fd2), hscale)).all()
