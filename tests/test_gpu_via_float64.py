"""float32 arrays evaluated in float64 (``sphx_forward_f32_via_f64``), on the GPU.

The entry point has no counterpart in the reference. What pins it: the float64
oracle (itself pinned against the reference's vectors and its compiled CPU
code) evaluated on the widened points and rounded to float32 by numpy gives
the expected arrays number for number, since both the widening and the final
rounding are exact, correctly rounded conversions.
"""

import ctypes

import numpy as np
import pytest
import torch

import sphericart_amd
from gpu_utils import MODE_INDEX, METHOD, announce, run_launch_layer
from helpers import same_numbers, special_points

pytestmark = pytest.mark.gpu


def expected(oracle, xyz32, l_max, normalized, mode):
    want = oracle.compute(xyz32.astype(np.float64), l_max, normalized, mode)
    with np.errstate(over="ignore"):
        return tuple(None if w is None else w.astype(np.float32) for w in want)


def run_via_float64(library, xyz_dev, l_max, normalized, mode, workspace_bytes):
    n, ny, k = xyz_dev.shape[0], (l_max + 1) ** 2, MODE_INDEX[mode]
    opts = dict(dtype=torch.float32, device="cuda")
    out = (
        torch.full((n, ny), -7.0, **opts),
        torch.full((n, 3, ny), -7.0, **opts) if k >= 1 else None,
        torch.full((n, 3, 3, ny), -7.0, **opts) if k >= 2 else None,
    )
    workspace = None
    if workspace_bytes is not None:
        workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device="cuda")
    status = library.sphx_forward_f32_via_f64(
        xyz_dev.data_ptr(), n, l_max, int(bool(normalized)), k,
        out[0].data_ptr(), out[1].data_ptr() if out[1] is not None else None,
        out[2].data_ptr() if out[2] is not None else None,
        workspace.data_ptr() if workspace is not None else None,
        workspace_bytes or 0, torch.cuda.current_stream().cuda_stream,
    )
    torch.cuda.synchronize()
    return status, out


@pytest.mark.parametrize("l_max,mode", [(3, "hessians"), (6, "gradients"), (8, "gradients"), (12, "hessians"),
                                        (20, "values"), (33, "gradients"), (40, "values")])
@pytest.mark.parametrize("normalized", [True, False])
def test_equals_the_rounded_float64_oracle(oracle, library, l_max, mode, normalized):
    rng = np.random.default_rng(l_max)
    n = 777
    xyz = special_points(np.float32, rng, n)
    want = expected(oracle, xyz, l_max, normalized, mode)
    xyz_dev = torch.from_numpy(xyz).cuda()
    per_point = library.sphx_forward_f32_via_f64_workspace(1, l_max, MODE_INDEX[mode])
    assert per_point == 8 * (3 + (l_max + 1) ** 2 * (1, 4, 13)[MODE_INDEX[mode]])
    # one chunk; chunks of 128 and of 100 points (the latter not a multiple of a tile); the
    # library's own workspace
    for workspace_bytes in (n * per_point, 128 * per_point + 5, 100 * per_point, None):
        announce("via float64", l_max, mode, normalized, workspace_bytes)
        status, got = run_via_float64(library, xyz_dev, l_max, normalized, mode, workspace_bytes)
        assert status == 0, library.sphx_last_error()
        for g, w in zip(got, want):
            if w is not None:
                assert same_numbers(g.cpu().numpy(), w).all(), workspace_bytes


@pytest.mark.parametrize("l_max,mode,n", [(7, "values", 20000), (9, "gradients", 6000), (2, "hessians", 9000),
                                          (8, "hessians", 3000), (14, "hessians", 900), (17, "gradients", 3001),
                                          (20, "gradients", 2500), (24, "values", 2000), (32, "gradients", 1200),
                                          (40, "values", 700), (24, "hessians", 150), (48, "gradients", 130)])
@pytest.mark.parametrize("normalized", [True, False])
def test_one_launch_beyond_the_closed_forms(library, l_max, mode, normalized, n):
    """Beyond the closed forms the recursion kernel itself computes in float64 and stages float
    rows. Checked against the float64 arrays of ``sphx_forward_f64`` for the widened points
    (pinned against the oracle in test_gpu_parity.py), rounded by torch: both conversions are
    exact or correctly rounded, so the numbers must be the same. Sizes: many tiles per
    workgroup, whole and cut rows, tiles of one point to dozens. The workspace handed in must
    come back untouched."""
    rng = np.random.default_rng(l_max * 3 + n)
    xyz = special_points(np.float32, rng, n)
    xyz_dev = torch.from_numpy(xyz).cuda()
    k, ny = MODE_INDEX[mode], (l_max + 1) ** 2
    announce("via float64 in one launch", l_max, mode, normalized, n)
    status, want = run_launch_layer(library, xyz_dev.double(), l_max, normalized, mode)
    assert status == 0, library.sphx_last_error()
    workspace_bytes = 4096
    workspace = torch.full((workspace_bytes,), 0xAB, dtype=torch.uint8, device="cuda")
    opts = dict(dtype=torch.float32, device="cuda")
    got = (
        torch.full((n, ny), -7.0, **opts),
        torch.full((n, 3, ny), -7.0, **opts) if k >= 1 else None,
        torch.full((n, 3, 3, ny), -7.0, **opts) if k >= 2 else None,
    )
    status = library.sphx_forward_f32_via_f64(
        xyz_dev.data_ptr(), n, l_max, int(bool(normalized)), k, got[0].data_ptr(),
        got[1].data_ptr() if got[1] is not None else None, got[2].data_ptr() if got[2] is not None else None,
        workspace.data_ptr(), workspace_bytes, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert status == 0, library.sphx_last_error()
    assert bool((workspace == 0xAB).all())
    for g, w in zip(got, want):
        if g is not None:
            assert same_numbers(g.cpu().numpy(), w.to(torch.float32).cpu().numpy()).all()


def test_finite_where_float32_arithmetic_is_not(oracle, library):
    """l_max = 40, points on the unit sphere: the float32 kernels (and the reference) give NaN
    from l = 29 on, the float64 evaluation gives numbers of order one."""
    rng = np.random.default_rng(5)
    xyz = rng.normal(size=(500, 3))
    xyz = (xyz / np.linalg.norm(xyz, axis=1, keepdims=True)).astype(np.float32)
    xyz_dev = torch.from_numpy(xyz).cuda()
    announce("via float64 finite", 40)
    status, plain = run_launch_layer(library, xyz_dev, 40, True, "gradients")
    torch.cuda.synchronize()
    assert status == 0
    assert not torch.isfinite(plain[0][:, 29 * 29:]).all()
    status, got = run_via_float64(library, xyz_dev, 40, True, "gradients", None)
    assert status == 0
    assert torch.isfinite(got[0]).all() and torch.isfinite(got[1]).all()
    # sum over m of Y_l^m squared is (2l + 1) / (4 pi) on the unit sphere (addition theorem)
    sph = got[0].double().cpu().numpy()
    for l in (0, 7, 29, 40):
        total = (sph[:, l * l:(l + 1) * (l + 1)] ** 2).sum(axis=1)
        np.testing.assert_allclose(total, (2 * l + 1) / (4 * np.pi), rtol=2e-5)


def test_python_keyword(oracle):
    rng = np.random.default_rng(11)
    xyz = special_points(np.float32, rng, 300)
    xyz_dev = torch.from_numpy(xyz).cuda()
    for cls, normalized in ((sphericart_amd.SphericalHarmonics, True), (sphericart_amd.SolidHarmonics, False)):
        for mode in ("values", "gradients", "hessians"):
            announce("via float64 python", cls.__name__, mode)
            calc = cls(10, float32_via_float64=True)
            got = getattr(calc, METHOD[mode])(xyz_dev)
            got = (got,) if mode == "values" else got
            want = expected(oracle, xyz, 10, normalized, mode)
            for g, w in zip(got, want):
                assert g.dtype == torch.float32
                assert same_numbers(g.cpu().numpy(), w).all()
            # float64 input is not affected by the keyword
            got64 = calc.compute(xyz_dev.double())
            want64 = oracle.compute(xyz.astype(np.float64), 10, normalized, "values")[0]
            assert same_numbers(got64.cpu().numpy(), want64).all()


def test_errors(library):
    xyz = torch.randn(10, 3, device="cuda")
    sph = torch.empty(10, 16, device="cuda")
    small = torch.empty(64, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    announce("via float64 errors")
    status = library.sphx_forward_f32_via_f64(
        xyz.data_ptr(), 10, 3, 1, 0, sph.data_ptr(), None, None, small.data_ptr(), 64, stream)
    assert status != 0 and b"workspace" in library.sphx_last_error()
    status = library.sphx_forward_f32_via_f64(
        xyz.data_ptr(), 10, 3, 1, 1, sph.data_ptr(), None, None, None, 0, stream)
    assert status != 0 and b"dsph" in library.sphx_last_error()
    status = library.sphx_forward_f32_via_f64(
        xyz.data_ptr(), 10, 65, 1, 0, sph.data_ptr(), None, None, None, 0, stream)
    assert status != 0
    assert library.sphx_forward_f32_via_f64_workspace(10, -1, 0) == 0
    assert library.sphx_forward_f32_via_f64(
        xyz.data_ptr(), 0, 3, 1, 0, sph.data_ptr(), None, None, None, 0, stream) == 0
    torch.cuda.synchronize()
