"""``sphx_forward_f32_via_f64_static``: the variant of ``sphx_forward_f32_via_f64`` for callers that cannot
allocate device memory. Within the closed forms (l_max <= 6, or <= 1 with second derivatives) it stages its
float64 rows in the library's own scratch array instead of a workspace; beyond, it is the same single launch. Checked number for number against the existing entry point (which
``tests/test_gpu_via_float64.py`` pins against the rounded float64 oracle) on consecutive calls
that share the scratch, the later ones smaller, and against the oracle directly.
"""

import numpy as np
import pytest
import torch

from gpu_utils import MODE_INDEX, announce
from helpers import same_numbers, special_points

pytestmark = pytest.mark.gpu


def outputs(n, l_max, k):
    ny = (l_max + 1) ** 2
    opts = dict(dtype=torch.float32, device="cuda")
    return (
        torch.full((n, ny), -7.0, **opts),
        torch.full((n, 3, ny), -7.0, **opts) if k >= 1 else None,
        torch.full((n, 3, 3, ny), -7.0, **opts) if k >= 2 else None,
    )


def pointers(out):
    return [o.data_ptr() if o is not None else None for o in out]


def with_workspace(library, xyz_dev, l_max, normalized, mode):
    n, k = xyz_dev.shape[0], MODE_INDEX[mode]
    out = outputs(n, l_max, k)
    nbytes = library.sphx_forward_f32_via_f64_workspace(n, l_max, k)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    status = library.sphx_forward_f32_via_f64(
        xyz_dev.data_ptr(), n, l_max, int(normalized), k, *pointers(out), workspace.data_ptr(), nbytes,
        torch.cuda.current_stream().cuda_stream)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    return out


def without_allocation(library, xyz_dev, l_max, normalized, mode, out):
    n, k = xyz_dev.shape[0], MODE_INDEX[mode]
    status = library.sphx_forward_f32_via_f64_static(
        xyz_dev.data_ptr(), n, l_max, int(normalized), k, *pointers(out),
        torch.cuda.current_stream().cuda_stream)
    assert status == 0, library.sphx_last_error()


def test_consecutive_calls_share_the_scratch(oracle, library):
    """Calls in a row on one stream, each smaller or differently shaped than the one before, so
    that the scratch still holds the previous call's rows: every result equals the existing
    entry point's, number for number. The outputs are allocated before the calls; between the
    calls nothing is allocated and nothing waits."""
    rng = np.random.default_rng(77)
    cases = [(6, True, "gradients", 5000), (6, True, "gradients", 1201), (33, True, "gradients", 700),
             (33, False, "gradients", 64), (12, False, "hessians", 300), (1, True, "hessians", 3000),
             (1, False, "hessians", 100), (12, True, "hessians", 7), (40, True, "values", 2049),
             (5, True, "values", 4097), (3, False, "values", 1)]
    prepared = []
    for l_max, normalized, mode, n in cases:
        xyz = special_points(np.float32, rng, n)
        xyz_dev = torch.from_numpy(xyz).cuda()
        hard = 1 if mode == "hessians" else 6
        assert l_max > hard or n <= library.sphx_forward_f32_via_f64_static_capacity(l_max, MODE_INDEX[mode])
        prepared.append((xyz, xyz_dev, with_workspace(library, xyz_dev, l_max, normalized, mode),
                         outputs(n, l_max, MODE_INDEX[mode])))
    torch.cuda.synchronize()
    for (l_max, normalized, mode, n), (xyz, xyz_dev, want, got) in zip(cases, prepared):
        announce("static scratch", l_max, normalized, mode, n)
        without_allocation(library, xyz_dev, l_max, normalized, mode, got)
    torch.cuda.synchronize()
    for (l_max, normalized, mode, n), (xyz, xyz_dev, want, got) in zip(cases, prepared):
        reference = oracle.compute(xyz.astype(np.float64), l_max, normalized, mode)
        for g, w, r in zip(got, want, reference):
            if w is not None:
                assert same_numbers(g.cpu().numpy(), w.cpu().numpy()).all(), (l_max, mode, n)
                with np.errstate(over="ignore"):
                    assert same_numbers(g.cpu().numpy(), r.astype(np.float32)).all(), (l_max, mode, n)


def test_more_points_than_the_scratch_holds_are_refused(library):
    l_max, k = 6, 1
    capacity = library.sphx_forward_f32_via_f64_static_capacity(l_max, k)
    n = capacity + 1
    xyz_dev = torch.ones((n, 3), dtype=torch.float32, device="cuda")
    out = outputs(n, l_max, k)
    status = library.sphx_forward_f32_via_f64_static(
        xyz_dev.data_ptr(), n, l_max, 1, k, *pointers(out), torch.cuda.current_stream().cuda_stream)
    assert status == 2  # SPHX_ERR_UNSUPPORTED
    message = library.sphx_last_error().decode()
    assert "scratch" in message and str(capacity) in message
    torch.cuda.synchronize()
    assert (out[0] == -7.0).all()  # nothing was launched
    # exactly the capacity is accepted
    status = library.sphx_forward_f32_via_f64_static(
        xyz_dev.data_ptr(), capacity, l_max, 1, k, *pointers(out), torch.cuda.current_stream().cuda_stream)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    assert torch.isfinite(out[0][:capacity]).all() and (out[0][capacity:] == -7.0).all()


def test_beyond_the_closed_forms_no_scratch_is_needed(oracle, library):
    """More points than the scratch would hold, at an l_max that the one-launch kernel covers."""
    l_max, k = 20, 1
    n = library.sphx_forward_f32_via_f64_static_capacity(l_max, k) + 77
    xyz = special_points(np.float32, np.random.default_rng(78), n)
    xyz_dev = torch.from_numpy(xyz).cuda()
    got = outputs(n, l_max, k)
    without_allocation(library, xyz_dev, l_max, True, "gradients", got)
    torch.cuda.synchronize()
    reference = oracle.compute(xyz.astype(np.float64), l_max, True, "gradients")
    for g, r in zip(got[:2], reference[:2]):
        assert same_numbers(g.cpu().numpy(), r.astype(np.float32)).all()
