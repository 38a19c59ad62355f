"""Seeded random shapes through the launch layer against the oracle, number for number.

Each case draws precision, class, derivative order, l_max, the number of points, how far the
outputs are shifted inside their allocations (NaN guard bands on both sides) and, for two cases
in three, one planner override (so that kernels and tile sizes the planner would not pick for
the shape are exercised as well). The run stops at its first failure.
"""

import numpy as np
import pytest
import torch

from gpu_utils import announce
from helpers import same_numbers, special_points

pytestmark = pytest.mark.gpu

MODES = ("values", "gradients", "hessians")
L_MAX_CAP = (40, 36, 24)
OVERRIDES = (
    None, None, None,
    ("SPHX_GRADIENT_LANES", (0,)), ("SPHX_HESSIAN_LANES", (0, 2)), ("SPHX_VALUES_LDS", (1,)),
    ("SPHX_JOB_LIST", (0, 1, 2)), ("SPHX_PREFIX_INSIDE", (0,)), ("SPHX_TILE", (1, 2, 3, 5, 7, 8)),
    ("SPHX_SEQUENCE_WAVES", (1, 2, 3, 4)), ("SPHX_CHUNK_SHIFT", (0, 1, 2, 3)),
    ("SPHX_AZ_SHIFT", (0, 1, 2, 3)), ("SPHX_SPLIT_SIDES", (0,)), ("SPHX_TILE_POW2", (1,)),
    ("SPHX_SPLIT_BELOW", (0, 64)), ("SPHX_GRADIENT_LANES_PARTS", (1, 2)), ("SPHX_GROUP_THREADS", (512, 1024)),
    ("SPHX_GROUP_THREADS", (1024,)), ("SPHX_SPREAD_KINDS", (0, 1)), ("SPHX_SLICE_WAVES", (0, 1, 2, 3)),
    ("SPHX_VALUES_TILE_STEP", (0, 1, 2, 8)), ("SPHX_VALUES_MIN_TILE", (8, 16, 48)),
    ("SPHX_VALUES_PACK", (1, 2, 4)), ("SPHX_VALUES_ALONE", (0, 1)),
    ("SPHX_WAVE_PRIORITIES", (1, 2, 3)),
)


def draw(rng):
    mode = int(rng.integers(0, 3))
    dtype = np.float32 if rng.random() < 0.5 else np.float64
    l_max = int(rng.integers(0, L_MAX_CAP[mode] + 1))
    normalized = bool(rng.integers(0, 2))
    n = int(rng.choice([1, 2, 5, 31, 64, 65, 100, 333, 1000, 2049, 4100, int(rng.integers(1, 60001))]))
    per_point = (l_max + 1) ** 2 * (1, 4, 13)[mode]
    while n > 1 and per_point * n > 2e7:
        n //= 2
    shift = int(rng.integers(0, 8))
    override = OVERRIDES[int(rng.integers(0, len(OVERRIDES)))]
    if override is not None:
        override = (override[0], int(rng.choice(override[1])))
    return mode, dtype, l_max, normalized, n, shift, override


def test_random_shapes_equal_the_oracle(oracle, library, switches):
    rng = np.random.default_rng(20240607)
    stream = torch.cuda.current_stream().cuda_stream
    for case in range(300):
        mode, dtype, l_max, normalized, n, shift, override = draw(rng)
        announce("fuzz", case, MODES[mode], np.dtype(dtype).name, "l_max", l_max, "normalized", normalized,
                 "n", n, "shift", shift, "override", override)
        library.sphx_reset_switches()
        if override is not None:
            switches(*override)
        xyz = special_points(dtype, rng, n)
        want = oracle.compute(xyz, l_max, normalized, MODES[mode])
        ny = (l_max + 1) ** 2
        tdtype = torch.float32 if dtype == np.float32 else torch.float64
        sizes = (n * ny, 3 * n * ny, 9 * n * ny)
        shapes = ((n, ny), (n, 3, ny), (n, 3, 3, ny))
        raw = [torch.full((sizes[i] + 16,), float("nan"), dtype=tdtype, device="cuda") if i <= mode else None
               for i in range(3)]
        out = [raw[i][shift:shift + sizes[i]].view(shapes[i]) if i <= mode else None for i in range(3)]
        forward = library.sphx_forward_f32 if dtype == np.float32 else library.sphx_forward_f64
        xyz_dev = torch.from_numpy(xyz).cuda()
        status = forward(xyz_dev.data_ptr(), n, l_max, int(normalized), mode, out[0].data_ptr(),
                         out[1].data_ptr() if out[1] is not None else None,
                         out[2].data_ptr() if out[2] is not None else None, stream)
        assert status == 0, (case, library.sphx_last_error())
        torch.cuda.synchronize()
        for i in range(mode + 1):
            same = same_numbers(out[i].cpu().numpy(), want[i])
            assert same.all(), (case, "array", i, "differing numbers", int((~same).sum()))
            assert torch.isnan(raw[i][:shift]).all() and torch.isnan(raw[i][shift + sizes[i]:]).all(), \
                (case, "array", i, "written outside its bounds")
