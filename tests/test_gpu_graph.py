"""The launch layer under HIP graph capture: after one eager call per shape (tables uploaded,
kernel attributes set) the entry points only enqueue kernels, so a captured graph replays them."""

import numpy as np
import pytest
import torch

from gpu_utils import announce, run_launch_layer
from helpers import same_numbers, special_points

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("l_max,mode,dtype", [(6, "gradients", np.float32), (10, "values", np.float32),
                                              (9, "gradients", np.float64), (5, "hessians", np.float32)])
def test_forward_replays_from_a_graph(oracle, library, l_max, mode, dtype):
    rng = np.random.default_rng(3)
    n = 3000
    clouds = [special_points(dtype, rng, n) for _ in range(3)]
    static_xyz = torch.from_numpy(clouds[0]).cuda()
    announce("graph", l_max, mode, np.dtype(dtype).name)
    # eager first: device tables, kernel attributes
    status, out = run_launch_layer(library, static_xyz, l_max, True, mode)
    assert status == 0, library.sphx_last_error()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            status, _ = run_launch_layer(library, static_xyz, l_max, True, mode, out=out,
                                         stream=torch.cuda.current_stream().cuda_stream)
    assert status == 0, library.sphx_last_error()
    for xyz in clouds[::-1] + clouds:
        static_xyz.copy_(torch.from_numpy(xyz).cuda())
        for o in out:
            if o is not None:
                o.fill_(-3.0)  # eager work between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle.compute(xyz, l_max, True, mode)
        for o, w in zip(out, want):
            if w is not None:
                assert same_numbers(o.cpu().numpy(), w).all()
