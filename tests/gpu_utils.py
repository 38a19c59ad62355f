"""Helpers of the GPU tests: run the library on torch device buffers through its C entry points."""

import numpy as np
import torch

import sphericart_amd

MODE_INDEX = {"values": 0, "gradients": 1, "hessians": 2}
METHOD = {"values": "compute", "gradients": "compute_with_gradients", "hessians": "compute_with_hessians"}


def announce(*what):
    """Name the case before touching the GPU, so that a fault can be traced to it."""
    print("[gpu case]", *what, flush=True)


def run_calculator(xyz, l_max, normalized, mode):
    """Through the Python calculators, i.e. the sphericart_cuda_* C API. Returns numpy arrays."""
    cls = sphericart_amd.SphericalHarmonics if normalized else sphericart_amd.SolidHarmonics
    calc = cls(l_max)
    device_xyz = torch.from_numpy(np.ascontiguousarray(xyz)).cuda()
    out = getattr(calc, METHOD[mode])(device_xyz)
    torch.cuda.synchronize()
    if mode == "values":
        out = (out,)
    out = tuple(o.cpu().numpy() for o in out)
    return out + (None,) * (3 - len(out))


def run_launch_layer(library, xyz_dev, l_max, normalized, mode, out=None, stream=None):
    """Through sphx_forward_* directly, on caller-provided device tensors."""
    n = xyz_dev.shape[0]
    ny = (l_max + 1) ** 2
    k = MODE_INDEX[mode]
    opts = dict(dtype=xyz_dev.dtype, device=xyz_dev.device)
    if out is None:
        out = (
            torch.empty((n, ny), **opts),
            torch.empty((n, 3, ny), **opts) if k >= 1 else None,
            torch.empty((n, 3, 3, ny), **opts) if k >= 2 else None,
        )
    fn = library.sphx_forward_f32 if xyz_dev.dtype == torch.float32 else library.sphx_forward_f64
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    status = fn(
        xyz_dev.data_ptr(), n, l_max, int(bool(normalized)), k,
        out[0].data_ptr(), out[1].data_ptr() if out[1] is not None else None,
        out[2].data_ptr() if out[2] is not None else None, stream,
    )
    return status, out
