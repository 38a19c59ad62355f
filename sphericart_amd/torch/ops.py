"""Torch operators over the HIP library, with the reference's autograd rules.

The reference registers six operators in the ``sphericart_torch`` namespace
(sphericart-torch/src/torch.cpp:367-385) and gives them autograd, fake-tensor
and vmap rules from Python (sphericart-torch/python/sphericart/torch/register.py:60-185).
The same six live here in the ``sphericart_amd`` namespace with the same
schemas; their device implementation calls ``sphx_forward_*`` on the tensor's
current stream, from C++ where ``libsphericart_amd_torch.so`` has been built
(csrc/sphx_torch.cpp), otherwise from the functions below over ctypes. Only the
GPU key has an implementation: CPU tensors raise.
Unless the reference's own extension already owns it, the ``sphericart_torch``
namespace is defined as well, with the reference's eight schemas (the six
operators and the two ``*_omp_num_threads``), each forwarding to its
``sphericart_amd`` twin: code, scripted modules included, that names
``torch.ops.sphericart_torch.*`` resolves against this library.

The backward formulas are the reference's (register.py:82-175). Where it writes
the vector-Jacobian products as ``torch.sum(grad.unsqueeze(1) * dsph, dim=2)``,
two more operators, ``contract_gradients`` and ``contract_hessians``, do the
same sums in one pass over ``dsph`` / ``ddsph`` (``sphx_backward_*``) without
the product array. The backward pass of the value operators does not build
``dsph`` at all: ``*_vjp`` (``sphx_vjp_*``) evaluates the gradients on the chip
and contracts them on the fly. All of these are differentiable themselves, so
double backward works as it does in the reference.
"""

import ctypes
import os

import torch

from .._c_lib import LIBRARY_PATH, get_library

NAMESPACE = "sphericart_amd"
_MODES = {"": 0, "_with_gradients": 1, "_with_hessians": 2}

# The schemas and the device implementations live in C++ (csrc/sphx_torch.cpp ->
# libsphericart_amd_torch.so, built next to the HIP library) where that library has been built: a call
# then costs the host the dispatcher, its outputs and one C call. Without it, or with
# SPHERICART_AMD_PYTHON_OPERATORS=1, the same operators are defined here and implemented over ctypes;
# either way the work is done by the same entry points of libsphericart_amd.so.
TORCH_LIBRARY_PATH = os.path.join(os.path.dirname(LIBRARY_PATH), "libsphericart_amd_torch.so")


def _load_cpp_operators():
    if os.environ.get("SPHERICART_AMD_PYTHON_OPERATORS", "0") not in ("", "0"):
        return False
    if not os.path.exists(TORCH_LIBRARY_PATH):
        return False
    get_library()  # fails loudly when the HIP library itself is missing
    torch.ops.load_library(TORCH_LIBRARY_PATH)
    return True


cpp_operators = _load_cpp_operators()
_lib = torch.library.Library(NAMESPACE, "FRAGMENT" if cpp_operators else "DEF")
if not cpp_operators:
    for _prefix in ("spherical_harmonics", "solid_harmonics"):
        _lib.define(f"{_prefix}(Tensor xyz, int l_max) -> Tensor")
        _lib.define(f"{_prefix}_with_gradients(Tensor xyz, int l_max) -> (Tensor, Tensor)")
        _lib.define(f"{_prefix}_with_hessians(Tensor xyz, int l_max) -> (Tensor, Tensor, Tensor)")
        _lib.define(f"{_prefix}_vjp(Tensor xyz, Tensor sph_grad, int l_max) -> Tensor")
    _lib.define("contract_gradients(Tensor dsph, Tensor sph_grad) -> Tensor")
    _lib.define("contract_hessians(Tensor ddsph, Tensor dsph_grad) -> Tensor")


def _suffix(tensor):
    if tensor.dtype == torch.float32:
        return "f32"
    if tensor.dtype == torch.float64:
        return "f64"
    raise TypeError(f"spherical harmonics are implemented for float32 and float64, not {tensor.dtype}")


def _check(status, library):
    if status != 0:
        raise RuntimeError(library.sphx_last_error().decode())


def _pointer(tensor):
    return ctypes.c_void_p(tensor.data_ptr()) if tensor is not None and tensor.numel() > 0 else None


def _forward(xyz, l_max, normalized, mode):
    """Counterpart of compute_raw / _compute_raw_cuda (sphericart-torch/src/torch.cpp:126-146,238-294)."""
    if xyz.dim() != 2 or xyz.shape[1] != 3:
        raise ValueError("xyz tensor must be a 2D array with shape `n_samples x 3`")
    if l_max < 0:
        raise ValueError("l_max must be non-negative")
    suffix = _suffix(xyz)
    xyz = xyz.detach().contiguous()
    n, ny = xyz.shape[0], (l_max + 1) ** 2
    sph = torch.empty((n, ny), dtype=xyz.dtype, device=xyz.device)
    dsph = torch.empty((n, 3, ny), dtype=xyz.dtype, device=xyz.device) if mode >= 1 else None
    ddsph = torch.empty((n, 3, 3, ny), dtype=xyz.dtype, device=xyz.device) if mode >= 2 else None
    library = get_library()
    with torch.cuda.device(xyz.device):
        stream = torch.cuda.current_stream(xyz.device).cuda_stream
        status = getattr(library, f"sphx_forward_{suffix}")(
            _pointer(xyz), n, l_max, int(normalized), mode,
            _pointer(sph), _pointer(dsph), _pointer(ddsph), ctypes.c_void_p(stream),
        )
    _check(status, library)
    return sph, dsph, ddsph


def _contract(name, derivatives, upstream):
    suffix = _suffix(derivatives)
    if upstream.dtype != derivatives.dtype or upstream.device != derivatives.device:
        raise ValueError("the two tensors of a contraction must share dtype and device")
    if derivatives.shape[:-1] != upstream.shape[:1] + derivatives.shape[1:-1] or (
        upstream.shape != derivatives.shape[:1] + derivatives.shape[2:]
    ):
        raise ValueError(f"shapes {tuple(derivatives.shape)} and {tuple(upstream.shape)} do not contract")
    derivatives = derivatives.detach().contiguous()
    upstream = upstream.detach().contiguous()
    n, n_total = derivatives.shape[0], derivatives.shape[-1]
    out = torch.empty((n, 3), dtype=derivatives.dtype, device=derivatives.device)
    library = get_library()
    with torch.cuda.device(derivatives.device):
        stream = torch.cuda.current_stream(derivatives.device).cuda_stream
        status = getattr(library, f"{name}_{suffix}")(
            _pointer(derivatives), _pointer(upstream), n, n_total, _pointer(out), 0,
            ctypes.c_void_p(stream),
        )
    _check(status, library)
    return out


def _vjp(xyz, sph_grad, l_max, normalized):
    suffix = _suffix(xyz)
    if sph_grad.dtype != xyz.dtype or sph_grad.device != xyz.device:
        raise ValueError("xyz and sph_grad must share dtype and device")
    if sph_grad.shape != (xyz.shape[0], (l_max + 1) ** 2):
        raise ValueError(f"sph_grad must have shape {(xyz.shape[0], (l_max + 1) ** 2)}")
    xyz = xyz.detach().contiguous()
    sph_grad = sph_grad.detach().contiguous()
    out = torch.empty_like(xyz)
    library = get_library()
    with torch.cuda.device(xyz.device):
        stream = torch.cuda.current_stream(xyz.device).cuda_stream
        status = getattr(library, f"sphx_vjp_{suffix}")(
            _pointer(xyz), _pointer(sph_grad), xyz.shape[0], l_max, int(normalized), _pointer(out), 0,
            ctypes.c_void_p(stream),
        )
    _check(status, library)
    return out


def _no_cpu(*args, **kwargs):
    raise RuntimeError(
        "sphericart_amd evaluates on AMD GPUs only: move the tensor to the device "
        "(there is no CPU implementation behind these operators)"
    )


def _register_forward(prefix, normalized):
    def value(xyz, l_max):
        return _forward(xyz, l_max, normalized, 0)[0]

    def gradients(xyz, l_max):
        return _forward(xyz, l_max, normalized, 1)[:2]

    def hessians(xyz, l_max):
        return _forward(xyz, l_max, normalized, 2)

    def vjp(xyz, sph_grad, l_max):
        return _vjp(xyz, sph_grad, l_max, normalized)

    for name, fn in ((prefix, value), (f"{prefix}_with_gradients", gradients),
                     (f"{prefix}_with_hessians", hessians), (f"{prefix}_vjp", vjp)):
        _lib.impl(name, fn, "CUDA")
        _lib.impl(name, _no_cpu, "CPU")


if not cpp_operators:
    _register_forward("spherical_harmonics", True)
    _register_forward("solid_harmonics", False)
    _lib.impl("contract_gradients", lambda d, g: _contract("sphx_backward", d, g), "CUDA")
    _lib.impl("contract_hessians", lambda d, g: _contract("sphx_backward_second", d, g), "CUDA")
    _lib.impl("contract_gradients", _no_cpu, "CPU")
    _lib.impl("contract_hessians", _no_cpu, "CPU")

_ops = getattr(torch.ops, NAMESPACE)


# ---- shapes for fake tensors (register.py:60-69) -----------------------------

def _register_fake(name, outputs):
    @torch.library.register_fake(f"{NAMESPACE}::{name}")
    def fake(xyz, l_max):
        sph = xyz.new_empty((xyz.shape[0], (l_max + 1) ** 2))
        if outputs == 1:
            return sph
        dsph = xyz.new_empty((xyz.shape[0], 3, sph.shape[1]))
        if outputs == 2:
            return sph, dsph
        return sph, dsph, xyz.new_empty((xyz.shape[0], 3, 3, sph.shape[1]))


@torch.library.register_fake(f"{NAMESPACE}::contract_gradients")
def _fake_contract_gradients(dsph, sph_grad):
    return dsph.new_empty((dsph.shape[0], 3))


@torch.library.register_fake(f"{NAMESPACE}::contract_hessians")
def _fake_contract_hessians(ddsph, dsph_grad):
    return ddsph.new_empty((ddsph.shape[0], 3))


# ---- autograd of the contractions (plain torch: only double backward gets here) ----

def _contract_gradients_backward(ctx, grad):
    dsph, sph_grad = ctx.saved_tensors
    d_dsph = d_sph_grad = None
    if ctx.needs_input_grad[0]:
        d_dsph = grad.unsqueeze(2) * sph_grad.unsqueeze(1)
    if ctx.needs_input_grad[1]:
        d_sph_grad = torch.sum(grad.unsqueeze(2) * dsph, dim=1)
    return d_dsph, d_sph_grad


def _contract_hessians_backward(ctx, grad):
    ddsph, dsph_grad = ctx.saved_tensors
    d_ddsph = d_dsph_grad = None
    if ctx.needs_input_grad[0]:
        # out[i, b] = sum_{a, k} ddsph[i, a, b, k] * dsph_grad[i, a, k]
        d_ddsph = grad.unsqueeze(1).unsqueeze(3) * dsph_grad.unsqueeze(2)
    if ctx.needs_input_grad[1]:
        d_dsph_grad = torch.sum(grad.unsqueeze(1).unsqueeze(3) * ddsph, dim=2)
    return d_ddsph, d_dsph_grad


def _save_inputs(ctx, inputs, output):
    ctx.save_for_backward(*inputs)


torch.library.register_autograd(
    f"{NAMESPACE}::contract_gradients", _contract_gradients_backward, setup_context=_save_inputs
)
torch.library.register_autograd(
    f"{NAMESPACE}::contract_hessians", _contract_hessians_backward, setup_context=_save_inputs
)


# ---- autograd of the six operators (register.py:82-175) ----------------------

def _register_vjp(prefix):
    """Shapes and derivatives of the fused product xyz_grad[i, a] = sum_k dsph[i, a, k] w[i, k]."""
    hessians = getattr(_ops, f"{prefix}_with_hessians")

    @torch.library.register_fake(f"{NAMESPACE}::{prefix}_vjp")
    def fake(xyz, sph_grad, l_max):
        return xyz.new_empty((xyz.shape[0], 3))

    def setup_context(ctx, inputs, output):
        xyz, sph_grad, ctx.l_max = inputs
        ctx.save_for_backward(xyz, sph_grad)

    def backward(ctx, grad):
        xyz, sph_grad = ctx.saved_tensors
        _, dsph, ddsph = hessians(xyz, ctx.l_max)
        d_xyz = d_sph_grad = None
        if ctx.needs_input_grad[0]:
            # d/d xyz[i, b]: sum_{a, k} grad[i, a] w[i, k] ddsph[i, a, b, k]
            d_xyz = _ops.contract_hessians(ddsph, grad.unsqueeze(2) * sph_grad.unsqueeze(1))
        if ctx.needs_input_grad[1]:
            d_sph_grad = torch.sum(grad.unsqueeze(2) * dsph, dim=1)
        return d_xyz, d_sph_grad, None

    torch.library.register_autograd(f"{NAMESPACE}::{prefix}_vjp", backward, setup_context=setup_context)


def _register_value_autograd(prefix):
    vjp = getattr(_ops, f"{prefix}_vjp")

    def setup_context(ctx, inputs, output):
        xyz, ctx.l_max = inputs
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(xyz)

    def backward(ctx, grad_sph):
        if not ctx.needs_input_grad[0] or grad_sph is None:
            return None, None
        (xyz,) = ctx.saved_tensors
        return vjp(xyz, grad_sph, ctx.l_max), None

    torch.library.register_autograd(f"{NAMESPACE}::{prefix}", backward, setup_context=setup_context)


def _register_gradients_autograd(prefix):
    hessians = getattr(_ops, f"{prefix}_with_hessians")

    def setup_context(ctx, inputs, output):
        xyz, ctx.l_max = inputs
        ctx.set_materialize_grads(False)  # outputs that were not used arrive as None
        ctx.save_for_backward(xyz, output[1])

    def backward(ctx, grad_sph, grad_dsph):
        if not ctx.needs_input_grad[0]:
            return None, None
        xyz, dsph = ctx.saved_tensors
        xyz_grad = None
        if grad_sph is not None:
            xyz_grad = _ops.contract_gradients(dsph, grad_sph)
        if grad_dsph is not None:
            ddsph = hessians(xyz, ctx.l_max)[2]
            extra = _ops.contract_hessians(ddsph, grad_dsph)
            xyz_grad = extra if xyz_grad is None else xyz_grad + extra
        return xyz_grad, None

    torch.library.register_autograd(
        f"{NAMESPACE}::{prefix}_with_gradients", backward, setup_context=setup_context
    )


def _register_hessians_autograd(prefix):
    def setup_context(ctx, inputs, output):
        ctx.set_materialize_grads(False)
        ctx.save_for_backward(output[1], output[2])

    def backward(ctx, grad_sph, grad_dsph, grad_ddsph):
        if grad_ddsph is not None:
            raise RuntimeError(
                "Third derivatives of the spherical harmonics with respect to "
                "the Cartesian coordinates are not supported."
            )
        dsph, ddsph = ctx.saved_tensors
        xyz_grad = None
        if grad_sph is not None:
            xyz_grad = _ops.contract_gradients(dsph, grad_sph)
        if grad_dsph is not None:
            extra = _ops.contract_hessians(ddsph, grad_dsph)
            xyz_grad = extra if xyz_grad is None else xyz_grad + extra
        return xyz_grad, None

    torch.library.register_autograd(
        f"{NAMESPACE}::{prefix}_with_hessians", backward, setup_context=setup_context
    )


def _register_vmap(name, out_dims):
    """Batching rule (register.py:72-79): the batch axis is folded into the sample axis."""
    op = getattr(_ops, name)

    def rule(info, in_dims, xyz, l_max):
        if in_dims[0] is None:
            return op(xyz, l_max), None if isinstance(out_dims, int) else (None,) * len(out_dims)
        xyz = xyz.movedim(in_dims[0], 0)
        if xyz.dim() == 2:  # a batch of single points
            return op(xyz, l_max), out_dims
        batch, n = xyz.shape[0], xyz.shape[1]
        flat = op(xyz.reshape(batch * n, 3), l_max)
        if isinstance(flat, torch.Tensor):
            return flat.reshape(batch, n, *flat.shape[1:]), out_dims
        return tuple(t.reshape(batch, n, *t.shape[1:]) for t in flat), out_dims

    torch.library.register_vmap(f"{NAMESPACE}::{name}", rule)


for _prefix in ("spherical_harmonics", "solid_harmonics"):
    _register_fake(_prefix, 1)
    _register_fake(f"{_prefix}_with_gradients", 2)
    _register_fake(f"{_prefix}_with_hessians", 3)
    _register_vjp(_prefix)
    _register_value_autograd(_prefix)
    _register_gradients_autograd(_prefix)
    _register_hessians_autograd(_prefix)
    _register_vmap(_prefix, 0)
    _register_vmap(f"{_prefix}_with_gradients", (0, 0))
    _register_vmap(f"{_prefix}_with_hessians", (0, 0, 0))


# ---- the reference's namespace (sphericart-torch/src/torch.cpp:367-385) ---------------------
#
# Aliases: every operator forwards to its twin above through a composite implementation, so the
# autograd, fake-tensor and vmap rules registered there apply unchanged. The two
# *_omp_num_threads operators report 1: there is no host evaluator and no OpenMP team behind
# these operators. Skipped when the namespace is taken (the reference's extension is loaded).

REFERENCE_NAMESPACE = "sphericart_torch"
reference_namespace_defined = False


def _define_reference_namespace():
    global _reference_lib, reference_namespace_defined
    if cpp_operators:
        # libsphericart_amd_torch.so defined it when it was loaded, unless the namespace was taken
        reference_namespace_defined = bool(_ops.owns_reference_namespace())
        return
    try:
        _reference_lib = torch.library.Library(REFERENCE_NAMESPACE, "DEF")
    except RuntimeError:
        return  # another library owns the namespace
    for prefix in ("spherical_harmonics", "solid_harmonics"):
        _reference_lib.define(f"{prefix}(Tensor xyz, int l_max) -> Tensor")
        _reference_lib.define(f"{prefix}_with_gradients(Tensor xyz, int l_max) -> (Tensor, Tensor)")
        _reference_lib.define(f"{prefix}_with_hessians(Tensor xyz, int l_max) -> (Tensor, Tensor, Tensor)")
        _reference_lib.define(f"{prefix}_omp_num_threads(int l_max) -> int")
        for suffix in ("", "_with_gradients", "_with_hessians"):
            twin = getattr(_ops, prefix + suffix)
            _reference_lib.impl(prefix + suffix, (lambda op: lambda xyz, l_max: op(xyz, l_max))(twin),
                                "CompositeImplicitAutograd")
        _reference_lib.impl(f"{prefix}_omp_num_threads", lambda l_max: 1, "CompositeExplicitAutograd")
    reference_namespace_defined = True


_define_reference_namespace()
