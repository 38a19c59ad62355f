"""ctypes prototypes of the shared library.

Mirrors the device half of the reference's loader
(python/src/sphericart/_c_lib.py:240-400): the same twenty
``sphericart_cuda_*`` symbols with the same argument lists, plus the plain
launch layer of ``include/sphx_launch.h``.
"""

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libsphericart_amd.so")

_library = None

C_API_SYMBOLS = [
    f"sphericart_cuda_{kind}_harmonics_{name}{suffix}"
    for kind in ("spherical", "solid")
    for name in ("new", "delete", "compute_array", "compute_array_with_gradients", "compute_array_with_hessians")
    for suffix in ("", "_f")
]

LAUNCH_SYMBOLS = [
    "sphx_forward_f32",
    "sphx_forward_f64",
    "sphx_backward_f32",
    "sphx_backward_f64",
    "sphx_backward_second_f32",
    "sphx_backward_second_f64",
    "sphx_vjp_f32",
    "sphx_vjp_f64",
    "sphx_forward_f32_via_f64",
    "sphx_forward_f32_via_f64_workspace",
    "sphx_forward_f32_via_f64_static",
    "sphx_forward_f32_via_f64_static_capacity",
    "sphx_prefactors_f32",
    "sphx_prefactors_f64",
    "sphx_device_count",
    "sphx_last_error",
    "sphx_plan",
    "sphx_describe_plan",
    "sphx_set_switch",
    "sphx_reset_switches",
    "sphx_probe_empty_launch",
    "sphx_probe_fill",
    "sphx_probe_host_cost_f64",
]


def _declare(lib):
    c_void_p, c_size_t, c_int = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int
    for kind in ("spherical", "solid"):
        for suffix in ("", "_f"):
            prefix = f"sphericart_cuda_{kind}_harmonics"
            new = getattr(lib, f"{prefix}_new{suffix}")
            new.restype = c_void_p
            new.argtypes = [c_size_t]
            delete = getattr(lib, f"{prefix}_delete{suffix}")
            delete.restype = None
            delete.argtypes = [c_void_p]
            fn = getattr(lib, f"{prefix}_compute_array{suffix}")
            fn.restype = None
            fn.argtypes = [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p]
            fn = getattr(lib, f"{prefix}_compute_array_with_gradients{suffix}")
            fn.restype = None
            fn.argtypes = [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p]
            fn = getattr(lib, f"{prefix}_compute_array_with_hessians{suffix}")
            fn.restype = None
            fn.argtypes = [c_void_p, c_void_p, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]
    for suffix in ("f32", "f64"):
        fn = getattr(lib, f"sphx_forward_{suffix}")
        fn.restype = c_int
        fn.argtypes = [c_void_p, c_size_t, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]
        for name in ("sphx_backward", "sphx_backward_second"):
            fn = getattr(lib, f"{name}_{suffix}")
            fn.restype = c_int
            fn.argtypes = [c_void_p, c_void_p, c_size_t, c_int, c_void_p, c_int, c_void_p]
        fn = getattr(lib, f"sphx_vjp_{suffix}")
        fn.restype = c_int
        fn.argtypes = [c_void_p, c_void_p, c_size_t, c_int, c_int, c_void_p, c_int, c_void_p]
        fn = getattr(lib, f"sphx_prefactors_{suffix}")
        fn.restype = c_int
        fn.argtypes = [c_int, c_void_p]
    lib.sphx_forward_f32_via_f64.restype = c_int
    lib.sphx_forward_f32_via_f64.argtypes = [
        c_void_p, c_size_t, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]
    lib.sphx_forward_f32_via_f64_workspace.restype = c_size_t
    lib.sphx_forward_f32_via_f64_workspace.argtypes = [c_size_t, c_int, c_int]
    lib.sphx_forward_f32_via_f64_static.restype = c_int
    lib.sphx_forward_f32_via_f64_static.argtypes = [
        c_void_p, c_size_t, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]
    lib.sphx_forward_f32_via_f64_static_capacity.restype = c_size_t
    lib.sphx_forward_f32_via_f64_static_capacity.argtypes = [c_int, c_int]
    lib.sphx_describe_plan.restype = c_int
    lib.sphx_describe_plan.argtypes = [c_size_t, c_int, c_int, c_int, c_int, ctypes.c_char_p, c_size_t]
    lib.sphx_set_switch.restype = c_int
    lib.sphx_set_switch.argtypes = [ctypes.c_char_p, c_int]
    lib.sphx_reset_switches.restype = None
    lib.sphx_reset_switches.argtypes = []
    lib.sphx_device_count.restype = c_int
    lib.sphx_device_count.argtypes = []
    lib.sphx_last_error.restype = ctypes.c_char_p
    lib.sphx_last_error.argtypes = []
    lib.sphx_plan.restype = c_int
    lib.sphx_plan.argtypes = [c_size_t, c_int, c_int, c_int] + [ctypes.POINTER(c_int)] * 4
    lib.sphx_probe_empty_launch.restype = c_int
    lib.sphx_probe_empty_launch.argtypes = [c_void_p]
    lib.sphx_probe_fill.restype = c_int
    lib.sphx_probe_fill.argtypes = [c_void_p, c_size_t, c_void_p]
    lib.sphx_probe_host_cost_f64.restype = c_int
    lib.sphx_probe_host_cost_f64.argtypes = [c_int, c_void_p, c_size_t, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                             ctypes.POINTER(ctypes.c_double)]


def get_library():
    """Load ``libsphericart_amd.so``; there is no fallback when it is missing."""
    global _library
    if _library is None:
        if not os.path.exists(LIBRARY_PATH):
            raise RuntimeError(
                f"{LIBRARY_PATH} is missing: build it with `python -m sphericart_amd.build` "
                "(sphericart_amd has no CPU or pure-Python evaluation path)"
            )
        lib = ctypes.CDLL(LIBRARY_PATH)
        _declare(lib)
        _library = lib
    return _library
