"""TEST INFRASTRUCTURE ONLY: ctypes access to the CPU checker libraries.

Importers allowed: the test-suite, the smoke check and the CPU-baseline leg of
the benchmark. The shipped package never imports this module.

Three flavours share one calling convention:

* ``"oracle"``  -- ``oracle/libsphx_oracle.so``, this repository's restatement
  of the reference CPU evaluator (``oracle/sphx_oracle.cpp``), built without
  FMA contraction;
* ``"ref"``     -- ``oracle/_ref/libsphx_ref.so``, the reference's own
  ``sphericart/src/sphericart.cpp`` compiled with the same strict flags;
* ``"ref_fma"`` -- ``oracle/_ref/libsphx_ref_fma.so``, the same reference source
  built the way its own build system does on an FMA machine (-O3, contraction).

The ``_ref`` files exist only where the reference checkout was present at build
time (or where prebuilt files were carried along); ``available()`` tells.
"""

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_PATHS = {
    "oracle": os.path.join(_HERE, "libsphx_oracle.so"),
    "ref": os.path.join(_HERE, "_ref", "libsphx_ref.so"),
    "ref_fma": os.path.join(_HERE, "_ref", "libsphx_ref_fma.so"),
}
_PREFIX = {"oracle": "sphx_oracle", "ref": "sphx_ref", "ref_fma": "sphx_ref"}
_LIBS = {}

MODES = {"values": 0, "gradients": 1, "hessians": 2}


def build(reference="/root/reference"):
    """Compile the checker libraries (``make -C oracle``)."""
    subprocess.run(
        ["make", "-C", _HERE, "all", f"REFERENCE={reference}"],
        check=True,
        stdout=subprocess.DEVNULL,
    )


def available(flavour="oracle"):
    return os.path.exists(_PATHS[flavour])


def _lib(flavour):
    if flavour in _LIBS:
        return _LIBS[flavour]
    path = _PATHS[flavour]
    if not os.path.exists(path):
        if flavour == "oracle":
            build()
        if not os.path.exists(path):
            raise FileNotFoundError(f"checker library not built: {path}")
    lib = ctypes.CDLL(path)
    pre = _PREFIX[flavour]
    for suffix, ct in (("f64", ctypes.c_double), ("f32", ctypes.c_float)):
        ptr = ctypes.POINTER(ct)
        fn = getattr(lib, f"{pre}_compute_{suffix}")
        fn.restype = ctypes.c_int
        fn.argtypes = [ptr, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ptr, ptr, ptr]
        fn = getattr(lib, f"{pre}_recursion_route_{suffix}")
        fn.restype = ctypes.c_int
        fn.argtypes = [ptr, ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_int, ptr, ptr]
        fn = getattr(lib, f"{pre}_prefactors_{suffix}")
        fn.restype = None
        fn.argtypes = [ctypes.c_int, ptr]
        if flavour == "oracle":
            for name in ("backward", "backward_second"):
                fn = getattr(lib, f"{pre}_{name}_{suffix}")
                fn.restype = None
                fn.argtypes = [ptr, ptr, ctypes.c_size_t, ctypes.c_int, ptr]
    getattr(lib, f"{pre}_max_threads").restype = ctypes.c_int
    _LIBS[flavour] = lib
    return lib


def _suffix(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float64:
        return "f64", ctypes.c_double
    if dtype == np.float32:
        return "f32", ctypes.c_float
    raise TypeError("float32 or float64 expected")


def _ptr(a, ct):
    return a.ctypes.data_as(ctypes.POINTER(ct)) if a is not None else None


def max_threads(flavour="oracle"):
    return getattr(_lib(flavour), f"{_PREFIX[flavour]}_max_threads")()


def prefactors(l_max, dtype=np.float64, flavour="oracle"):
    """F_l^m block followed by the Q-recursion block, (l_max+1)(l_max+2) numbers."""
    suffix, ct = _suffix(dtype)
    out = np.empty((l_max + 1) * (l_max + 2), dtype=dtype)
    getattr(_lib(flavour), f"{_PREFIX[flavour]}_prefactors_{suffix}")(l_max, _ptr(out, ct))
    return out


def compute(xyz, l_max, normalized, mode="values", flavour="oracle", out=None):
    """Evaluate on the CPU. Returns ``(sph, dsph, ddsph)`` (``None`` where not asked).

    ``out`` may carry preallocated ``(sph, dsph, ddsph)`` arrays (for timing).
    """
    mode = MODES[mode] if isinstance(mode, str) else int(mode)
    xyz = np.ascontiguousarray(xyz)
    suffix, ct = _suffix(xyz.dtype)
    if xyz.ndim != 2 or xyz.shape[1] != 3:
        raise ValueError("xyz must be N x 3")
    n = xyz.shape[0]
    ny = (l_max + 1) ** 2
    if out is None:
        sph = np.empty((n, ny), dtype=xyz.dtype)
        dsph = np.empty((n, 3, ny), dtype=xyz.dtype) if mode >= 1 else None
        ddsph = np.empty((n, 3, 3, ny), dtype=xyz.dtype) if mode >= 2 else None
    else:
        sph, dsph, ddsph = out
    fn = getattr(_lib(flavour), f"{_PREFIX[flavour]}_compute_{suffix}")
    status = fn(_ptr(xyz, ct), n, l_max, int(bool(normalized)), mode, _ptr(sph, ct), _ptr(dsph, ct), _ptr(ddsph, ct))
    if status != 0:
        raise RuntimeError(f"{flavour} compute failed with status {status}")
    return sph, dsph, ddsph


def recursion_route(xyz, l_max, normalized, mode="values", flavour="oracle"):
    """Same quantities through the recursion from l = 2 on (closed form only for l <= 1)."""
    mode = MODES[mode] if isinstance(mode, str) else int(mode)
    xyz = np.ascontiguousarray(xyz)
    suffix, ct = _suffix(xyz.dtype)
    n = xyz.shape[0]
    ny = (l_max + 1) ** 2
    sph = np.empty((n, ny), dtype=xyz.dtype)
    dsph = np.empty((n, 3, ny), dtype=xyz.dtype) if mode >= 1 else None
    fn = getattr(_lib(flavour), f"{_PREFIX[flavour]}_recursion_route_{suffix}")
    status = fn(_ptr(xyz, ct), n, l_max, int(bool(normalized)), mode, _ptr(sph, ct), _ptr(dsph, ct))
    if status != 0:
        raise RuntimeError(f"{flavour} recursion route failed with status {status}")
    return sph, dsph


def backward(dsph, sph_grad):
    """``xyz_grad[i, a] = sum_k dsph[i, a, k] * sph_grad[i, k]`` in the arrays' precision."""
    dsph = np.ascontiguousarray(dsph)
    sph_grad = np.ascontiguousarray(sph_grad, dtype=dsph.dtype)
    suffix, ct = _suffix(dsph.dtype)
    n, three, n_total = dsph.shape
    if three != 3 or sph_grad.shape != (n, n_total):
        raise ValueError("dsph must be N x 3 x n_total and sph_grad N x n_total")
    out = np.empty((n, 3), dtype=dsph.dtype)
    getattr(_lib("oracle"), f"sphx_oracle_backward_{suffix}")(
        _ptr(dsph, ct), _ptr(sph_grad, ct), n, n_total, _ptr(out, ct)
    )
    return out


def backward_second(ddsph, dsph_grad):
    """``xyz_grad[i, b] = sum_a sum_k ddsph[i, a, b, k] * dsph_grad[i, a, k]``."""
    ddsph = np.ascontiguousarray(ddsph)
    dsph_grad = np.ascontiguousarray(dsph_grad, dtype=ddsph.dtype)
    suffix, ct = _suffix(ddsph.dtype)
    n, n_total = ddsph.shape[0], ddsph.shape[3]
    if ddsph.shape[1:3] != (3, 3) or dsph_grad.shape != (n, 3, n_total):
        raise ValueError("ddsph must be N x 3 x 3 x n_total and dsph_grad N x 3 x n_total")
    out = np.empty((n, 3), dtype=ddsph.dtype)
    getattr(_lib("oracle"), f"sphx_oracle_backward_second_{suffix}")(
        _ptr(ddsph, ct), _ptr(dsph_grad, ct), n, n_total, _ptr(out, ct)
    )
    return out
