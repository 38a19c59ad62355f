"""Build the HIP library in-tree: ``python -m sphericart_amd.build``.

``hipcc`` compiles the kernels for gfx950 and the host-side C and C++ API, one
translation unit per process, and links them into
``sphericart_amd/libsphericart_amd.so``. hipcc cross-compiles, so this works on a
machine without a GPU. Where torch is importable, ``g++`` then compiles the
torch operators' C++ side (``csrc/sphx_torch.cpp``, host code only) against its
headers into ``sphericart_amd/libsphericart_amd_torch.so``.
"""

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBRARY = os.path.join(HERE, "libsphericart_amd.so")

OBJECTS = os.path.join(HERE, "build")

# the translation units with the most kernels first: they take longest
SOURCES = [
    "sphx_forward_f64_hessians.hip", "sphx_forward_f32_hessians.hip", "sphx_wide_hessians.hip",
    "sphx_forward_f64_gradients.hip", "sphx_forward_f32_gradients.hip", "sphx_wide_gradients.hip",
    "sphx_forward_f64_values.hip", "sphx_forward_f32_values.hip", "sphx_wide_values.hip",
    "sphx_vjp_f64.hip", "sphx_vjp_f32.hip", "sphx_pairs.hip", "sphx_backward.hip", "sphx_via_f64.hip",
    "sphx_probe.hip",
    "sphx_runtime.cpp", "sphx_plan.cpp", "sphx_tables.cpp", "device_api.cpp", "capi.cpp",
]

# -ffp-contract=off: one rounding per source-level operation, on device and
#   host alike; results then match the reference CPU evaluator built the same
#   way bit for bit instead of merely within tolerance.
# -packed-fp32-ops off: no v_pk_*_f32 code generation.
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fPIC",
    "-fvisibility=hidden",
]


TORCH_SOURCE = os.path.join(CSRC, "sphx_torch.cpp")
TORCH_LIBRARY = os.path.join(HERE, "libsphericart_amd_torch.so")

EXAMPLE_SOURCE = os.path.join(os.path.dirname(HERE), "examples", "device_example.cpp")
EXAMPLE = os.path.join(HERE, "device_example")


def hipcc():
    found = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(found):
        raise RuntimeError("hipcc not found; a ROCm toolchain is required to build sphericart_amd")
    return found


def build(verbose=False, extra_flags=(), jobs=None):
    """Compile ``libsphericart_amd.so``; raises ``RuntimeError`` with the compiler output on failure."""
    os.makedirs(OBJECTS, exist_ok=True)

    def compile_one(source):
        target = os.path.join(OBJECTS, os.path.splitext(source)[0] + ".o")
        command = [hipcc(), *FLAGS, *extra_flags, "-c", os.path.join(CSRC, source), "-o", target]
        if verbose:
            print(" ".join(command), flush=True)
        done = subprocess.run(command, capture_output=True, text=True)
        if done.returncode != 0:
            raise RuntimeError(f"hipcc failed on {source} ({done.returncode}):\n{done.stdout}\n{done.stderr}")
        return target

    workers = jobs or min(len(SOURCES), os.cpu_count() or 1, 16)
    with ThreadPoolExecutor(max_workers=workers) as pool:
        objects = list(pool.map(compile_one, SOURCES))
    command = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *objects, "-o", LIBRARY]
    if verbose:
        print(" ".join(command), flush=True)
    done = subprocess.run(command, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"hipcc failed to link ({done.returncode}):\n{done.stdout}\n{done.stderr}")
    build_example(verbose)
    build_torch_operators(verbose)
    return LIBRARY


def build_torch_operators(verbose=False):
    """``libsphericart_amd_torch.so``: schemas and device implementations of the torch operators, against the
    headers of the torch that is installed. Returns None (and builds nothing) where torch is not importable: the
    operators are then implemented in Python (sphericart_amd/torch/ops.py)."""
    # (run as a script from its own directory, the package's `torch` subpackage would shadow torch itself)
    shadowed = [path for path in sys.path if os.path.abspath(path or ".") == HERE]
    for path in shadowed:
        sys.path.remove(path)
    try:
        import torch
        from torch.utils import cpp_extension
    except ImportError:
        if verbose:
            print("torch is not importable: libsphericart_amd_torch.so not built", flush=True)
        return None
    libraries = os.path.join(os.path.dirname(torch.__file__), "lib")
    command = [
        shutil.which("g++") or "g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
        "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}",
        *["-I" + path for path in cpp_extension.include_paths()], "-I/opt/rocm/include",
        TORCH_SOURCE, "-L" + HERE, "-lsphericart_amd", "-L" + libraries,
        "-ltorch", "-ltorch_cpu", "-lc10", "-lc10_hip", "-ltorch_hip", "-Wl,-rpath,$ORIGIN", "-o", TORCH_LIBRARY,
    ]
    if verbose:
        print(" ".join(command), flush=True)
    done = subprocess.run(command, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"g++ failed on sphx_torch.cpp ({done.returncode}):\n{done.stdout}\n{done.stderr}")
    return TORCH_LIBRARY


def build_example(verbose=False):
    """The C++ consumer of the device classes that the GPU tests run (host code only)."""
    command = [
        hipcc(), "-O2", "-std=c++17", "-I" + os.path.join(os.path.dirname(HERE), "include"),
        EXAMPLE_SOURCE, "-L" + HERE, "-lsphericart_amd", "-Wl,-rpath,$ORIGIN", "-o", EXAMPLE,
    ]
    if verbose:
        print(" ".join(command), flush=True)
    done = subprocess.run(command, capture_output=True, text=True)
    if done.returncode != 0:
        raise RuntimeError(f"hipcc failed on the example ({done.returncode}):\n{done.stdout}\n{done.stderr}")
    return EXAMPLE


if __name__ == "__main__":
    print(build(verbose=True))
