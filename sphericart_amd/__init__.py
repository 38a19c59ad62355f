"""MI355X-native (gfx950, HIP) evaluator of real spherical and solid harmonics.

Host-side mirror of the reference's Python calculators
(python/src/sphericart/spherical_harmonics.py:9-236) for arrays that live on
the GPU: ``SphericalHarmonics(l_max)`` / ``SolidHarmonics(l_max)`` with
``compute``, ``compute_with_gradients`` and ``compute_with_hessians``. Where the
reference takes CuPy arrays and hands their pointers to the
``sphericart_cuda_*`` C functions, this package takes ``torch`` tensors on a
ROCm device and hands their pointers to the same functions of
``libsphericart_amd.so``. torch only provides device memory and the current
stream; all arithmetic happens in the HIP kernels of the library. There is no
CPU path: CPU tensors are rejected.
"""

from ._c_lib import get_library
from .spherical_harmonics import SolidHarmonics, SphericalHarmonics

__all__ = ["SphericalHarmonics", "SolidHarmonics", "get_library"]
