"""``torch.nn.Module`` calculators with autograd, as ``sphericart.torch`` has them.

Same two classes and methods as the reference's
sphericart-torch/python/sphericart/torch/spherical_hamonics.py (``forward``,
``compute``, ``compute_with_gradients``, ``compute_with_hessians``, ``l_max``);
the operators behind them are registered in :mod:`sphericart_amd.torch.ops`.
Tensors must live on the GPU. ``omp_num_threads`` reports 1: there is no host
evaluator and no OpenMP team behind the operators.
"""

from typing import Tuple

import torch
from torch import Tensor

from . import ops  # noqa: F401  (registers the operators)


class SphericalHarmonics(torch.nn.Module):
    """Real spherical harmonics of the directions of ``xyz`` up to ``l_max``, differentiable.

    The operator names are written out (no lookup by string), so that ``torch.jit.script`` and
    ``torch.compile(fullgraph=True)`` see through the module."""

    def __init__(self, l_max: int):
        super().__init__()
        if l_max < 0:
            raise ValueError("l_max must be non-negative")
        self._l_max = int(l_max)

    def forward(self, xyz: Tensor) -> Tensor:
        return torch.ops.sphericart_amd.spherical_harmonics(xyz, self._l_max)

    def compute(self, xyz: Tensor) -> Tensor:
        return self.forward(xyz)

    def compute_with_gradients(self, xyz: Tensor) -> Tuple[Tensor, Tensor]:
        return torch.ops.sphericart_amd.spherical_harmonics_with_gradients(xyz, self._l_max)

    def compute_with_hessians(self, xyz: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
        return torch.ops.sphericart_amd.spherical_harmonics_with_hessians(xyz, self._l_max)

    def omp_num_threads(self) -> int:
        """Threads of the host evaluator in the reference; 1 here (GPU only)."""
        return 1

    def l_max(self) -> int:
        return self._l_max


class SolidHarmonics(torch.nn.Module):
    """Solid harmonics ``r^l Y_l^m`` of ``xyz`` up to ``l_max``, differentiable."""

    def __init__(self, l_max: int):
        super().__init__()
        if l_max < 0:
            raise ValueError("l_max must be non-negative")
        self._l_max = int(l_max)

    def forward(self, xyz: Tensor) -> Tensor:
        return torch.ops.sphericart_amd.solid_harmonics(xyz, self._l_max)

    def compute(self, xyz: Tensor) -> Tensor:
        return self.forward(xyz)

    def compute_with_gradients(self, xyz: Tensor) -> Tuple[Tensor, Tensor]:
        return torch.ops.sphericart_amd.solid_harmonics_with_gradients(xyz, self._l_max)

    def compute_with_hessians(self, xyz: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
        return torch.ops.sphericart_amd.solid_harmonics_with_hessians(xyz, self._l_max)

    def omp_num_threads(self) -> int:
        """See :py:meth:`SphericalHarmonics.omp_num_threads`."""
        return 1

    def l_max(self) -> int:
        return self._l_max


from .e3nn import e3nn_spherical_harmonics, patch_e3nn, unpatch_e3nn  # noqa: E402

__all__ = ["SphericalHarmonics", "SolidHarmonics", "e3nn_spherical_harmonics", "patch_e3nn", "unpatch_e3nn"]
