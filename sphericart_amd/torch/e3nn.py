"""Spherical harmonics in the conventions of ``e3nn.o3.spherical_harmonics``.

Counterpart of sphericart-torch/python/sphericart/torch/e3nn.py: the same three
functions with the same arguments, evaluated by this package's differentiable
GPU calculators. e3nn itself is not needed (and not imported).

What differs between the two conventions:

* axes: e3nn's real harmonics of degree one are ordered and signed like
  ``(x, y, z)``, sphericart's like ``(y, z, x)``; evaluating sphericart's at the
  rotated point ``(z, x, y)`` gives e3nn's ordering for every degree;
* scale: ``"integral"`` is sphericart's own (orthonormal on the sphere),
  ``"component"`` multiplies by ``sqrt(4 pi)``, ``"norm"`` additionally divides
  degree ``l`` by ``sqrt(2l + 1)``.
"""

import math
from typing import List, Union

import torch

from . import SolidHarmonics, SphericalHarmonics

_SCALES = ("integral", "norm", "component")


def e3nn_spherical_harmonics(l_list: Union[List[int], int], x: torch.Tensor, normalize: bool = False,
                             normalization: str = "integral") -> torch.Tensor:
    """Harmonics of the degrees in ``l_list`` (an integer or a list of integers) of the points
    ``x`` (``[n, 3]``), one block of ``2l + 1`` columns per requested degree, in the order given.

    Every degree up to ``max(l_list)`` is evaluated and the requested ones are picked.
    ``normalize=True`` evaluates at ``x / |x|`` (spherical harmonics), ``False`` gives the solid
    harmonics ``r^l Y_l^m``. ``normalization`` is one of ``"integral"``, ``"component"``, ``"norm"``.
    """
    degrees = [int(l_list)] if not hasattr(l_list, "__len__") else [int(l) for l in l_list]
    if not degrees or min(degrees) < 0:
        raise ValueError("l_list must name at least one non-negative degree")
    if normalization not in _SCALES:
        raise ValueError(f"normalization must be one of {_SCALES}")
    l_max = max(degrees)
    calculator = SphericalHarmonics(l_max) if normalize else SolidHarmonics(l_max)
    everything = calculator(x[:, [2, 0, 1]])

    factors = []
    for l in degrees:
        factor = 1.0 if normalization == "integral" else math.sqrt(4.0 * math.pi)
        if normalization == "norm":
            factor /= math.sqrt(2 * l + 1)
        factors.append(factor)
    if degrees == list(range(l_max + 1)) and normalization != "norm":
        return everything if normalization == "integral" else everything * factors[0]
    blocks = [everything[:, l * l:(l + 1) * (l + 1)] * f for l, f in zip(degrees, factors)]
    return torch.cat(blocks, dim=-1)


_original = None


def patch_e3nn(e3nn_module) -> None:
    """Make ``e3nn_module.o3.spherical_harmonics`` call :func:`e3nn_spherical_harmonics`."""
    global _original
    if _original is not None:
        raise RuntimeError("It appears that e3nn has already been patched")
    _original = e3nn_module.o3.spherical_harmonics
    e3nn_module.o3.spherical_harmonics = e3nn_spherical_harmonics


def unpatch_e3nn(e3nn_module) -> None:
    """Put back what :func:`patch_e3nn` replaced."""
    global _original
    if _original is None:
        raise RuntimeError("It appears that e3nn has not been patched")
    e3nn_module.o3.spherical_harmonics = _original
    _original = None
