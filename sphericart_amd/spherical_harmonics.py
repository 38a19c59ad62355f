"""Calculator classes over the ``sphericart_cuda_*`` C API."""

from typing import Tuple

import torch

from ._c_lib import get_library


class _BaseHarmonics:
    # reference: python/src/sphericart/spherical_harmonics.py:9-202
    _cuda_prefix = ""
    _normalized = 0

    def __init__(self, l_max: int, float32_via_float64: bool = False):
        """``float32_via_float64`` (not in the reference, off by default): float32 arrays are
        evaluated in float64 and rounded once (``sphx_forward_f32_via_f64``), which keeps
        l_max >= 29 finite where float32 arithmetic, the reference's included, overflows."""
        if int(l_max) != l_max or l_max < 0:
            raise ValueError("l_max must be a non-negative integer")
        self._l_max = int(l_max)
        self._float32_via_float64 = bool(float32_via_float64)
        self._lib = get_library()
        self._calculator_cuda = None
        self._calculator_cuda_f = None

    def __del__(self):
        self._delete_calculator(f"{self._cuda_prefix}_delete", "_calculator_cuda")
        self._delete_calculator(f"{self._cuda_prefix}_delete_f", "_calculator_cuda_f")

    def _delete_calculator(self, function_name: str, attribute: str):
        calculator = getattr(self, attribute, None)
        if calculator is not None:
            getattr(self._lib, function_name)(calculator)
            setattr(self, attribute, None)

    def _validate_xyz(self, xyz):
        if not isinstance(xyz, torch.Tensor):
            raise TypeError("xyz must be a torch.Tensor on a ROCm device")
        if xyz.dtype not in (torch.float32, torch.float64):
            raise TypeError("xyz must be an array of 32 or 64-bit floats")
        if xyz.dim() != 2 or xyz.shape[1] != 3:
            raise ValueError("xyz array must be a `N x 3` array")
        if not xyz.is_cuda:
            raise ValueError(
                "xyz must live on a ROCm device: sphericart_amd has no CPU evaluation path"
            )
        return xyz.contiguous()

    def _ensure_cuda_calculators(self):
        if self._calculator_cuda is not None and self._calculator_cuda_f is not None:
            return
        self._calculator_cuda = getattr(self._lib, f"{self._cuda_prefix}_new")(self._l_max)
        self._calculator_cuda_f = getattr(self._lib, f"{self._cuda_prefix}_new_f")(self._l_max)
        if self._calculator_cuda and self._calculator_cuda_f:
            return
        self._delete_calculator(f"{self._cuda_prefix}_delete", "_calculator_cuda")
        self._delete_calculator(f"{self._cuda_prefix}_delete_f", "_calculator_cuda_f")
        raise RuntimeError(
            "failed to initialize the device calculators; a HIP device must be visible and "
            "l_max must not exceed what the device tables cover"
        )

    def _compute_impl(self, xyz, gradients: bool = False, hessians: bool = False):
        xyz = self._validate_xyz(xyz)
        self._ensure_cuda_calculators()

        n_samples = xyz.shape[0]
        lmtotal = (self._l_max + 1) ** 2
        options = dict(dtype=xyz.dtype, device=xyz.device)
        sph = torch.empty((n_samples, lmtotal), **options)
        dsph = torch.empty((n_samples, 3, lmtotal), **options) if gradients else None
        ddsph = torch.empty((n_samples, 3, 3, lmtotal), **options) if hessians else None

        if self._float32_via_float64 and xyz.dtype == torch.float32 and n_samples > 0:
            self._compute_via_float64(xyz, sph, dsph, ddsph)
            return (sph, dsph, ddsph) if hessians else (sph, dsph) if gradients else sph

        with torch.cuda.device(xyz.device):
            stream = torch.cuda.current_stream().cuda_stream
            suffix = "" if xyz.dtype == torch.float64 else "_f"
            calculator = self._calculator_cuda if xyz.dtype == torch.float64 else self._calculator_cuda_f
            if ddsph is not None:
                function = getattr(self._lib, f"{self._cuda_prefix}_compute_array_with_hessians{suffix}")
                function(
                    calculator, xyz.data_ptr(), n_samples, sph.data_ptr(), dsph.data_ptr(),
                    ddsph.data_ptr(), stream,
                )
            elif dsph is not None:
                function = getattr(self._lib, f"{self._cuda_prefix}_compute_array_with_gradients{suffix}")
                function(calculator, xyz.data_ptr(), n_samples, sph.data_ptr(), dsph.data_ptr(), stream)
            else:
                function = getattr(self._lib, f"{self._cuda_prefix}_compute_array{suffix}")
                function(calculator, xyz.data_ptr(), n_samples, sph.data_ptr(), stream)

        if hessians:
            return sph, dsph, ddsph
        if gradients:
            return sph, dsph
        return sph

    def _compute_via_float64(self, xyz, sph, dsph, ddsph):
        derivatives = 2 if ddsph is not None else (1 if dsph is not None else 0)
        n_samples = xyz.shape[0]
        # Beyond the closed forms the library evaluates in one launch and needs no workspace (if a
        # shape should not fit that launch it takes one from the device's pool, in stream order).
        # Below, a workspace from torch's allocator: at most 256 MiB, the library walks over the
        # points in chunks of what it holds.
        workspace, size = None, 0
        if self._l_max <= (1 if derivatives == 2 else 6):
            wanted = self._lib.sphx_forward_f32_via_f64_workspace(n_samples, self._l_max, derivatives)
            floor = self._lib.sphx_forward_f32_via_f64_workspace(min(n_samples, 64), self._l_max, derivatives)
            size = max(min(wanted, 256 << 20), floor)
            workspace = torch.empty(size, dtype=torch.uint8, device=xyz.device)
        with torch.cuda.device(xyz.device):
            stream = torch.cuda.current_stream()
            status = self._lib.sphx_forward_f32_via_f64(
                xyz.data_ptr(), n_samples, self._l_max, self._normalized, derivatives,
                sph.data_ptr(), dsph.data_ptr() if dsph is not None else None,
                ddsph.data_ptr() if ddsph is not None else None,
                workspace.data_ptr() if workspace is not None else None, size, stream.cuda_stream,
            )
            if workspace is not None:
                workspace.record_stream(stream)
        if status != 0:
            raise RuntimeError(self._lib.sphx_last_error().decode())

    def compute(self, xyz):
        """Values, ``(n_samples, (l_max+1)**2)``."""
        return self._compute_impl(xyz)

    def compute_with_gradients(self, xyz) -> Tuple[torch.Tensor, torch.Tensor]:
        """Values and Cartesian gradients, ``(n_samples, 3, (l_max+1)**2)``."""
        return self._compute_impl(xyz, gradients=True)

    def compute_with_hessians(self, xyz) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """Values, gradients and Hessians, ``(n_samples, 3, 3, (l_max+1)**2)``."""
        return self._compute_impl(xyz, gradients=True, hessians=True)


class SphericalHarmonics(_BaseHarmonics):
    """Real spherical harmonics :math:`Y^m_l` up to ``l_max`` of points given in Cartesian coordinates."""

    _cuda_prefix = "sphericart_cuda_spherical_harmonics"
    _normalized = 1


class SolidHarmonics(_BaseHarmonics):
    """Solid harmonics :math:`r^l Y^m_l` up to ``l_max``."""

    _cuda_prefix = "sphericart_cuda_solid_harmonics"
