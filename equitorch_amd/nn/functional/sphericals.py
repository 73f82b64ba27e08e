"""``equitorch/nn/functional/sphericals.py``: spherical harmonics and the Cartesian / spherical conversions."""
import math
from typing import Optional

import torch
from torch import Tensor

from ...ops.spherical_harmonics import spherical_harmonics as _spherical_harmonics
from .angular import sincos

_INV_SQRT_4PI = 1.0 / (2.0 * math.sqrt(math.pi))


def spherical_harmonics(input: Tensor, l_max: int, dim: int = -1, integral_normalize: bool = False,
                        normalize_input: bool = False) -> Tensor:
    """``equitorch/nn/functional/sphericals.py:9-14``; ``integral_normalize`` scales by ``1/sqrt(4 pi)`` (inside
    the kernel).  ``normalize_input`` (not in the reference's signature) fuses the normalisation that
    ``SphericalHarmonics`` applies beforehand."""
    return _spherical_harmonics(input, l_max, dim, normalize=normalize_input,
                                scale=_INV_SQRT_4PI if integral_normalize else 1.0)


def xyz_to_spherical(xyz: Tensor, normalize_input: bool = True, with_r: bool = False, eps: float = 1e-14,
                     dim: int = -1):
    """``(theta, phi[, r])`` of Cartesian vectors (``equitorch/nn/functional/sphericals.py:17-74``): polar angle
    from the z axis, azimuth from the x axis in the x-y plane; same clamping constants."""
    if xyz.shape[dim] != 3:
        raise ValueError(f"Input `xyz` is expected to have 3 components along dimension `dim`={dim}, "
                         f"but got {xyz.shape[dim]}.")
    x, y, z = torch.unbind(xyz, dim=dim)
    r = torch.sqrt(xyz.pow(2).sum(dim=-1).clamp_min(eps))
    if normalize_input:
        x, y, z = x / r, y / r, z / r
    theta = torch.acos(torch.clamp(z, -1.0 + eps, 1.0 - eps))
    phi = torch.atan2(y, x + eps)
    return (theta, phi, r) if with_r else (theta, phi)


def spherical_to_xyz(theta: Tensor, phi: Tensor, r: Optional[Tensor] = None, dim: int = -1) -> Tensor:
    """Inverse of :func:`xyz_to_spherical` (``equitorch/nn/functional/sphericals.py:77-112``)."""
    st = torch.sin(theta)
    xyz = torch.stack([st * torch.cos(phi), st * torch.sin(phi), torch.cos(theta)], dim=dim)
    return xyz if r is None else xyz * r.unsqueeze(dim)


def xyz_to_sincos(xyz: Tensor, max_m: int, normalize_input: bool = True, component_normalize: bool = False,
                  eps: float = 1e-14, dim: int = -1):
    """``(sincos(theta), sincos(phi))`` of the polar angles of ``xyz``
    (``equitorch/nn/functional/sphericals.py:116-156``)."""
    theta, phi = xyz_to_spherical(xyz, normalize_input=normalize_input, with_r=False, eps=eps, dim=dim)
    return (sincos(theta, max_m, component_normalize=component_normalize),
            sincos(phi, max_m, component_normalize=component_normalize))
