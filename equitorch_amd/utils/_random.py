"""Random test inputs (``equitorch/utils/_random.py:5-84``)."""
import math

import torch


def rand_spherical_xyz(shape, device=None, dtype=None, generator=None) -> torch.Tensor:
    """Gaussian-normalised random unit vectors of shape ``(*shape, 3)``."""
    xyz = torch.randn(*shape, 3, device=device, dtype=dtype, generator=generator)
    return xyz / xyz.norm(dim=-1, keepdim=True)


def rand_spherical_angles(shape, device=None, dtype=None, generator=None):
    """``(theta, phi)`` of points uniform on the sphere: ``theta = acos(u)`` with ``u`` uniform on (-1, 1]
    (polar angle from +z), ``phi`` uniform on [0, 2 pi)."""
    theta = torch.acos(2 * torch.rand(shape, device=device, dtype=dtype, generator=generator) - 1)
    phi = 2 * math.pi * torch.rand(shape, device=device, dtype=dtype, generator=generator)
    return theta, phi


def rand_rotation_angles(shape, device=None, dtype=None, generator=None):
    """ZYZ Euler angles ``(alpha, beta, gamma)`` of Haar-uniform rotations: ``beta`` as the polar angle above,
    ``alpha`` and ``gamma`` uniform on [0, 2 pi).  Drawn in the order beta, alpha, gamma."""
    beta = torch.acos(2 * torch.rand(shape, device=device, dtype=dtype, generator=generator) - 1)
    alpha = 2 * math.pi * torch.rand(shape, device=device, dtype=dtype, generator=generator)
    gamma = 2 * math.pi * torch.rand(shape, device=device, dtype=dtype, generator=generator)
    return alpha, beta, gamma


def rand_rotation_matrices(shape, device=None, dtype=None, generator=None) -> torch.Tensor:
    """Rotation matrices ``(*shape, 3, 3)`` about a uniformly random axis by an angle uniform on [0, 2 pi)
    (Rodrigues: ``R = cos t I + sin t [a]x + (1 - cos t) a a^T``)."""
    axis = rand_spherical_xyz(shape, device, dtype, generator)
    angle = 2 * math.pi * torch.rand(shape, device=device, dtype=dtype, generator=generator)
    cos, sin = torch.cos(angle)[..., None, None], torch.sin(angle)[..., None, None]
    ax, ay, az = axis.unbind(-1)
    zero = torch.zeros_like(ax)
    cross = torch.stack([zero, -az, ay, az, zero, -ax, -ay, ax, zero], dim=-1).reshape(*axis.shape[:-1], 3, 3)
    eye = torch.eye(3, device=axis.device, dtype=axis.dtype)
    return cos * eye + sin * cross + (1 - cos) * (axis[..., :, None] * axis[..., None, :])
