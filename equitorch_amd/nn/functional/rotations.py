"""``angles_to_matrix`` (``equitorch/nn/functional/rotations.py``): ZYZ Euler angles to 3x3 rotation matrices."""
from typing import Optional

import torch
from torch import Tensor


def _axis_rotation(angle: Tensor, axis: str) -> Tensor:
    c, s, o, z = torch.cos(angle), torch.sin(angle), torch.ones_like(angle), torch.zeros_like(angle)
    rows = {"z": [c, -s, z, s, c, z, z, z, o], "y": [c, z, s, z, o, z, -s, z, c]}[axis]
    return torch.stack(rows, dim=-1).reshape(*angle.shape, 3, 3)


def angles_to_matrix(alpha: Optional[Tensor] = None, beta: Optional[Tensor] = None,
                     gamma: Optional[Tensor] = None) -> Tensor:
    """``R_z(gamma) R_y(beta) R_z(alpha)`` for broadcastable angle tensors (an angle given as ``None`` is zero), the
    order of the reference (``:100``: ``R_gamma @ R_beta @ R_alpha``).  Note that ``wigner_d_matrix(alpha, beta,
    gamma)`` represents ``R_z(alpha) R_y(beta) R_z(gamma)``, i.e. this function with alpha and gamma exchanged."""
    given = [a for a in (alpha, beta, gamma) if a is not None]
    if not given:
        raise ValueError("At least one of alpha, beta, or gamma must be provided.")
    try:
        shape = torch.broadcast_shapes(*(a.shape for a in given))
    except RuntimeError as e:
        raise ValueError(f"Could not broadcast shapes of alpha, beta, gamma: {[a.shape for a in given]}. Error: {e}")
    zero = torch.zeros(shape, dtype=given[0].dtype, device=given[0].device)
    a, b, g = (zero if t is None else t.expand(shape) for t in (alpha, beta, gamma))
    return _axis_rotation(g, "z") @ _axis_rotation(b, "y") @ _axis_rotation(a, "z")
