"""``AnglesToMatrix`` (``equitorch/nn/rotations.py``)."""
from typing import Optional

from torch import Tensor, nn

from .functional.rotations import angles_to_matrix


class AnglesToMatrix(nn.Module):
    """ZYZ Euler angles -> rotation matrices ``(..., 3, 3)``."""

    def forward(self, alpha: Optional[Tensor] = None, beta: Optional[Tensor] = None,
                gamma: Optional[Tensor] = None) -> Tensor:
        return angles_to_matrix(alpha=alpha, beta=beta, gamma=gamma)
