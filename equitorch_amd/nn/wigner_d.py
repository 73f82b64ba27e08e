"""Rotation modules (``equitorch/nn/wigner_d.py``)."""
from typing import Optional

import torch
from torch import Tensor, nn

from ..irreps import check_irreps
from ..structs import WignerRotationInfo
from ..utils._structs import wigner_d_info
from .functional.wigner_d import align_to_z_wigner_d, sparse_wigner_rotation, wigner_d_matrix


class _RotationModule(nn.Module):
    info: WignerRotationInfo

    def __init__(self, irreps, with_identity: bool):
        super().__init__()
        self.irreps = check_irreps(irreps)
        self.max_m = max((ir.l for ir in self.irreps), default=0)
        self.info = wigner_d_info(self.irreps)
        if with_identity:
            self.register_buffer("identity", torch.eye(self.irreps.dim))

    def _apply(self, *args, **kwargs):
        mod = super()._apply(*args, **kwargs)
        mod.info = self.info._apply(*args, **kwargs)
        return mod


class SparseWignerRotation(_RotationModule):
    """Rotates features ``(N, irreps.dim, C)`` by Euler angles given as ``sincos`` embeddings, without forming the
    Wigner matrix (reference ``:16-61``)."""

    def __init__(self, irreps):
        super().__init__(irreps, with_identity=False)

    def forward(self, input: Tensor, sincos_alpha: Optional[Tensor], sincos_beta: Optional[Tensor],
                sincos_gamma: Optional[Tensor]) -> Tensor:
        return sparse_wigner_rotation(input, sincos_alpha, sincos_beta, sincos_gamma, self.info)

    def extra_repr(self) -> str:
        return f"irreps={self.irreps}, max_m={self.max_m}"


class DenseWignerRotation(nn.Module):
    """``wigner_d (N, dim, dim) @ input (N, dim, C)`` (reference ``:63-84``)."""

    def __init__(self, irreps):
        super().__init__()
        self.irreps = check_irreps(irreps)

    def forward(self, input: Tensor, wigner_d: Tensor) -> Tensor:
        return wigner_d @ input

    def extra_repr(self) -> str:
        return f"irreps={self.irreps}"


class WignerD(_RotationModule):
    """Dense Wigner matrices ``D(alpha, beta, gamma)`` from angles or their ``sincos`` embeddings
    (reference ``:87-146``)."""

    def __init__(self, irreps):
        super().__init__(irreps, with_identity=True)

    def forward(self, alpha: Optional[Tensor] = None, beta: Optional[Tensor] = None, gamma: Optional[Tensor] = None,
                sincos_alpha: Optional[Tensor] = None, sincos_beta: Optional[Tensor] = None,
                sincos_gamma: Optional[Tensor] = None) -> Tensor:
        return wigner_d_matrix(self.identity, alpha, beta, gamma, sincos_alpha, sincos_beta, sincos_gamma, self.info)

    def extra_repr(self) -> str:
        return f"irreps={self.irreps}"


class AlignToZWignerD(_RotationModule):
    """Wigner matrices of the rotations that take the vectors ``xyz (N, 3)`` to the z axis
    (reference ``:149-268``)."""

    def __init__(self, irreps, normalized: bool = True, eps: float = 1e-14):
        super().__init__(irreps, with_identity=True)
        self.normalized, self.eps = normalized, eps

    def forward(self, xyz: Tensor) -> Tensor:
        return align_to_z_wigner_d(eye=self.identity, xyz=xyz, max_m=self.max_m, info=self.info,
                                   normalized=self.normalized, eps=self.eps)

    def extra_repr(self) -> str:
        return f"irreps={self.irreps}, normalized={self.normalized}, eps={self.eps}"
