"""Invariant norm modules (``equitorch/nn/norm.py``)."""
from torch import Tensor

from ._irreps_module import IrrepsModule
from .functional.norm import batch_mean_squared_norm, channel_mean_squared_norm, norm, squared_norm


class SquaredNorm(IrrepsModule):
    """``(..., irreps.dim, C) -> (..., len(irreps), C)``: squared L2 norm of every irrep block, divided by the
    block's dimension when ``scaled`` (reference ``:12-45``)."""

    def __init__(self, irreps, scaled: bool = True):
        super().__init__(irreps)
        self.scaled = scaled

    def forward(self, input_tensor: Tensor) -> Tensor:
        self._check_dim(input_tensor)
        return squared_norm(input_tensor, self.irreps_info, self.scaled)

    def extra_repr(self):
        return f"irreps='{self.irreps}', scaled={self.scaled}"


class Norm(SquaredNorm):
    """L2 norm of every irrep block, times ``dim^-1/2`` when ``scaled``; zero gradient at a zero block
    (reference ``:48-79``)."""

    def forward(self, input_tensor: Tensor) -> Tensor:
        self._check_dim(input_tensor)
        return norm(input_tensor, self.irreps_info, self.scaled)


class MeanSquaredNorm(IrrepsModule):
    """Squared norm averaged over the batch axis (``dim=0`` -> ``(len(irreps), C)``) or the channel axis
    (``dim=-1`` or ``2`` -> ``(..., len(irreps))``) (reference ``:82-133``)."""

    def __init__(self, irreps, scaled: bool = True, dim: int = -1):
        super().__init__(irreps)
        if dim not in (0, -1, 2):
            raise ValueError(f"Unsupported dim value: {dim}. Allowed values are 0, -1, 2.")
        self.scaled = scaled
        self.dim = -1 if dim == 2 else dim

    def forward(self, input_tensor: Tensor) -> Tensor:
        self._check_dim(input_tensor)
        fn = batch_mean_squared_norm if self.dim == 0 else channel_mean_squared_norm
        return fn(input_tensor, self.irreps_info, self.scaled)

    def extra_repr(self):
        return f"irreps='{self.irreps}', scaled={self.scaled}, dim={self.dim}"
