"""RMS normalisation layers (``equitorch/nn/normalization.py``)."""
import torch
from torch import Tensor, nn

from ._irreps_module import IrrepsModule
from .functional.normalization import batch_rms_norm, layer_rms_norm


class _RMSNormBase(IrrepsModule):
    def __init__(self, irreps, channels: int, eps: float, affine: bool, scaled: bool):
        super().__init__(irreps)
        self.channels, self.eps, self.affine, self.scaled = channels, eps, affine, scaled
        self.num_irreps = len(self.irreps)
        if affine:
            self.weight = nn.Parameter(torch.ones(self.num_irreps, channels))
        else:
            self.register_parameter("weight", None)

    def _check(self, input_tensor: Tensor) -> None:
        if input_tensor.ndim != 3:
            raise ValueError(f"Input tensor must be 3D (N, irreps_dim, C), got {input_tensor.ndim}D. "
                             f"Shape: {input_tensor.shape}")
        self._check_dim(input_tensor)
        if input_tensor.shape[-1] != self.channels:
            raise ValueError(f"Input tensor's channel dimension ({input_tensor.shape[-1]}) does not match expected "
                             f"channels ({self.channels})")

    def reset_parameters(self) -> None:
        if self.weight is not None:
            nn.init.ones_(self.weight)


class BatchRMSNorm(_RMSNormBase):
    """Divides every irrep block and channel by the root of its batch-mean squared norm (running average in
    evaluation mode), then scales by a learnable ``(len(irreps), C)`` weight (reference ``:9-118``)."""

    def __init__(self, irreps, channels: int, eps: float = 1e-5, momentum: float = 0.1, affine: bool = True,
                 scaled: bool = True):
        super().__init__(irreps, channels, eps, affine, scaled)
        self.momentum = momentum
        self.register_buffer("running_squared_norm", torch.ones(self.num_irreps, channels))

    def reset_running_stats(self) -> None:
        self.running_squared_norm.fill_(1.0)

    def reset_parameters(self) -> None:
        self.reset_running_stats()
        super().reset_parameters()

    def forward(self, input_tensor: Tensor) -> Tensor:
        self._check(input_tensor)
        return batch_rms_norm(input_tensor, self.running_squared_norm, self.irreps_info, self.weight,
                              scaled=self.scaled, training=self.training, momentum=self.momentum, eps=self.eps)

    def extra_repr(self):
        return (f"irreps='{self.irreps}', channels={self.channels}, eps={self.eps}, momentum={self.momentum}, "
                f"affine={self.affine}, scaled={self.scaled}")


class LayerRMSNorm(_RMSNormBase):
    """Divides every irrep block of every sample by the root of its channel-mean squared norm, then scales by a
    learnable ``(len(irreps), C)`` weight (reference ``:121-238``)."""

    def __init__(self, irreps, channels: int, eps: float = 1e-5, affine: bool = True, scaled: bool = True):
        super().__init__(irreps, channels, eps, affine, scaled)

    def forward(self, input_tensor: Tensor) -> Tensor:
        self._check(input_tensor)
        return layer_rms_norm(input_tensor, self.irreps_info, self.weight, scaled=self.scaled, eps=self.eps)

    def extra_repr(self):
        return (f"irreps='{self.irreps}', channels={self.channels}, eps={self.eps}, affine={self.affine}, "
                f"scaled={self.scaled}")
