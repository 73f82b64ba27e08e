"""``Gate`` (``equitorch/nn/activations.py:11-175``): scalar gates multiplied onto irrep blocks."""
import torch
from torch import Tensor, nn

from ._irreps_module import IrrepsModule
from .functional.activations import gating


class Gate(IrrepsModule):
    r"""``out[..., M, c] = input[..., M, c] * act(gate)[..., i, c]`` with ``i`` the irrep of component ``M``
    (``irrep_wise=True``, gate ``(..., len(irreps), C)`` or shared ``(len(irreps), C)``) or one gate for all
    components (``irrep_wise=False``, gate ``(..., 1, C)``).  With ``gate=None`` the last ``len(irreps)`` rows of
    ``input`` (``(..., irreps.dim + len(irreps), C)``) are the gates."""

    def __init__(self, irreps, activation: nn.Module = None, irrep_wise: bool = True):
        super().__init__(irreps)
        self.activation = activation
        self.irrep_wise = irrep_wise
        self.num_gates = len(self.irreps)

    def forward(self, input: Tensor, gate: Tensor = None) -> Tensor:
        channels = input.shape[-1]
        if gate is None:
            total = self.irreps_dim + self.num_gates
            assert input.shape[-2] == total, \
                f"Input spherical dim mismatch (concatenated mode): expected {total} (irreps.dim + num_gates), " \
                f"got {input.shape[-2]}"
            features, gate = torch.split(input, [self.irreps_dim, self.num_gates], dim=-2)
        else:
            features = input
            assert features.shape[-2] == self.irreps_dim, \
                f"Input feature spherical dim mismatch: expected {self.irreps_dim}, got {features.shape[-2]}"
            per_gate = (self.num_gates if self.irrep_wise else 1) * channels
            assert gate.numel() in (per_gate, per_gate * input.shape[0]), \
                f"Gate numel mismatch: expected {per_gate} or {per_gate * input.shape[0]}, got {gate.numel()}"
        if not self.irrep_wise:
            gate = gate.reshape(-1, 1, channels)
            if self.activation is not None:
                gate = self.activation(gate)
            return features * gate
        shared = gate.numel() == self.num_gates * channels          # an empty batch has an empty, batched gate
        gate = gate.reshape(self.num_gates, channels) if shared else gate.reshape(-1, self.num_gates, channels)
        if self.activation is not None:
            gate = self.activation(gate)
        lead = features.shape[:-2]
        out = gating(features.reshape(-1, self.irreps_dim, channels), gate, self.irreps_info)
        return out.reshape(*lead, self.irreps_dim, channels)

    def __repr__(self):
        return (f"{self.__class__.__name__}(irreps={self.irreps.short_repr()}, activation={self.activation}, "
                f"irrep_wise={self.irrep_wise}, num_gates={self.num_gates})")
