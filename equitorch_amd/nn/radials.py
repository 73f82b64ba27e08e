"""Radial basis (``equitorch/nn/radials.py``)."""
import math

import torch
from torch import Tensor, nn

from .functional import _radial


class BesselBasis(nn.Module):
    r"""``b_n(r) = (2 / r_max) sin(n pi r / r_max) / r`` for ``n = 1..num_basis`` (reference ``:10-58``); the
    frequencies ``n pi`` are a parameter when ``trainable``, a buffer otherwise.  ``(...,) -> (..., num_basis)``.  fp32 /
    fp64 tensors on the GPU take one kernel forward and one for the gradient; everything else the tensor expression."""

    def __init__(self, r_max, num_basis=8, trainable=True):
        super().__init__()
        self.trainable = trainable
        self.num_basis = num_basis
        self.r_max = float(r_max)
        self.prefactor = 2.0 / self.r_max
        freq = torch.linspace(start=1.0, end=num_basis, steps=num_basis) * math.pi
        if trainable:
            self.bessel_weights = nn.Parameter(freq)
        else:
            self.register_buffer("bessel_weights", freq)

    def _expression(self, x: Tensor, freq: Tensor) -> Tensor:
        r = x.unsqueeze(-1)
        return self.prefactor * (torch.sin(freq * r / self.r_max) / r)

    def forward(self, x: Tensor) -> Tensor:
        if _radial.fused(x, self.bessel_weights):      # one launch each way instead of the expression's five
            return _radial.bessel(x, self.bessel_weights, self.r_max, self._expression)
        return self._expression(x, self.bessel_weights)
