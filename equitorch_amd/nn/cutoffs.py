"""Cutoff modules (``equitorch/nn/cutoffs.py``): the edge length mapped to [0, 1] over ``[r_min, r_max]``, then one
of the envelopes of ``functional.cutoffs``."""
from torch import Tensor, nn

from .functional.cutoffs import cosine_cutoff, mollifier_cutoff, polynomial_cutoff, radial_standarize


class _Cutoff(nn.Module):
    def __init__(self, r_max: float, r_min: float = 0.0):
        super().__init__()
        self.r_max, self.r_min = r_max, r_min
        self.range = float(r_max - r_min)

    def _unit(self, input: Tensor) -> Tensor:
        return radial_standarize(input, self.range, self.r_min)


class PolynomialCutoff(_Cutoff):
    """Polynomial envelope of order ``p >= 2`` (reference ``:7-42``)."""

    def __init__(self, r_max: float, r_min: float = 0., p: float = 6):
        assert r_max >= r_min
        assert p >= 2.0
        super().__init__(r_max, r_min)
        self.p = float(p)

    def forward(self, input: Tensor) -> Tensor:
        return polynomial_cutoff(self._unit(input), p=self.p)


class CosineCutoff(_Cutoff):
    """Cosine envelope (reference ``:44-80``)."""

    def __init__(self, r_max: float, r_min: float = 0):
        assert r_min < r_max
        super().__init__(r_max, r_min)

    def forward(self, input: Tensor) -> Tensor:
        return cosine_cutoff(self._unit(input))


class MollifierCutoff(_Cutoff):
    """Mollifier envelope (reference ``:82-131``)."""

    def __init__(self, r_max: float, r_min: float = 0, eps: float = 1e-7):
        assert r_min < r_max
        super().__init__(r_max, r_min)
        self.eps = eps

    def forward(self, input: Tensor) -> Tensor:
        return mollifier_cutoff(self._unit(input), eps=self.eps)
