"""Cutoff modules (``equitorch/nn/cutoffs.py``): the edge length mapped to [0, 1] over ``[r_min, r_max]``, then one
of the envelopes of ``functional.cutoffs``.  The functions there are tensor expressions, as in the reference; the modules
here take one kernel each way for fp32 / fp64 tensors on the GPU (``functional/_radial.py``)."""
from torch import Tensor, nn

from .functional import _radial
from .functional.cutoffs import cosine_cutoff, mollifier_cutoff, polynomial_cutoff, radial_standarize


class _Cutoff(nn.Module):
    def __init__(self, r_max: float, r_min: float = 0.0):
        super().__init__()
        self.r_max, self.r_min = r_max, r_min
        self.range = float(r_max - r_min)

    def _unit(self, input: Tensor) -> Tensor:
        return radial_standarize(input, self.range, self.r_min)

    def _apply_envelope(self, input: Tensor, kind: int, param: float, expression) -> Tensor:
        """fp32 / fp64 tensors on the GPU: standardisation, envelope and (in the backward) their derivative in one
        launch; everything else the tensor expression."""
        if _radial.fused(input):
            return _radial.cutoff(input, kind, self.r_min, self.range, param, expression)
        return expression(input)


class PolynomialCutoff(_Cutoff):
    """Polynomial envelope of order ``p >= 2`` (reference ``:7-42``)."""

    def __init__(self, r_max: float, r_min: float = 0., p: float = 6):
        assert r_max >= r_min
        assert p >= 2.0
        super().__init__(r_max, r_min)
        self.p = float(p)

    def forward(self, input: Tensor) -> Tensor:
        return self._apply_envelope(input, _radial.POLYNOMIAL, self.p, lambda r: polynomial_cutoff(self._unit(r), p=self.p))


class CosineCutoff(_Cutoff):
    """Cosine envelope (reference ``:44-80``)."""

    def __init__(self, r_max: float, r_min: float = 0):
        assert r_min < r_max
        super().__init__(r_max, r_min)

    def forward(self, input: Tensor) -> Tensor:
        return self._apply_envelope(input, _radial.COSINE, 0.0, lambda r: cosine_cutoff(self._unit(r)))


class MollifierCutoff(_Cutoff):
    """Mollifier envelope (reference ``:82-131``)."""

    def __init__(self, r_max: float, r_min: float = 0, eps: float = 1e-7):
        assert r_min < r_max
        super().__init__(r_max, r_min)
        self.eps = eps

    def forward(self, input: Tensor) -> Tensor:
        return self._apply_envelope(input, _radial.MOLLIFIER, self.eps, lambda r: mollifier_cutoff(self._unit(r), eps=self.eps))
