"""TEST INFRASTRUCTURE ONLY: the radial basis and the cutoff envelopes as the reference defines them, in float64
torch (differentiable: autograd of these expressions is the gradient oracle).

* ``bessel``: ``equitorch/nn/radials.py:46-58`` — ``prefactor * sin(w r / r_max) / r`` with ``prefactor = 2 / r_max``
  (``:36``) and ``w = pi * (1 .. num_basis)`` (``:38-40``) unless trained.
* ``standardize``: ``equitorch/nn/functional/cutoffs.py:4-25`` — ``clamp((r - r_min) / range, 0, 1)``.
* ``polynomial``: ``:30-49``; ``cosine``: ``:52-64``; ``mollifier``: ``:67-80``.
* ``cutoff``: the modules' composition ``envelope(standardize(r))`` (``equitorch/nn/cutoffs.py:7-131``).

Pinned by (tests/test_radial.py), none of it a retyped formula: the Bessel functions vanish at ``r = r_max``, take the
value ``4 / r_max^2`` at ``r_max / 2`` for ``n = 1`` and are orthogonal with ``int_0^R b_n b_m r^2 dr = (2 / R) delta_nm``
(a wrong prefactor, frequency or power of r fails one of the three); the polynomial envelope is 1 at 0 and 0 at 1 with
vanishing first and second derivatives at both ends and equals ``1 - 28 u^6 + 48 u^7 - 21 u^8`` at ``p = 6`` (any wrong
coefficient breaks a derivative condition); the cosine envelope is 1, 1/2, 0 at u = 0, 1/2, 1; the mollifier is
``exp(-1/3)`` at ``u = 1/2`` for ``eps -> 0`` and below 1e-300 at 1; all envelopes are constant outside ``[r_min, r_max]``.
"""
import math

import torch


def bessel(r: torch.Tensor, r_max: float, num_basis: int = 8, weights: torch.Tensor = None) -> torch.Tensor:
    w = (torch.arange(1, num_basis + 1, dtype=r.dtype) * math.pi) if weights is None else weights
    x = r.unsqueeze(-1)
    return (2.0 / r_max) * (torch.sin(w * x / r_max) / x)


def standardize(r: torch.Tensor, span: float, r_min: float) -> torch.Tensor:
    if r_min != 0:
        r = r - r_min
    return (r / span).clamp(0, 1)


def polynomial(u: torch.Tensor, p: float = 6.0) -> torch.Tensor:
    out = 1.0
    out = out - (((p + 1.0) * (p + 2.0) / 2.0) * torch.pow(u, p))
    out = out + (p * (p + 2.0) * torch.pow(u, p + 1.0))
    out = out - ((p * (p + 1.0) / 2) * torch.pow(u, p + 2.0))
    return out


def cosine(u: torch.Tensor) -> torch.Tensor:
    return 0.5 * (1.0 + torch.cos(math.pi * u))


def mollifier(u: torch.Tensor, eps: float = 1e-12) -> torch.Tensor:
    return torch.exp(1 - 1 / (1 - u ** 2 + eps))


def cutoff(kind: str, r: torch.Tensor, r_max: float, r_min: float = 0.0, param: float = None) -> torch.Tensor:
    u = standardize(r, r_max - r_min, r_min)
    if kind == "polynomial":
        return polynomial(u, 6.0 if param is None else param)
    if kind == "cosine":
        return cosine(u)
    return mollifier(u, 1e-12 if param is None else param)
