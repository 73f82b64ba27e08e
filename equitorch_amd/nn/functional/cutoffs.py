"""Radial cutoff envelopes (``equitorch/nn/functional/cutoffs.py``).  Element-wise functions of the edge length;
like the reference they are plain tensor expressions (no kernel of this library is involved)."""
import math

import torch
from torch import Tensor


def radial_standarize(input: Tensor, range: float, r_min: float) -> Tensor:
    """``clamp((input - r_min) / range, 0, 1)`` (reference ``:4-10``)."""
    if r_min != 0:
        input = input - r_min
    return (input / range).clamp(0, 1)


def polynomial_cutoff(input: Tensor, p: float = 6.0) -> Tensor:
    """``1 - (p+1)(p+2)/2 u^p + p(p+2) u^(p+1) - p(p+1)/2 u^(p+2)`` on ``u`` in [0, 1] (reference ``:14-24``): value 1
    and vanishing first and second derivatives at 0, all three zero at 1."""
    a, b, c = (p + 1.0) * (p + 2.0) / 2.0, p * (p + 2.0), p * (p + 1.0) / 2
    return 1.0 - a * torch.pow(input, p) + b * torch.pow(input, p + 1.0) - c * torch.pow(input, p + 2.0)


def cosine_cutoff(input: Tensor) -> Tensor:
    """``(1 + cos(pi u)) / 2`` (reference ``:26-29``)."""
    return 0.5 * (1.0 + torch.cos(math.pi * input))


def mollifier_cutoff(input: Tensor, eps: float = 1e-12) -> Tensor:
    """``exp(1 - 1 / (1 - u^2 + eps))`` (reference ``:31-34``)."""
    return torch.exp(1 - 1 / (1 - input ** 2 + eps))
