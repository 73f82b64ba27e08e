"""``sincos`` (``equitorch/nn/functional/angular.py``): the multiple-angle embedding the z rotations read."""
import torch
from torch import Tensor


def sincos(angle: Tensor, max_m: int, with_ones: bool = True, component_normalize: bool = False) -> Tensor:
    """``[1, sin a, cos a, sin 2a, cos 2a, ..., sin(max_m a), cos(max_m a)]`` along a new last axis (without the
    leading 1 if ``with_ones`` is false; sines and cosines times ``sqrt 2`` under ``component_normalize``).
    ``max_m == 0`` gives the single column of ones."""
    if max_m == 0:
        return torch.ones_like(angle).unsqueeze(-1)
    m = torch.arange(1, max_m + 1, dtype=angle.dtype, device=angle.device)
    ma = angle.unsqueeze(-1) * m
    pairs = torch.stack([torch.sin(ma), torch.cos(ma)], dim=-1)
    if component_normalize:
        pairs = pairs * (2 ** 0.5)
    pairs = pairs.flatten(-2, -1)
    return torch.cat([torch.ones_like(angle).unsqueeze(-1), pairs], dim=-1) if with_ones else pairs
