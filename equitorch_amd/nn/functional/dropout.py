"""``irrep_wise_dropout`` (``equitorch/nn/functional/dropout.py``): whole irrep blocks of a channel are dropped
together, which keeps the result equivariant."""
import torch
from torch import Tensor

from ...structs import IrrepsInfo
from .activations import gating


def irrep_wise_dropout(input: Tensor, p: float, training: bool, irreps_info: IrrepsInfo) -> Tensor:
    """One Bernoulli(1 - p) draw per (sample, irrep, channel), scaled by ``1 / (1 - p)``, multiplied onto the irrep's
    components with the gating kernel.  Identity when ``p == 0`` or not ``training``."""
    if p < 0.0 or p > 1.0:
        raise ValueError(f"dropout probability has to be between 0 and 1, but got {p}")
    if p == 0.0 or not training:
        return input
    if irreps_info is None:
        raise ValueError("irreps_info cannot be None for irrep_wise_dropout")
    shape = (input.shape[0], irreps_info.num_irreps, input.shape[-1])
    mask = torch.bernoulli(torch.full(shape, 1.0 - p, dtype=input.dtype, device=input.device))
    mask = mask.div_(1.0 - p).nan_to_num_(nan=0)
    return gating(input, mask, irreps_info)
