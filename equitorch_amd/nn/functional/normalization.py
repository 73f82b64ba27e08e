"""RMS normalisation of equivariant features (``equitorch/nn/functional/normalization.py``)."""
import torch
from torch import Tensor

from ...structs import IrrepsInfo
from .activations import _broadcast_infos
from .norm import channel_mean_squared_norm, squared_norm
from .sparse_product import sparse_mul, sparse_vecsca


def batch_rms_norm(input: Tensor, running_squared_norm: Tensor, irreps_info: IrrepsInfo, weight: Tensor = None,
                   scaled: bool = True, training: bool = False, momentum: float = 0.1, eps: float = 1e-05) -> Tensor:
    """``out[n, M, c] = input[n, M, c] * weight[i, c] / sqrt(s[i, c] + eps)`` with ``i`` the irrep of ``M`` and
    ``s`` the batch mean of the per-sample squared norms when ``training`` (then also blended into
    ``running_squared_norm`` in place with ``momentum``), else ``running_squared_norm`` (reference ``:10-72``)."""
    if training:
        stat = squared_norm(input, irreps_info, scaled).mean(dim=0)
        running_squared_norm.data.lerp_(stat.detach().to(running_squared_norm.dtype), momentum)
    else:
        stat = running_squared_norm
    scale = torch.rsqrt(stat + eps)
    if weight is not None:
        scale = weight * scale
    return sparse_mul(input, scale, *_broadcast_infos(irreps_info))


def layer_rms_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, weight: Tensor = None, scaled: bool = True,
                   eps: float = 1e-05) -> Tensor:
    """``out[n, M, c] = input[n, M, c] * weight[i, c] / sqrt(mean_c |x[n, block i, c]|^2 + eps)``
    (reference ``:75-118``)."""
    rsigma = torch.rsqrt(channel_mean_squared_norm(input_tensor, irreps_info, scaled) + eps)
    infos = _broadcast_infos(irreps_info)
    out = sparse_vecsca(input_tensor, rsigma, *infos)
    if weight is not None:
        out = sparse_mul(out, weight, *infos)
    return out
