"""Invariant norms per irrep block (``equitorch/nn/functional/norm.py``).

The reference reduces ``input.pow(2)`` with ``torch_geometric.utils.segment`` and writes each backward by hand;
here the squared norm is the table-driven product of the input with itself, segmented by irrep
(``z[k] = sum_{M in irrep k} x[M] x[M]``), whose gradients of every order come from the contraction kernels' own
autograd closure.  ``scaled`` divides the squared norm by the irrep dimension (the norm by its square root).
"""
import torch
from torch import Tensor

from ...structs import IrrepsInfo, SparseProductInfo
from .sparse_product import sparse_inner, sparse_mul


def _block_sum_info(irreps_info: IrrepsInfo) -> SparseProductInfo:
    return SparseProductInfo(seg_out=irreps_info.irrep_seg)


def _flat(input: Tensor) -> Tensor:
    return input.reshape(-1, *input.shape[-2:])


def squared_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """``(..., dim, C) -> (..., num_irreps, C)`` (reference ``SquaredNorm``, ``:15-68``)."""
    x = _flat(input_tensor)
    out = sparse_mul(x, x, _block_sum_info(irreps_info))
    if scaled:
        out = out * irreps_info.rdims.unsqueeze(-1)
    return out.reshape(*input_tensor.shape[:-2], *out.shape[-2:])


def norm(input_tensor: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """``sqrt`` of the unscaled squared norm, times ``dim^-1/2`` when ``scaled`` (reference ``Norm``, ``:71-129``).
    The gradient at a zero block is zero, as in the reference."""
    sq = squared_norm(input_tensor, irreps_info, scaled=False)
    positive = sq > 0
    out = torch.where(positive, torch.sqrt(torch.where(positive, sq, torch.ones_like(sq))), torch.zeros_like(sq))
    if scaled:
        out = out * irreps_info.rsqrt_dims.unsqueeze(-1)
    return out


def channel_mean_squared_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """``(..., dim, C) -> (..., num_irreps)``: squared norm averaged over channels (reference ``:132-190``)."""
    x = _flat(input_tensor)
    out = sparse_inner(x, x, _block_sum_info(irreps_info)) / input_tensor.shape[-1]
    if scaled:
        out = out * irreps_info.rdims
    return out.reshape(*input_tensor.shape[:-2], out.shape[-1])


def batch_mean_squared_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """``(N, dim, C) -> (num_irreps, C)``: squared norm averaged over the batch axis (reference ``:193-255``); the
    sum over rows happens inside the kernel launch (fixed order, no atomics)."""
    out = sparse_mul(input_tensor, input_tensor, _block_sum_info(irreps_info), out_accumulated=True)
    out = out / input_tensor.shape[0]
    if scaled:
        out = out * irreps_info.rdims.unsqueeze(-1)
    return out
