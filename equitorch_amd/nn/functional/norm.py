"""Invariant norms per irrep block (``equitorch/nn/functional/norm.py``).

The reference reduces ``input.pow(2)`` with ``torch_geometric.utils.segment`` and writes each backward by hand;
here the squared norm is the table-driven product of the input with itself, segmented by irrep
(``z[k] = sum_{M in irrep k} x[M] x[M]``), whose gradients of every order come from the contraction kernels' own
autograd closure.  ``scaled`` divides the squared norm by the irrep dimension (the norm by its square root).
"""
import torch
from torch import Tensor
from torch.autograd import Function

from ...structs import IrrepsInfo, SparseProductInfo
from .sparse_product import sparse_inner, sparse_mul, sparse_vecsca


def _block_sum_info(irreps_info: IrrepsInfo) -> SparseProductInfo:
    return SparseProductInfo(seg_out=irreps_info.irrep_seg)


def _flat(input: Tensor) -> Tensor:
    return input.reshape(-1, *input.shape[-2:])


class _BlockSumOfSquares(Function):
    """``z[.., k, ..] = sum_{M in irrep k} x[M]^2`` per channel (``mode 'mul'``), summed over channels (``'inner'``)
    or per channel and summed over rows (``'rows'``).  As a product of ``x`` with itself the gradient would be two
    equal contractions and their sum; it is written here as the one it is, ``2 x[M] g[k(M)]`` — a gate with the
    incoming gradient, again differentiable."""

    @staticmethod
    def forward(ctx, x: Tensor, irreps_info: IrrepsInfo, mode: str):
        ctx.save_for_backward(x)
        ctx.irreps_info, ctx.mode = irreps_info, mode
        info = _block_sum_info(irreps_info)
        if mode == "inner":
            return sparse_inner(x, x, info)
        return sparse_mul(x, x, info, out_accumulated=(mode == "rows"))

    @staticmethod
    def backward(ctx, g):
        (x,) = ctx.saved_tensors
        from .activations import _broadcast_infos
        infos = _broadcast_infos(ctx.irreps_info)
        if ctx.mode == "inner":
            return sparse_vecsca(x, 2 * g, *infos), None, None
        return sparse_mul(x, 2 * g, *infos), None, None


def squared_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """``(..., dim, C) -> (..., num_irreps, C)`` (reference ``SquaredNorm``, ``:15-68``)."""
    x = _flat(input_tensor)
    out = _BlockSumOfSquares.apply(x, irreps_info, "mul")
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
    out = _BlockSumOfSquares.apply(x, irreps_info, "inner") / input_tensor.shape[-1]
    if scaled:
        out = out * irreps_info.rdims
    return out.reshape(*input_tensor.shape[:-2], out.shape[-1])


def batch_mean_squared_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """``(N, dim, C) -> (num_irreps, C)``: squared norm averaged over the batch axis (reference ``:193-255``); the
    sum over rows happens inside the kernel launch (fixed order, no atomics)."""
    out = _BlockSumOfSquares.apply(input_tensor, irreps_info, "rows")
    out = out / input_tensor.shape[0]
    if scaled:
        out = out * irreps_info.rdims.unsqueeze(-1)
    return out
