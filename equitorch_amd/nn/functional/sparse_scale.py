"""``sparse_scale``: differentiable indexed scale-segment reduction
(``equitorch/nn/functional/sparse_scale.py:14-46``)."""
from typing import Optional

from torch import Tensor
from torch.autograd import Function

from ...ops.indexed_scale_segment_op import indexed_scale_segment
from ...structs import SparseScaleInfo


class SparseScale(Function):
    """``forward(input (N, in_size, C), info_fwd, info_bwd)``; the backward applies ``info_bwd`` (the
    transposed table from ``sparse_scale_infos``) to the incoming gradient."""

    @staticmethod
    def forward(ctx, input, info_fwd, info_bwd):
        ctx.infos = (info_fwd, info_bwd)
        return indexed_scale_segment(input, info_fwd.scale, info_fwd.index, info_fwd.seg_out, info_fwd.out_size)

    @staticmethod
    def backward(ctx, grad_output):
        info_fwd, info_bwd = ctx.infos
        grad_in = None
        if ctx.needs_input_grad[0]:
            if info_bwd is None:
                raise RuntimeError("sparse_scale needs info_bwd to be differentiated")
            grad_in = SparseScale.apply(grad_output, info_bwd, info_fwd)
        return grad_in, None, None


def sparse_scale(input: Tensor, info_fwd: SparseScaleInfo, info_bwd: Optional[SparseScaleInfo] = None) -> Tensor:
    return SparseScale.apply(input, info_fwd, info_bwd)
