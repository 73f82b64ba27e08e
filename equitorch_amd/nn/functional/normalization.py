"""RMS normalisation of equivariant features (``equitorch/nn/functional/normalization.py``)."""
import torch
from torch import Tensor
from torch.autograd import Function

from ...ops import kernels
from ...structs import IrrepsInfo
from .activations import _broadcast_infos
from .norm import batch_mean_squared_norm, channel_mean_squared_norm
from .sparse_product import sparse_mul, sparse_vecsca


def batch_rms_norm(input: Tensor, running_squared_norm: Tensor, irreps_info: IrrepsInfo, weight: Tensor = None,
                   scaled: bool = True, training: bool = False, momentum: float = 0.1, eps: float = 1e-05) -> Tensor:
    """``out[n, M, c] = input[n, M, c] * weight[i, c] / sqrt(s[i, c] + eps)`` with ``i`` the irrep of ``M`` and
    ``s`` the batch mean of the per-sample squared norms when ``training`` (then also blended into
    ``running_squared_norm`` in place with ``momentum``), else ``running_squared_norm`` (reference ``:10-72``)."""
    if training:
        stat = batch_mean_squared_norm(input, irreps_info, scaled)      # summed over the batch inside the launch
        running_squared_norm.data.lerp_(stat.detach().to(running_squared_norm.dtype), momentum)
    else:
        stat = running_squared_norm
    scale = torch.rsqrt(stat + eps)
    if weight is not None:
        scale = weight * scale
    return sparse_mul(input, scale, *_broadcast_infos(irreps_info))


def _layer_rms_composed(input_tensor: Tensor, irreps_info: IrrepsInfo, weight: Tensor, scaled: bool, eps: float):
    """The reference's composition (``:111-157``) on the table-driven kernels; differentiable to any order."""
    rsigma = torch.rsqrt(channel_mean_squared_norm(input_tensor, irreps_info, scaled) + eps)
    infos = _broadcast_infos(irreps_info)
    out = sparse_vecsca(input_tensor, rsigma, *infos)
    if weight is not None:
        out = sparse_mul(out, weight, *infos)
    return out


class _LayerRMSFused(Function):
    """One launch per direction (``cgtp_layer_rms_forward`` / ``cgtp_layer_rms_backward``); gradients of higher
    order are taken through the composition above."""

    @staticmethod
    def forward(ctx, x: Tensor, weight, irreps_info: IrrepsInfo, scaled: bool, eps: float):
        need = x.requires_grad or (weight is not None and weight.requires_grad)
        out, rsigma = kernels.layer_rms_forward(x, weight, irreps_info.irrep_seg, irreps_info.rdims, scaled, eps, need)
        ctx.save_for_backward(x, weight, rsigma)
        ctx.irreps_info, ctx.scaled, ctx.eps = irreps_info, scaled, eps
        return out

    @staticmethod
    def backward(ctx, g):
        x, weight, rsigma = ctx.saved_tensors
        need_x, need_w = ctx.needs_input_grad[0], weight is not None and ctx.needs_input_grad[1]
        if torch.is_grad_enabled():
            with torch.enable_grad():
                out = _layer_rms_composed(x, ctx.irreps_info, weight, ctx.scaled, ctx.eps)
                wanted = [t for t, n in ((x, need_x), (weight, need_w)) if n]
                grads = list(torch.autograd.grad(out, wanted, g, create_graph=True))
            gx = grads.pop(0) if need_x else None
            gw = grads.pop(0) if need_w else None
            return gx, gw, None, None, None
        gx, gw = kernels.layer_rms_backward(x, weight, rsigma, g.contiguous(), ctx.irreps_info.irrep_seg,
                                            ctx.irreps_info.rdims, ctx.scaled,
                                            need_x, need_w)
        return gx, gw, None, None, None


def layer_rms_norm(input_tensor: Tensor, irreps_info: IrrepsInfo, weight: Tensor = None, scaled: bool = True,
                   eps: float = 1e-05) -> Tensor:
    """``out[n, M, c] = input[n, M, c] * weight[i, c] / sqrt(mean_c |x[n, block i, c]|^2 + eps)``
    (reference ``:111-157``).  fp32 / fp64 features of up to 256 (128) channels and irreps up to l = 6 run on the
    fused kernels; everything else on the reference's composition of table-driven products."""
    x = input_tensor
    if (x.is_cuda and x.ndim >= 3 and (weight is None or (weight.dtype == x.dtype and weight.ndim == 2))
            and kernels.layer_rms_supported(irreps_info.irrep_seg, x.shape[-1], x.dtype)):
        flat = x.reshape(-1, *x.shape[-2:]).contiguous()
        w = None if weight is None else weight.contiguous()
        return _LayerRMSFused.apply(flat, w, irreps_info, bool(scaled), float(eps)).reshape(x.shape)
    return _layer_rms_composed(input_tensor, irreps_info, weight, scaled, eps)
