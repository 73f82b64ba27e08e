"""Tensor products where both operands carry channels (``equitorch/nn/functional/tensor_products.py``).

    uuu : out[n,M,c] = sum_t c_t x[n,M1_t,c] y[n,M2_t,c] W[(n),p_t,c]                 (:9-90)
    uvw : out[n,M,o] = sum_t c_t sum_{u,v} x[n,M1_t,u] y[n,M2_t,v] W[(n),p_t,u,v,o]   (:92-172)
    dot : out[n,k,c] = sum_{M in irrep k} x[n,M,c] y[n,M,c]                           (:173-237)
"""
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
V = "u"  # channel axes of a per-channel operand
from ...ops import kernels
from ...structs import IrrepsInfo, SparseProductInfo, TensorProductInfo
from ._tri import spec_from_tp_info, tri


class _UuuCompiled(Function):
    """uuu on the block-wise kernels with a compiled-in table (``cgtp_uvu_fwd`` / ``cgtp_uvu_bwd`` with
    ``y_channels``); gradients of higher order go through the differentiable table-driven contraction."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info: TensorProductInfo, cfg: int):
        out = kernels.uvu_forward(cfg, kernels.uvu_dims(cfg), x, y, w)
        ctx.save_for_backward(x, y, w)
        ctx.tp_info, ctx.cfg = tp_info, cfg
        return out

    @staticmethod
    def backward(ctx, g):
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        if torch.is_grad_enabled():
            with torch.enable_grad():
                spec = spec_from_tp_info(ctx.tp_info)
                gx = tri(spec.grad_spec(0), (V, V, V), V, g, y, w) if need[0] else None
                gy = tri(spec.grad_spec(1), (V, V, V), V, x, g, w) if need[1] else None
                gw = tri(spec.grad_spec(2), (V, V, V), V, x, y, g, out_shared=(w.ndim == 2)) if need[2] else None
            return gx, gy, gw, None, None
        res = kernels.uvu_backward(ctx.cfg, kernels.uvu_dims(ctx.cfg), x, y, w, g.contiguous(), need)
        return (*res, None, None)


def tensor_product_uuu(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1, C)``, ``input2 (N, D2, C)``, ``weight (P, C) | (N, P, C)`` -> ``(N, DO, C)``."""
    _lib.require_gpu(input1, input2, weight)
    if (input1.ndim == 3 and input2.ndim == 3 and input1.dtype == input2.dtype == weight.dtype == torch.float32
            and input1.shape[-1] == input2.shape[-1]):
        cfg = kernels.uvu_config_of(tp_info_forward)
        x, y, w = input1.contiguous(), input2.contiguous(), weight.contiguous()
        if cfg >= 0 and kernels.uvu_launchable(cfg, x, y, w):
            kernels.log_tier("tensor_product_uuu", "compiled table", f"config {int(cfg)}")
            return _UuuCompiled.apply(x, y, w, tp_info_forward, cfg)
    kernels.log_tier("tensor_product_uuu", "table-driven kernel", str(input1.dtype))
    return tri(spec_from_tp_info(tp_info_forward), (V, V, V), V, input1, input2, weight)


def tensor_product_uvw(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1, C1)``, ``input2 (N, D2, C2)``, ``weight (P, C1, C2, C_out) | (N, P, C1, C2, C_out)`` ->
    ``(N, DO, C_out)``.  Two stages as in the reference (``tensor_products.py:100-101``): the outer products per
    stage-1 segment on the table-driven kernel, then the contraction with the weights as one library GEMM per
    output irrep (``_uvw_gemm``)."""
    _lib.require_gpu(input1, input2, weight)
    if weight.ndim not in (4, 5) or input1.dtype != input2.dtype or input1.dtype != weight.dtype:
        raise _lib.CgtpError(f"tensor_product_uvw: operands {input1.dtype}, {input2.dtype}, {weight.dtype} with "
                             f"weight of {weight.ndim} dims")
    from . import _uv_native, _uvw_gemm
    if _uv_native.uvw_supported(input1, input2, weight, tp_info_forward):
        kernels.log_tier("tensor_product_uvw", "fp32 matrix-core kernel (table-driven)")
        return _uv_native.uvw(input1, input2, weight, tp_info_forward)
    if (weight.ndim == 4 and input1.ndim == 3 and input2.ndim == 3 and input1.dtype in (torch.float32, torch.float64)
            and any(c % 4 for c in weight.shape[1:])):
        # channel counts that are not multiples of 4: zero channels appended to the operands and the weight, the result
        # cut back
        u, v, wc = weight.shape[1:]
        u4, v4, w4 = (-(-c // 4) * 4 for c in (u, v, wc))
        if _uv_native.uvw_fits(input1.shape[0], u4, v4, w4, tp_info_forward, input1.dtype):
            kernels.log_tier("tensor_product_uvw", "channel counts padded to multiples of 4", f"{u} x {v} -> {wc}")
            pad = torch.nn.functional.pad
            out = tensor_product_uvw(pad(input1, (0, u4 - u)), pad(input2, (0, v4 - v)),
                                     pad(weight, (0, w4 - wc, 0, v4 - v, 0, u4 - u)), tp_info_forward)
            return out[..., :wc].contiguous()
    if (input1.dtype in (torch.bfloat16, torch.float16) and input1.ndim == 3 and input2.ndim == 3 and (
            weight.ndim == 5 or _uv_native.uvw_fits(input1.shape[0], weight.shape[1], weight.shape[2], weight.shape[3],
                                                    tp_info_forward, torch.float32))):
        # 16-bit operands: the table-driven kernels in fp32 arithmetic on widened copies, the result rounded once
        kernels.log_tier("tensor_product_uvw", "operands widened to fp32", str(input1.dtype))
        return tensor_product_uvw(input1.float(), input2.float(), weight.float(), tp_info_forward).to(input1.dtype)
    if weight.ndim == 5 and input1.ndim == 3 and input2.ndim == 3:
        from . import _psw
        table = _psw.table_of_coo(kernels.coo_of(tp_info_forward), tp_info_forward.info_Mij_fwd.scale, 1, input1.device)
        w4 = weight.contiguous().flatten(2, 3)
        if _psw.launchable(table, input1, input2, w4):
            kernels.log_tier("tensor_product_uvw", "per-sample weight streaming kernel", str(input1.dtype))
            u, v = weight.shape[2:4]
            return _psw.product(table, input1, input2, w4,
                                lambda x, y, w: _uvw_gemm.uvw(x, y, w.unflatten(2, (u, v)), tp_info_forward))
    kernels.log_tier("tensor_product_uvw", "table-driven outer products + library GEMM", str(input1.dtype))
    return _uvw_gemm.uvw(input1.contiguous(), input2.contiguous(), weight, tp_info_forward)


def tensor_dot_uu(input1: Tensor, input2: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """Irrep-wise, channel-wise dot product ``(..., dim, C), (..., dim, C) -> (..., num_irreps, C)``, divided by
    ``sqrt(2l+1)`` when ``scaled`` (``TensorDotUU``, reference ``:173-223``).  One segmented product on the
    table-driven kernel; its gradients of every order come from that kernel's autograd closure."""
    from .sparse_product import sparse_mul
    _lib.require_gpu(input1, input2)
    lead = torch.broadcast_shapes(input1.shape[:-2], input2.shape[:-2])
    x = input1.expand(*lead, *input1.shape[-2:]).reshape(-1, *input1.shape[-2:])
    y = input2.expand(*lead, *input2.shape[-2:]).reshape(-1, *input2.shape[-2:])
    out = sparse_mul(x, y, SparseProductInfo(seg_out=irreps_info.irrep_seg))
    if scaled:
        out = out * irreps_info.rsqrt_dims.unsqueeze(-1)
    return out.reshape(*lead, *out.shape[-2:])


def tensor_dot_uv(input1: Tensor, input2: Tensor, irreps_info: IrrepsInfo, scaled: bool = True) -> Tensor:
    """Declared but not implemented by the reference (``TensorDotUV``, ``:225-237`` raises); same here."""
    raise NotImplementedError()
