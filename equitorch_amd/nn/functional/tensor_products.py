"""Tensor products where both operands carry channels (``equitorch/nn/functional/tensor_products.py``).

    uuu : out[n,M,c] = sum_t c_t x[n,M1_t,c] y[n,M2_t,c] W[(n),p_t,c]                 (:9-90)
    uvw : out[n,M,o] = sum_t c_t sum_{u,v} x[n,M1_t,u] y[n,M2_t,v] W[(n),p_t,u,v,o]   (:92-172)
"""
from typing import Optional

from torch import Tensor

from ... import _lib
V = "u"  # channel axes of a per-channel operand
from ...structs import TensorProductInfo
from ._tri import spec_from_tp_info, tri


def tensor_product_uuu(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1, C)``, ``input2 (N, D2, C)``, ``weight (P, C) | (N, P, C)`` -> ``(N, DO, C)``."""
    _lib.require_gpu(input1, input2, weight)
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
    from . import _uvw_gemm
    return _uvw_gemm.uvw(input1.contiguous(), input2.contiguous(), weight, tp_info_forward)
