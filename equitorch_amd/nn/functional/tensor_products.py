"""Tensor products where both operands carry channels (``equitorch/nn/functional/tensor_products.py``).

    uuu : out[n,M,c] = sum_t c_t x[n,M1_t,c] y[n,M2_t,c] W[(n),p_t,c]        (:9-90)
"""
from typing import Optional

from torch import Tensor

from ... import _lib
from ..._lib import OPERAND_VEC as V
from ...structs import TensorProductInfo
from ._tri import spec_from_tp_info, tri


def tensor_product_uuu(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1, C)``, ``input2 (N, D2, C)``, ``weight (P, C) | (N, P, C)`` -> ``(N, DO, C)``."""
    _lib.require_gpu(input1, input2, weight)
    return tri(spec_from_tp_info(tp_info_forward), (V, V, V), V, input1, input2, weight)
