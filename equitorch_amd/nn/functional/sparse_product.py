"""Differentiable sparse products (the seven members of ``equitorch/nn/functional/sparse_product.py``).

Signatures follow the reference (``sparse_mul`` :71-99, ``sparse_inner`` :211-233, ``sparse_vecsca``
:345-365, ``sparse_scavec`` :412-432, ``sparse_outer`` :101-165, ``sparse_vecmat`` :235-298, ``sparse_mat_t_vec``
:434-500).  ``info_bwd1`` / ``info_bwd2`` are accepted and unused: the gradient
tables are derived from ``info_fwd`` itself.  ``out_accumulated=True`` sums the result over the batch axis.
"""
from typing import Optional

from torch import Tensor

S, V = "", "u"  # channel axes of an operand: none / one
from ...structs import SparseProductInfo
from ._tri import spec_from_product_info, tri


def _size(t: Tensor, axes: str) -> int:
    return t.shape[-1 - len(axes)]


def _binary(k1, k2, ko, input1, input2, info_fwd, out_accumulated):
    spec = spec_from_product_info(info_fwd, _size(input1, k1), _size(input2, k2))
    return tri(spec, (k1, k2, None), ko, input1, input2, None, out_shared=out_accumulated)


def sparse_mul(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
               info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
               out_accumulated: bool = False) -> Tensor:
    """``z[n,M,c] = sum_t s_t x[n,i1_t,c] y[n,i2_t,c]``."""
    return _binary(V, V, V, input1, input2, info_fwd, out_accumulated)


def sparse_inner(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
                 info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
                 out_accumulated: bool = False) -> Tensor:
    """``z[n,M] = sum_t s_t sum_c x[n,i1_t,c] y[n,i2_t,c]``."""
    return _binary(V, V, S, input1, input2, info_fwd, out_accumulated)


def sparse_vecsca(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
                  info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
                  out_accumulated: bool = False) -> Tensor:
    """``z[n,M,c] = sum_t s_t x[n,i1_t,c] y[n,i2_t]``."""
    return _binary(V, S, V, input1, input2, info_fwd, out_accumulated)


def sparse_scavec(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
                  info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
                  out_accumulated: bool = False) -> Tensor:
    """``z[n,M,c] = sum_t s_t x[n,i1_t] y[n,i2_t,c]``."""
    return _binary(S, V, V, input1, input2, info_fwd, out_accumulated)


def sparse_outer(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
                 info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
                 out_accumulated: bool = False) -> Tensor:
    """``z[n,M,u,w] = sum_t s_t x[n,i1_t,u] y[n,i2_t,w]`` (reference ``sparse_product.py:101-165``)."""
    return _binary("u", "w", "uw", input1, input2, info_fwd, out_accumulated)


def sparse_vecmat(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
                  info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
                  out_accumulated: bool = False) -> Tensor:
    """``z[n,M,w] = sum_t s_t sum_u x[n,i1_t,u] Y[(n),i2_t,u,w]`` (reference ``:235-298``)."""
    return _binary("u", "uw", "w", input1, input2, info_fwd, out_accumulated)


def sparse_mat_t_vec(input1: Tensor, input2: Tensor, info_fwd: SparseProductInfo,
                     info_bwd1: Optional[SparseProductInfo] = None, info_bwd2: Optional[SparseProductInfo] = None,
                     out_accumulated: bool = False) -> Tensor:
    """``z[n,M,w] = sum_t s_t sum_u Y[(n),i1_t,u,w] x[n,i2_t,u]``: the matrix ``(.., M1, C_in, C_out)`` first, the vector
    ``(.., M2, C_in)`` second, contracted over the matrix's first channel axis — ``input1.T @ input2`` entry by entry
    (reference ``:434-500``, which calls the vector-matrix product with the operands exchanged,
    ``ops/batched_sparse_dense_op.py:1200-1238``)."""
    return _binary("uw", "u", "w", input1, input2, info_fwd, out_accumulated)
