"""The reference's batched sparse-dense product family (``equitorch/ops/batched_sparse_dense_op.py``) on the
table-driven HIP kernels: the element-wise members below on the single-axis kernel, the matrix members
(outer, vecmat, mat_t_vec; end of file) on the two-axis kernel.

    mul    : z[n,M,c] = sum_t s_t x[n,i1_t,c] y[n,i2_t,c]          (:156-299)
    vecsca : z[n,M,c] = sum_t s_t x[n,i1_t,c] y[n,i2_t]            (:1665-1818)
    scavec : z[n,M,c] = sum_t s_t x[n,i1_t]   y[n,i2_t,c]          (:994-1035)
    inner  : z[n,M]   = sum_t s_t sum_c x[n,i1_t,c] y[n,i2_t,c]    (:713-855)

An operand without its batch axis is shared over the batch; ``out_accumulated`` sums the result over the
batch (gradient of a shared operand).  ``gather_index`` / ``index_out`` are never produced by the table
builders and are rejected.
"""
from typing import Optional

import torch
from torch import Tensor

from .. import _lib
from .._lib import OPERAND_SCALAR, OPERAND_VEC
from . import kernels


def _product(input1: Tensor, kind1: int, input2: Tensor, kind2: int, scale, index1, index2, seg,
             gather_index, index_out, out, out_accumulated: bool, out_size: Optional[int],
             reduce_c: bool) -> Tensor:
    if gather_index is not None or index_out is not None:
        raise NotImplementedError("gather_index / index_out tables are not supported")
    _lib.require_gpu(input1, input2, scale, index1, index2, seg)
    dtype = torch.result_type(input1, input2)
    input1, input2 = input1.to(dtype).contiguous(), input2.to(dtype).contiguous()
    full1 = 3 if kind1 == OPERAND_VEC else 2
    full2 = 3 if kind2 == OPERAND_VEC else 2
    shared1, shared2 = input1.ndim == full1 - 1, input2.ndim == full2 - 1
    n_rows = 1
    if not shared1:
        n_rows = input1.shape[0]
    if not shared2:
        n_rows = max(n_rows, input2.shape[0])
    if not shared1 and not shared2 and input1.shape[0] != input2.shape[0]:
        raise _lib.CgtpError("batch sizes of the two operands differ")
    vec = input1 if kind1 == OPERAND_VEC else input2
    channels = vec.shape[-1]
    sparse1 = input1.shape[-2] if kind1 == OPERAND_VEC else input1.shape[-1]
    n_entries = (index1.shape[0] if index1 is not None else index2.shape[0] if index2 is not None
                 else scale.shape[0] if scale is not None else sparse1)
    if scale is not None:
        scale = scale.to(dtype)
    table, n_seg = kernels.product_tri_table(scale, index1, index2, seg, n_entries, dtype, input1.device)
    res = kernels.tri_contract(table, n_seg, (input1, kind1), (input2, kind2), (None, 0), n_rows, channels,
                               dtype, input1.device, reduce_c=reduce_c, reduce_rows=out_accumulated)
    if out_size is not None and out_size != n_seg:
        sparse_dim = 0 if out_accumulated else 1
        shape = list(res.shape)
        shape[sparse_dim] = out_size
        full = torch.zeros(shape, dtype=res.dtype, device=res.device)
        full.narrow(sparse_dim, 0, min(n_seg, out_size)).copy_(res.narrow(sparse_dim, 0, min(n_seg, out_size)))
        res = full
    if out is not None:
        out.copy_(res)
        return out
    return res


def indexed_mul_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                             gather_index=None, index_out=None, out=None, out_accumulated=False,
                             out_size=None, block_size_n=64, block_size_c=64, num_stages=2):
    return _product(input1, OPERAND_VEC, input2, OPERAND_VEC, scale, index1, index2, seg, gather_index,
                    index_out, out, out_accumulated, out_size, reduce_c=False)


def indexed_vecsca_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                                gather_index=None, index_out=None, out=None, out_accumulated=False,
                                out_size=None, block_size_n=64, block_size_c=64, num_stages=2):
    return _product(input1, OPERAND_VEC, input2, OPERAND_SCALAR, scale, index1, index2, seg, gather_index,
                    index_out, out, out_accumulated, out_size, reduce_c=False)


def indexed_scavec_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                                gather_index=None, index_out=None, out=None, out_accumulated=False,
                                out_size=None, block_size_n=64, block_size_c=64, num_stages=2):
    if input1.ndim >= 2 and input1.shape[-1] == 1 and input1.ndim == input2.ndim:
        input1 = input1.squeeze(-1)  # (N, M1, 1) form of the scalar operand
    return _product(input1, OPERAND_SCALAR, input2, OPERAND_VEC, scale, index1, index2, seg, gather_index,
                    index_out, out, out_accumulated, out_size, reduce_c=False)


def indexed_inner_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                               gather_index=None, index_out=None, out=None, out_accumulated=False,
                               out_size=None, block_size_n=32, block_size_c=32, num_stages=2,
                               loop_unroll_factor=4):
    return _product(input1, OPERAND_VEC, input2, OPERAND_VEC, scale, index1, index2, seg, gather_index,
                    index_out, out, out_accumulated, out_size, reduce_c=True)


def _matrix_product(input1, axes1, input2, axes2, out_axes, scale, index1, index2, seg, gather_index, index_out,
                    out, out_accumulated, out_size):
    """Matrix members of the family on the two-axis contraction kernel (no autograd at this layer)."""
    if gather_index is not None or index_out is not None:
        raise NotImplementedError("gather_index / index_out tables are not supported")
    from ..nn.functional._tri import spec_from_product_info, tri
    from ..structs import SparseProductInfo
    info = SparseProductInfo(scale, index1, index2, seg, None, None, out_size)
    size1, size2 = input1.shape[-1 - len(axes1)], input2.shape[-1 - len(axes2)]
    with torch.no_grad():
        res = tri(spec_from_product_info(info, size1, size2), (axes1, axes2, None), out_axes, input1, input2,
                  None, out_shared=out_accumulated)
    if out is not None:
        out.copy_(res)
        return out
    return res


def indexed_outer_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                               gather_index=None, index_out=None, out=None, out_accumulated=False,
                               out_size=None, block_size_n=8, block_size_c1=32, block_size_c2=32, num_stages=2):
    """``z[n,M,c1,c2] = sum_t s_t x[n,i1_t,c1] y[n,i2_t,c2]`` (reference ``:436-579``)."""
    return _matrix_product(input1, "u", input2, "w", "uw", scale, index1, index2, seg, gather_index, index_out,
                           out, out_accumulated, out_size)


def indexed_vecmat_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                                gather_index=None, index_out=None, out=None, out_accumulated=False,
                                out_size=None, block_size_n=8, block_size_c_out=32, block_size_c_in=32,
                                num_stages=1, loop_unroll_factor=4):
    """``z[n,M,w] = sum_t s_t sum_u x[n,i1_t,u] Y[(n),i2_t,u,w]`` (reference ``:1383-1534``)."""
    return _matrix_product(input1, "u", input2, "uw", "w", scale, index1, index2, seg, gather_index, index_out,
                           out, out_accumulated, out_size)


def indexed_mat_t_vec_scale_gather(input1, input2, scale=None, index1=None, index2=None, seg=None,
                                   gather_index=None, index_out=None, out=None, out_accumulated=False,
                                   out_size=None, block_size_n=8, block_size_c_out=32, block_size_c_in=32,
                                   num_stages=1, loop_unroll_factor=4):
    """``z[n,M,u] = sum_t s_t sum_w Y[(n),i1_t,u,w] x[n,i2_t,w]`` (reference ``:1200-1238``)."""
    return _matrix_product(input1, "uw", input2, "w", "u", scale, index1, index2, seg, gather_index, index_out,
                           out, out_accumulated, out_size)
