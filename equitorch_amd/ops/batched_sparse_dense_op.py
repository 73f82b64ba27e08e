"""The reference's batched sparse-dense product family (``equitorch/ops/batched_sparse_dense_op.py``) on the
table-driven HIP kernels: the element-wise members below on the single-axis kernel, the matrix members
(outer, vecmat, mat_t_vec; end of file) on the two-axis kernel.

    mul    : z[n,M,c] = sum_t s_t x[n,i1_t,c] y[n,i2_t,c]          (:156-299)
    vecsca : z[n,M,c] = sum_t s_t x[n,i1_t,c] y[n,i2_t]            (:1665-1818)
    scavec : z[n,M,c] = sum_t s_t x[n,i1_t]   y[n,i2_t,c]          (:994-1035)
    inner  : z[n,M]   = sum_t s_t sum_c x[n,i1_t,c] y[n,i2_t,c]    (:713-855)

An operand without its batch axis is shared over the batch; ``out_accumulated`` sums the result over the
batch (gradient of a shared operand).  ``gather_index`` (position inside a segment -> table entry, ``:103-106``)
and ``index_out`` (segment -> output row, ``:138-144``) are never produced by the table builders; they are
honoured by rewriting the table (entries permuted on the way in, result rows placed on the way out).  ``out=`` is
written as the reference's kernels write it: the rows of the segments only, added to when ``out_accumulated``
(``kernel_utils.py:139-155``: an atomic add onto what the tensor holds) and stored otherwise.
"""
from typing import Optional

import torch
from torch import Tensor

from .. import _lib
from .._lib import OPERAND_SCALAR, OPERAND_VEC
from . import kernels


def _gathered(scale, index1, index2, gather_index):
    """The table with its entries read through ``gather_index``: entry t of the new table is entry
    ``gather_index[t]`` of the old one (an operand without an index column is indexed by the entry number)."""
    if gather_index is None:
        return scale, index1, index2
    pick = lambda t: gather_index if t is None else t.index_select(0, gather_index)
    return (None if scale is None else scale.index_select(0, gather_index)), pick(index1), pick(index2)


def _finish(res: Tensor, dim: int, out: Optional[Tensor], out_accumulated: bool, out_size: Optional[int],
            index_out: Optional[Tensor]) -> Tensor:
    """Place the ``n_seg`` result rows: into a fresh zero tensor of ``out_size`` rows (rows past the segments and
    rows no segment names stay zero) or into ``out``, at rows ``0 .. n_seg-1`` or ``index_out``; ``dim`` is the axis
    of ``res`` that runs over the segments."""
    n_seg = res.shape[dim]
    fresh = out is None
    if fresh:
        size = n_seg if out_size is None else int(out_size)
        if index_out is None and size == n_seg:
            return res
        shape = list(res.shape)
        shape[dim] = size
        out = torch.zeros(shape, dtype=res.dtype, device=res.device)
    need = n_seg if index_out is None else (int(index_out.max()) + 1 if index_out.numel() else 0)
    if out.shape[dim] < need:
        raise _lib.CgtpError(f"the output has {out.shape[dim]} rows, the table writes row {need - 1}")
    res = res.to(out.dtype)
    if index_out is None:
        target = out.narrow(dim, 0, n_seg)
        target.add_(res) if (out_accumulated and not fresh) else target.copy_(res)
    elif out_accumulated:
        out.index_add_(dim, index_out, res)
    else:
        out.index_copy_(dim, index_out, res)
    return out


def _product(input1: Tensor, kind1: int, input2: Tensor, kind2: int, scale, index1, index2, seg,
             gather_index, index_out, out, out_accumulated: bool, out_size: Optional[int],
             reduce_c: bool) -> Tensor:
    _lib.require_gpu(input1, input2, scale, index1, index2, seg, gather_index, index_out)
    scale, index1, index2 = _gathered(scale, index1, index2, gather_index)
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
    return _finish(res, 0 if out_accumulated else 1, out, out_accumulated, out_size, index_out)


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
    from ..nn.functional._tri import spec_from_product_info, tri
    from ..structs import SparseProductInfo
    _lib.require_gpu(input1, input2, scale, index1, index2, seg, gather_index, index_out)
    scale, index1, index2 = _gathered(scale, index1, index2, gather_index)
    info = SparseProductInfo(scale, index1, index2, seg, None, None, None)
    size1, size2 = input1.shape[-1 - len(axes1)], input2.shape[-1 - len(axes2)]
    with torch.no_grad():
        res = tri(spec_from_product_info(info, size1, size2), (axes1, axes2, None), out_axes, input1, input2,
                  None, out_shared=out_accumulated)
    batched = res.ndim == 2 + len(out_axes)          # no batch axis when summed over it or when both operands are shared
    return _finish(res, 1 if batched else 0, out, out_accumulated, out_size, index_out)


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
    """``z[n,M,w] = sum_t s_t sum_u Y[(n),i1_t,u,w] x[n,i2_t,u]``: matrix ``(.., M1, C_in, C_out)`` first, vector
    ``(.., M2, C_in)`` second (reference ``:1200-1238``: the vector-matrix product with operands and index columns
    exchanged)."""
    return _matrix_product(input1, "uw", input2, "u", "w", scale, index1, index2, seg, gather_index, index_out,
                           out, out_accumulated, out_size)
