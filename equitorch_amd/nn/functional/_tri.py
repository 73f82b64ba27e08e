"""Autograd wrapper of the table-driven trilinear kernel.

``out[r, o, (c)] = sum_t coef_t * A[r, ia_t, (c)] * B[r, ib_t, (c)] * W[r, iw_t, (c)]`` is linear in each
operand, and its gradient with respect to one operand is the same contraction with that operand's index
column exchanged with the output column and the operand replaced by the incoming gradient.  The family is
therefore closed under differentiation: ``TriContract.backward`` calls ``TriContract`` again, which gives
gradients of every order without saving any intermediate (the reference reaches the same closure through
its sibling Functions and rotated tables, ``equitorch/nn/functional/sparse_product.py``,
``equitorch/nn/functional/linears.py:44-83``).
"""
from __future__ import annotations

from typing import Optional, Sequence, Tuple

import numpy as np
import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
from ..._lib import OPERAND_NONE, OPERAND_SCALAR, OPERAND_VEC
from ..._tables import pack_tri_table
from ...ops import kernels


class TriSpec:
    """COO description of a trilinear contraction: per non-zero the output index and one index per operand
    slot (``None`` for an absent slot), plus the size of every index space."""

    def __init__(self, out_idx, idx: Sequence[Optional[np.ndarray]], coef: Optional[np.ndarray], out_size: int,
                 sizes: Sequence[Optional[int]]):
        self.out_idx = np.asarray(out_idx, dtype=np.int64)
        self.idx = [None if i is None else np.asarray(i, dtype=np.int64) for i in idx]
        self.coef = None if coef is None else np.asarray(coef, dtype=np.float64)
        self.out_size = int(out_size)
        self.sizes = list(sizes)
        self._grad = {}
        self._packed = {}

    def grad_spec(self, slot: int) -> "TriSpec":
        """Contraction that yields the gradient w.r.t. operand ``slot`` (that slot then carries grad_out)."""
        if slot not in self._grad:
            idx = list(self.idx)
            sizes = list(self.sizes)
            idx[slot], sizes[slot] = self.out_idx, self.out_size
            self._grad[slot] = TriSpec(self.idx[slot], idx, self.coef, self.sizes[slot], sizes)
        return self._grad[slot]

    def packed(self, dtype: torch.dtype, device) -> dict:
        key = (dtype, str(device))
        if key not in self._packed:
            self._packed[key] = pack_tri_table(self.out_idx, self.idx[0], self.idx[1], self.idx[2], self.coef,
                                               self.out_size, dtype, device)
        return self._packed[key]


def _is_shared(t: Tensor, kind: int) -> bool:
    return t.ndim == (2 if kind == OPERAND_VEC else 1)


class TriContract(Function):
    """forward(spec, kinds, out_kind, out_shared, a, b, w) -> out; tensors with kind NONE are passed as None."""

    @staticmethod
    def forward(ctx, spec: TriSpec, kinds: Tuple[int, int, int], out_kind: int, out_shared: bool,
                a: Optional[Tensor], b: Optional[Tensor], w: Optional[Tensor]):
        ops = [a, b, w]
        present = [t for t, k in zip(ops, kinds) if k != OPERAND_NONE]
        _lib.require_gpu(*present)
        dtype = present[0].dtype
        for t in present[1:]:
            dtype = torch.promote_types(dtype, t.dtype)
        device = present[0].device
        ops = [None if k == OPERAND_NONE else t.to(dtype).contiguous() for t, k in zip(ops, kinds)]
        n_rows, channels = None, None
        for t, k in zip(ops, kinds):
            if k == OPERAND_NONE:
                continue
            if not _is_shared(t, k):
                if n_rows not in (None, t.shape[0]):
                    raise _lib.CgtpError(f"batch size mismatch: {n_rows} vs {t.shape[0]}")
                n_rows = t.shape[0]
            if k == OPERAND_VEC:
                if channels not in (None, t.shape[-1]):
                    raise _lib.CgtpError(f"channel mismatch: {channels} vs {t.shape[-1]}")
                channels = t.shape[-1]
        any_batched = n_rows is not None
        n_rows = 1 if n_rows is None else n_rows
        if channels is None:
            raise _lib.CgtpError("at least one operand must carry a channel axis")
        out = kernels.tri_contract(spec.packed(dtype, device), spec.out_size,
                                   (ops[0], kinds[0]), (ops[1], kinds[1]), (ops[2], kinds[2]),
                                   n_rows, channels, dtype, device,
                                   reduce_c=(out_kind == OPERAND_SCALAR), reduce_rows=out_shared)
        if not out_shared and not any_batched:
            out = out.squeeze(0)  # every operand shared -> result has no batch axis either
        ctx.spec, ctx.kinds, ctx.out_kind, ctx.out_shared = spec, kinds, out_kind, out_shared
        ctx.shared = [k != OPERAND_NONE and _is_shared(t, k) for t, k in zip(ops, kinds)]
        ctx.save_for_backward(*[t for t in ops if t is not None])
        ctx.present = [t is not None for t in ops]
        return out

    @staticmethod
    def backward(ctx, g):
        saved = list(ctx.saved_tensors)
        ops = [saved.pop(0) if p else None for p in ctx.present]
        grads = [None, None, None]
        for s in range(3):
            if ctx.kinds[s] == OPERAND_NONE or not ctx.needs_input_grad[4 + s]:
                continue
            new_ops = list(ops)
            new_kinds = list(ctx.kinds)
            new_ops[s], new_kinds[s] = g, ctx.out_kind
            grads[s] = TriContract.apply(ctx.spec.grad_spec(s), tuple(new_kinds), ctx.kinds[s], ctx.shared[s],
                                         *new_ops)
        return (None, None, None, None, *grads)


def tri(spec: TriSpec, kinds, out_kind, a, b, w=None, out_shared=False) -> Tensor:
    return TriContract.apply(spec, tuple(kinds), out_kind, out_shared, a, b, w)


# ---- spec builders -------------------------------------------------------------------------------------------
def spec_from_product_info(info, size1: int, size2: int) -> TriSpec:
    """``SparseProductInfo`` -> two-operand spec (slot w absent); cached on the info's anchor tensor."""
    anchor = next((t for t in (info.seg_out, info.index1, info.index2, info.scale) if t is not None), None)

    def build():
        n = None
        for t in (info.index1, info.index2, info.scale):
            if t is not None:
                n = t.shape[0]
                break
        if n is None:
            n = int(info.seg_out[-1]) if info.seg_out is not None else size1
        ident = np.arange(n, dtype=np.int64)
        i1 = ident if info.index1 is None else info.index1.detach().cpu().numpy()
        i2 = ident if info.index2 is None else info.index2.detach().cpu().numpy()
        if info.seg_out is None:
            out_idx, n_out = ident, n
        else:
            s = info.seg_out.detach().cpu().numpy().astype(np.int64)
            n_out = s.shape[0] - 1
            out_idx = np.repeat(np.arange(n_out, dtype=np.int64), np.diff(s))
        if info.out_size is not None:
            n_out = max(n_out, int(info.out_size))
        coef = None if info.scale is None else info.scale.detach().cpu().numpy().astype(np.float64)
        return TriSpec(out_idx, [i1, i2, None], coef, n_out, [size1, size2, None])

    if anchor is None:
        return build()
    return kernels.cached(anchor, ("spec2", id(info.scale), id(info.index1), id(info.index2), id(info.seg_out),
                                   size1, size2, info.out_size), build)


def spec_from_tp_info(tp_info) -> TriSpec:
    """Fused tensor product ``out[M] = sum coef * in1[M1] * in2[M2] * W[p]`` of one ``TensorProductInfo``."""
    def build():
        c = kernels.coo_of(tp_info)
        return TriSpec(c.M, [c.M1, c.M2, c.p], c.coef, c.DO, [c.D1, c.D2, c.P])
    return kernels.cached(tp_info.info_Mij_fwd.scale, "spec3", build)
