"""Fully connected ("uv") products outside the matrix-core kernel's domain (fp32 / fp64, per-sample weights, channel
counts it does not cover): the channel mixing is a plain GEMM per weight path on the library (``torch.matmul``), the
Clebsch-Gordan stage runs on the table-driven contraction kernel.

Weight-first order, as in the matrix-core kernel: ``z[n, q, :] = x[n, a_q, :] @ W[p_q]`` for every (path, input row)
pair ``q`` — one GEMM per input irrep against the side-by-side weights of its paths — then ``out[n, M] = sum_t coef_t * y[n, b_t] * z[n, q_t]``.  Every piece is differentiable (``matmul``,
``cat`` and the closed contraction family of ``_tri``), so gradients of any order come from autograd.  The bf16 case
with a shared weight does not come here (``_uvw_mfma``).  A per-sample weight ``(N, P, C_in, C_out)`` makes the
path GEMMs batched over the samples.
"""
from typing import List, Tuple

import numpy as np
import torch
from torch import Tensor

from ..._lib import OPERAND_NONE, OPERAND_SCALAR, OPERAND_VEC
from ...ops import kernels
from ._tri import TriSpec, tri


class _Plan:
    """Per table and channelled operand: the paths grouped by the input irrep they read, and the contraction of the
    second stage.  The (path, input row) pairs are numbered irrep by irrep, row-major inside an irrep
    (``q = q0 + (a - a0) * paths + path``), which is the layout one GEMM per input irrep produces."""

    def __init__(self, coo, chan_col: np.ndarray, other_col: np.ndarray, other_size: int):
        groups = {}
        for p in range(coo.P):
            rows = np.unique(chan_col[coo.p == p])
            if not (rows.size and np.array_equal(rows, np.arange(rows[0], rows[0] + rows.size))):
                raise ValueError("the rows a path reads must be contiguous (one irrep)")
            groups.setdefault((int(rows[0]), int(rows.size)), []).append(p)
        self.blocks: List[Tuple[int, int, Tuple[int, ...]]] = []      # (first row, rows, paths)
        q_of, q0 = {}, 0
        for (a0, na), paths in sorted(groups.items()):
            for j in range(na):
                for i, p in enumerate(paths):
                    q_of[(p, a0 + j)] = q0 + j * len(paths) + i
            self.blocks.append((a0, na, tuple(paths)))
            q0 += na * len(paths)
        q = np.array([q_of[(int(p), int(a))] for p, a in zip(coo.p, chan_col)], dtype=np.int64)
        self.n_q = q0
        self.spec = TriSpec(coo.M, [q, other_col, None], coo.coef, coo.DO, [q0, other_size, None])


def _plan(tp_info, chan: int) -> _Plan:
    def build():
        coo = kernels.coo_of(tp_info)
        if chan == 1:
            return _Plan(coo, coo.M1, coo.M2, coo.D2)
        return _Plan(coo, coo.M2, coo.M1, coo.D1)
    return kernels.cached(tp_info.info_Mij_fwd.scale, ("uv_gemm", chan), build)


def _mix(x: Tensor, weight: Tensor, plan: _Plan) -> Tensor:
    """``z[n, q, :] = x[n, a_q, :] @ weight[(n,) p_q]``: one GEMM per input irrep, against the weights of all the
    paths that read it laid side by side (``(C_in, paths * C_out)``)."""
    n, cout = x.shape[0], weight.shape[-1]
    pieces = []
    for a0, na, paths in plan.blocks:
        npth = len(paths)
        consecutive = paths == tuple(range(paths[0], paths[0] + npth))
        xs = x[:, a0:a0 + na, :]
        if weight.ndim == 3:
            w = weight[paths[0]:paths[0] + npth] if consecutive else weight[list(paths)]
            w = w.permute(1, 0, 2).reshape(w.shape[1], npth * cout)                  # (C_in, paths * C_out)
        else:
            w = weight[:, paths[0]:paths[0] + npth] if consecutive else weight[:, list(paths)]
            w = w.permute(0, 2, 1, 3).reshape(n, w.shape[2], npth * cout)
        pieces.append(torch.matmul(xs, w).reshape(n, na * npth, cout))
    return torch.cat(pieces, dim=1)


def supported(*tensors: Tensor) -> bool:
    """One floating dtype throughout and a weight ``(P, C_in, C_out)`` or ``(N, P, C_in, C_out)``."""
    dtypes = {t.dtype for t in tensors}
    return len(dtypes) == 1 and next(iter(dtypes)).is_floating_point and tensors[-1].ndim in (3, 4)


def u1v(input1: Tensor, input2: Tensor, weight: Tensor, tp_info) -> Tensor:
    plan = _plan(tp_info, 1)
    return tri(plan.spec, (OPERAND_VEC, OPERAND_SCALAR, OPERAND_NONE), OPERAND_VEC, _mix(input1, weight, plan), input2)


def one_vu(input1: Tensor, input2: Tensor, weight: Tensor, tp_info) -> Tensor:
    plan = _plan(tp_info, 2)
    return tri(plan.spec, (OPERAND_VEC, OPERAND_SCALAR, OPERAND_NONE), OPERAND_VEC, _mix(input2, weight, plan), input1)


def vu1(input1: Tensor, input2: Tensor, weight: Tensor, tp_info) -> Tensor:
    """``out[n, M] = sum_t coef_t * <x[n, a_t, :] @ W[p_t], y[n, b_t, :]>``."""
    plan = _plan(tp_info, 1)
    return tri(plan.spec, (OPERAND_VEC, OPERAND_VEC, OPERAND_NONE), OPERAND_SCALAR, _mix(input1, weight, plan), input2)
