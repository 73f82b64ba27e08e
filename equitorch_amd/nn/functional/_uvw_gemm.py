"""Fully connected product with channels on both operands (``TensorProduct('uvw')``) as the reference's two stages,
with the second stage on library GEMMs.

Stage 1 (table-driven contraction kernel): ``inter[n, q, u, v] = sum_{t in q} coef_t x[n, M1_t, u] y[n, M2_t, v]`` for
every (output row M, path p) pair ``q``.  The pairs are enumerated output irrep by output irrep, row-major inside an
irrep (``q = q0 + (M - M0) * paths + path``), so that stage 2 is one GEMM per output irrep,

    out[n, M0 + j, :] = inter[n, q0 + j * paths : q0 + (j + 1) * paths, :, :].flatten() @ W[(n,) p0 : p0 + paths].flatten(0, 2)

with ``K = paths * U * V`` — a view on both operands when the irrep's paths are consecutive in the weight, as they
are for the default path list.  Both stages are differentiable (the closed contraction family of ``_tri``,
``matmul``), so gradients of every order come from autograd; the gradient of a shared weight is a GEMM and not a
row-by-row reduction.
"""
from typing import List, NamedTuple, Tuple

import numpy as np
import torch
from torch import Tensor

from ...ops import kernels
from ._tri import TriSpec, tri


class _Block(NamedTuple):
    m0: int                 # first output row
    k: int                  # rows (2l+1)
    q0: int                 # first stage-1 row
    paths: Tuple[int, ...]  # weight indices, in the order the stage-1 rows interleave them


class _Plan:
    def __init__(self, coo):
        rows_of = {}
        for p in range(coo.P):
            rows = np.unique(coo.M[coo.p == p])
            if not (rows.size and np.array_equal(rows, np.arange(rows[0], rows[0] + rows.size))):
                raise ValueError("the output rows of a path must be contiguous (one irrep)")
            rows_of.setdefault((int(rows[0]), int(rows.size)), []).append(p)
        self.blocks: List[_Block] = []
        q_of, q0 = {}, 0
        for (m0, k), paths in sorted(rows_of.items()):
            for j in range(k):
                for i, p in enumerate(paths):
                    q_of[(p, m0 + j)] = q0 + j * len(paths) + i
            self.blocks.append(_Block(m0, k, q0, tuple(paths)))
            q0 += k * len(paths)
        end = 0
        for b in self.blocks:
            if b.m0 < end:
                raise ValueError("output irreps of different paths overlap")
            end = b.m0 + b.k
        self.n_q, self.out_size = q0, coo.DO
        q = np.array([q_of[(int(p), int(m))] for p, m in zip(coo.p, coo.M)], dtype=np.int64)
        self.spec = TriSpec(q, [coo.M1, coo.M2, None], coo.coef, q0, [coo.D1, coo.D2, None])


def _plan(tp_info) -> _Plan:
    return kernels.cached(tp_info.info_Mij_fwd.scale, "uvw_gemm", lambda: _Plan(kernels.coo_of(tp_info)))


def uvw(input1: Tensor, input2: Tensor, weight: Tensor, tp_info) -> Tensor:
    plan = _plan(tp_info)
    n = input1.shape[0]
    inter = tri(plan.spec, ("u", "w", None), "uw", input1, input2)           # (N, n_q, U, V)
    uv, cout = weight.shape[-3] * weight.shape[-2], weight.shape[-1]
    shared = weight.ndim == 4
    pieces, at = [], 0
    for b in plan.blocks:
        if b.m0 > at:
            pieces.append(inter.new_zeros(n, b.m0 - at, cout))
        npk = len(b.paths)
        lhs = inter[:, b.q0:b.q0 + b.k * npk].reshape(n, b.k, npk * uv)
        consecutive = b.paths == tuple(range(b.paths[0], b.paths[0] + npk))
        if shared:
            w = weight[b.paths[0]:b.paths[0] + npk] if consecutive else weight[list(b.paths)]
            pieces.append(torch.matmul(lhs, w.reshape(npk * uv, cout)))
        else:
            w = weight[:, b.paths[0]:b.paths[0] + npk] if consecutive else weight[:, list(b.paths)]
            pieces.append(torch.matmul(lhs, w.reshape(n, npk * uv, cout)))
        at = b.m0 + b.k
    if at < plan.out_size:
        pieces.append(inter.new_zeros(n, plan.out_size - at, cout))
    return torch.cat(pieces, dim=1)
