"""Constant index / coefficient tables of the sparse Clebsch-Gordan tensor product.

Public names and results follow ``equitorch/utils/_structs.py:22-333`` bit for bit (``int64`` index tensors,
default-dtype ``scale`` tensors created with ``torch.tensor(list_of_python_floats)``, identity index lists and
trivial CSR pointers collapsed to ``None``).  The arithmetic that produces the coefficients differs: exact
rational Clebsch-Gordan values from :mod:`equitorch_amd.constants` instead of a computer-algebra system.
"""
from typing import List, Optional, Tuple

import numpy as np
from torch import tensor

from ..constants import j_matrix, so3_clebsch_gordan
from ..irreps import Irreps, check_irreps, has_path, irrep_segments
from ..structs import (IrrepsInfo, IrrepsLinearInfo, SparseProductInfo, SparseScaleInfo, TensorProductInfo,
                       WignerRotationInfo)
from ._indices import _lex_order, extract_batch_segments, sort_by_column_key


def _csr_pointer(sorted_out: np.ndarray, out_size: Optional[int], shifted: bool):
    """CSR pointer over ``out_size`` output rows for an ascending list of output indices.

    With ``shifted`` the pointer reproduces ``sparse_product_info`` (reference ``:103-121``): there the list of
    run boundaries is left-padded with one zero per empty leading output row *before* it is indexed by the
    running count of non-empty rows, so for a first non-empty row ``z > 0`` the boundary read for the c-th
    non-empty row is the one of run ``c - z`` (or 0).  Rows past the last run repeat the previous pointer.
    """
    n = sorted_out.shape[0]
    change = np.ones(n, dtype=bool)
    change[1:] = sorted_out[1:] != sorted_out[:-1]
    starts = np.flatnonzero(change)
    rows = sorted_out[starts]                      # distinct output rows, ascending
    bounds = np.append(starts, n)                  # run boundaries
    if out_size is None:
        out_size = int(rows.shape[0])
    if shifted and rows[0] != 0:
        bounds = np.concatenate([np.zeros(int(rows[0]), dtype=bounds.dtype), bounds])
    ptr = [0]
    c = 0
    for m in range(out_size):
        if c < rows.shape[0] and rows[c] == m:
            ptr.append(int(bounds[c + 1]))
            c += 1
        else:
            ptr.append(ptr[-1])
    return ptr, out_size


def _is_arange(a: np.ndarray) -> bool:
    return bool(np.array_equal(a, np.arange(a.shape[0])))


def sparse_scale_info(index=None, index_out=None, scale=None, out_size=None) -> SparseScaleInfo:
    """Rows ``(index_out, index[, scale])`` sorted lexicographically and segmented by ``index_out``
    (reference ``:22-71``)."""
    assert index is not None or index_out is not None, "At least one index should be not None"
    n = len(index or index_out)
    idx = np.asarray(index or list(range(n)), dtype=np.int64)
    out = np.asarray(index_out or list(range(n)), dtype=np.int64)
    keys = [out, idx] + ([np.asarray(scale, dtype=np.float64)] if scale is not None else [])
    order = _lex_order(keys)
    out_s, idx_s = out[order], idx[order]
    ptr, out_size = _csr_pointer(out_s, out_size, shifted=False)
    return SparseScaleInfo(
        scale=tensor([scale[i] for i in order]) if scale is not None else None,
        index=None if _is_arange(idx_s) else tensor(idx_s.tolist()),
        seg_out=None if ptr == list(range(out_size + 1)) else tensor(ptr),
        index_out=None,
        out_size=out_size,
    )


def sparse_scale_infos(index=None, index_out=None, scale=None, out_size=None, in_size=None):
    """The table and its transpose (reference ``:73-77``)."""
    return (sparse_scale_info(index, index_out, scale, out_size),
            sparse_scale_info(index_out, index, scale, in_size))


def sparse_product_info(index1=None, index2=None, index=None, scale=None, out_size=None) -> SparseProductInfo:
    """Rows ``(index, index1, index2[, scale])`` sorted lexicographically and segmented by ``index``
    (reference ``:79-138``)."""
    assert index1 is not None or index2 is not None or index is not None, \
        "At least one of the indices should be not None"
    n = len(index1 or index2 or index)
    i1 = np.asarray(index1 or list(range(n)), dtype=np.int64)
    i2 = np.asarray(index2 or list(range(n)), dtype=np.int64)
    io = np.asarray(index or list(range(n)), dtype=np.int64)
    keys = [io, i1, i2] + ([np.asarray(scale, dtype=np.float64)] if scale is not None else [])
    order = _lex_order(keys)
    io_s, i1_s, i2_s = io[order], i1[order], i2[order]
    ptr, out_size = _csr_pointer(io_s, out_size, shifted=True)
    return SparseProductInfo(
        scale=tensor([scale[i] for i in order]) if scale is not None else None,
        index1=None if _is_arange(i1_s) else tensor(i1_s.tolist()),
        index2=None if _is_arange(i2_s) else tensor(i2_s.tolist()),
        seg_out=None if ptr == list(range(out_size + 1)) else tensor(ptr),
        index_out=None,
        out_size=out_size,
    )


def sparse_product_infos(index1=None, index2=None, index=None, scale=None, out_size=None, in1_size=None,
                         in2_size=None):
    """Forward table plus the two tables with the operand roles rotated (reference ``:141-147``)."""
    return (sparse_product_info(index1, index2, index, scale, out_size),
            sparse_product_info(index2, index, index1, scale, in1_size),
            sparse_product_info(index, index1, index2, scale, in2_size))


def generate_fully_connected_tp_paths(irreps_out: Irreps, irreps1: Irreps, irreps2: Irreps):
    """All ``(k, i, j)`` allowed by the selection rule, ``k`` outermost (reference ``:149-159``)."""
    return [(k, i, j)
            for k, ir_out in enumerate(irreps_out)
            for i, ir1 in enumerate(irreps1)
            for j, ir2 in enumerate(irreps2)
            if has_path(ir_out, ir1, ir2)]


def prepare_so3(irreps_out: Irreps, irreps1: Irreps, irreps2: Irreps,
                path: List[Tuple[int, int, int]] = None, path_norm: bool = True,
                channel_norm: bool = False, channel_scale: float = 1.0):
    """COO lists ``(coef, M, M1, M2, k, i, j, w_idx)`` of the non-zero coupling coefficients
    (reference ``:162-216``).  ``path_norm`` folds ``(#paths into output irrep k)**-0.5`` into ``coef`` in
    double precision; the count is the length of the run of consecutive equal ``k`` in ``path``."""
    if not path:
        path = generate_fully_connected_tp_paths(irreps_out, irreps1, irreps2)
    irs_out, irs1, irs2 = list(irreps_out), list(irreps1), list(irreps2)
    off_out, off1, off2 = irrep_segments(irreps_out), irrep_segments(irreps1), irrep_segments(irreps2)

    run = {}
    prev = None
    for k, _, _ in path:
        run[k] = run[k] + 1 if k == prev else 1
        prev = k

    coef, Ms, M1s, M2s, ks, is_, js, ws = ([] for _ in range(8))
    for w, (k, i, j) in enumerate(path):
        cg = so3_clebsch_gordan(irs_out[k].l, irs1[i].l, irs2[j].l)
        norm = (run[k] ** (-0.5) if path_norm else 1.0) * (channel_scale if channel_norm else 1.0)
        km, im, jm = np.nonzero(cg)          # C order: km slowest, jm fastest
        vals = cg[km, im, jm] * norm
        for v, a, b, c in zip(vals.tolist(), km.tolist(), im.tolist(), jm.tolist()):
            if v != 0.0:
                coef.append(v)
                Ms.append(off_out[k] + a)
                M1s.append(off1[i] + b)
                M2s.append(off2[j] + c)
                ks.append(k)
                is_.append(i)
                js.append(j)
                ws.append(w)
    return coef, Ms, M1s, M2s, ks, is_, js, ws, len(path)


def _runs(cols: np.ndarray):
    """(segment id per row, first row of each segment) for row-sorted integer columns ``cols`` (n, ncol)."""
    n = cols.shape[0]
    change = np.ones(n, dtype=bool)
    change[1:] = (cols[1:] != cols[:-1]).any(axis=1)
    return np.cumsum(change) - 1, np.flatnonzero(change)


def create_tp_info(cg_vals, M, M1, M2, k, i, j, w_idx, out_size, in1_size, in2_size) -> TensorProductInfo:
    """All fifteen tables of one direction (reference ``:219-291``).

    ``info_Mij_*``  : stage 1, ``inter[q] = sum_{t in q} coef * x[M1] * y[M2]`` with ``q = (k, M, i, j)``;
    ``info_M_*``    : stage 2, ``out[M] = sum_{q in M} inter[q] * W[w_idx[q]]``;
    ``info_kM1j_*``, ``info_kM1M2_*``, ``info_M_kM1M2_*`` : the weight-first evaluation order.
    """
    cols = np.array([k, M, i, j, M1, M2, w_idx], dtype=np.int64).T
    cg = np.asarray(cg_vals, dtype=np.float64)
    order = np.lexsort([cg] + [cols[:, c] for c in range(cols.shape[1] - 1, -1, -1)])
    cols, cg_sorted = cols[order], [cg_vals[t] for t in order]
    k_s, M_s, i_s, j_s, M1_s, M2_s, w_s = (cols[:, c] for c in range(7))

    q_of_t, q_first = _runs(cols[:, [0, 1, 2, 3, 6]])
    infos_inter = sparse_product_infos(M1_s.tolist(), M2_s.tolist(), q_of_t.tolist(), cg_sorted,
                                       in1_size=in1_size, in2_size=in2_size)
    M_q, w_q = M_s[q_first], w_s[q_first]
    row_of_q, _ = _runs(M_q[:, None])
    infos_M = sparse_product_infos(index2=w_q.tolist(), index=row_of_q.tolist(), out_size=out_size)

    # weight-first order: distinct (k,i,j,M1,M2,w) tuples, then distinct (k,i,M1,j,w) tuples among those
    u5, b5 = np.unique(cols[:, [0, 2, 3, 4, 5, 6]], axis=0, return_inverse=True)
    u4, b4 = np.unique(u5[:, [0, 1, 3, 2, 5]], axis=0, return_inverse=True)
    row_of_t, row_first = _runs(M_s[:, None])
    infos_kM1j = sparse_product_infos(index1=u4[:, 2].tolist(), index2=u4[:, 4].tolist(), in1_size=in1_size)
    infos_kM1M2 = sparse_product_infos(index1=b4.reshape(-1).tolist(), index2=u5[:, 4].tolist(),
                                       in2_size=in2_size)
    infos_M_kM1M2 = sparse_scale_infos(index=b5.reshape(-1).tolist(),
                                       index_out=M_s[row_first][row_of_t].tolist(),
                                       scale=cg_sorted, out_size=out_size)
    return TensorProductInfo(*infos_inter, *infos_M, *infos_kM1j, *infos_kM1M2, *infos_M_kM1M2,
                             out_size=out_size)


def tp_infos(irreps_out, irreps1, irreps2, path: List[Tuple[int, int, int]] = None, path_norm: bool = True,
             channel_norm: bool = False, channel_scale: float = 1.0):
    """``(tp_forward, tp_backward1, tp_backward2, num_paths)`` (reference ``:318-333``).

    ``tp_backward1`` treats ``input1`` as the output (roles ``in1 <- (in2, out)``), ``tp_backward2`` treats
    ``input2`` as the output (``in2 <- (out, in1)``); all three share the forward coefficients.
    """
    irreps_out, irreps1, irreps2 = check_irreps(irreps_out), check_irreps(irreps1), check_irreps(irreps2)
    cg, M, M1, M2, k, i, j, w, num_paths = prepare_so3(irreps_out, irreps1, irreps2, path, path_norm,
                                                       channel_norm, channel_scale)
    do, d1, d2 = irreps_out.dim, irreps1.dim, irreps2.dim
    return (create_tp_info(cg, M, M1, M2, k, i, j, w, do, d1, d2),
            create_tp_info(cg, M1, M2, M, i, j, k, w, d1, d2, do),
            create_tp_info(cg, M2, M, M1, j, k, i, w, d2, do, d1),
            num_paths)


# ---- irreps-preserving channel mixing (IrrepsLinear / IrrepWiseLinear) ---------------------------------------
def generate_fully_connected_irreps_linear_paths(irreps_out: Irreps, irreps_in: Irreps) -> List[Tuple[int, int]]:
    """All ``(i_out, i_in)`` with equal degree and compatible parity (reference ``:336-343``)."""
    return [(i, i0) for i, ir_out in enumerate(irreps_out) for i0, ir_in in enumerate(irreps_in)
            if has_path(ir_out, ir_in)]


def prepare_irreps_linear(irreps_out, irreps_in, path, path_norm, channel_norm, channel_scale: float = 1.0):
    """One entry ``(scale, M, M0, i, i0, path)`` per component of every path (reference ``:346-385``).  The scale
    is ``count(paths into i)^-1/2`` under ``path_norm`` (the Python int ``1`` otherwise, which makes the scale
    tensors integer-typed exactly as in the reference), times ``channel_scale`` under ``channel_norm``."""
    if not path:
        path = generate_fully_connected_irreps_linear_paths(irreps_out, irreps_in)
    seg_out, seg_in = irrep_segments(irreps_out), irrep_segments(irreps_in)
    current, path_count = None, {}
    for i, _ in path:
        path_count[i] = path_count[i] + 1 if i == current else 1
        current = i
    scales, M_s, M0_s, i_s, i0_s, ii0_s = [], [], [], [], [], []
    for w_idx, (i, i0) in enumerate(path):
        norm_scale = path_count[i] ** (-0.5) if path_norm else 1
        if channel_norm:
            norm_scale *= channel_scale
        for m in range(2 * irreps_out[i].l + 1):
            scales.append(norm_scale)
            M_s.append(seg_out[i] + m)
            M0_s.append(seg_in[i0] + m)
            i_s.append(i)
            i0_s.append(i0)
            ii0_s.append(w_idx)
    return scales, M_s, M0_s, i_s, i0_s, ii0_s, len(path)


def create_irreps_linear_info(scales, M_s, M0_s, ii0_s, out_size) -> IrrepsLinearInfo:
    """Reference ``:387-415``: the entries sorted by ``(M, M0, path, scale)`` with the CSR pointer over distinct
    ``M``, and sorted by ``(path, M, M0, scale)`` with the CSR pointer over paths."""
    M_MM0, M0_MM0, ii0_MM0, scales_MM0 = sort_by_column_key([M_s, M0_s, ii0_s, scales])
    _, M_seg_MM0, (M,) = extract_batch_segments([M_MM0])
    ii0_ii0MM0, M_ii0MM0, M0_ii0MM0, scales_ii0MM0 = sort_by_column_key([ii0_s, M_s, M0_s, scales])
    _, ii0_seg_ii0MM0, (_, scales_ii0) = extract_batch_segments([ii0_ii0MM0, scales_ii0MM0])
    return IrrepsLinearInfo(tensor(scales_MM0), tensor(M_seg_MM0), tensor(ii0_MM0), tensor(M0_MM0), tensor(M_MM0),
                            tensor(M), tensor(ii0_seg_ii0MM0), tensor(M_ii0MM0), tensor(M0_ii0MM0),
                            tensor(scales_ii0), out_size)


def irreps_linear_infos(irreps_out, irreps_in, path: List[Tuple[int, int]] = None, path_norm: bool = True,
                        channel_norm: bool = False, channel_scale: float = 1.0):
    """``(forward_info, backward_info, num_paths)`` (reference ``:432-443``); the backward tables exchange the
    roles of input and output components."""
    irreps_out, irreps_in = check_irreps(irreps_out), check_irreps(irreps_in)
    scales, M_s, M0_s, _, _, ii0_s, num_paths = prepare_irreps_linear(irreps_out, irreps_in, path, path_norm,
                                                                      channel_norm, channel_scale)
    return (create_irreps_linear_info(scales, M_s, M0_s, ii0_s, irreps_out.dim),
            create_irreps_linear_info(scales, M0_s, M_s, ii0_s, irreps_in.dim), num_paths)


def irreps_info(irreps) -> IrrepsInfo:
    """Reference ``:446-459``."""
    irreps = check_irreps(irreps)
    seg, idx, rsqrt_dim, rdims, acc = [], [], [], [], 0
    for i, irrep in enumerate(irreps):
        seg.append(acc)
        idx.extend(irrep.dim * [i])
        acc += irrep.dim
        rsqrt_dim.append(irrep.dim ** (-0.5))
        rdims.append(1 / irrep.dim)
    seg.append(acc)
    return IrrepsInfo(tensor(rsqrt_dim), tensor(rdims), tensor(idx), tensor(seg), len(irreps))


# ---- rotations: D(alpha, beta, gamma) = Z(alpha) J Z(beta) J Z(gamma) ------------------------------------------
def _component_index(irreps):
    """``{(irrep index, m): component}`` for ``m = -l..l`` of every irrep."""
    table, at = {}, 0
    for i, ir in enumerate(irreps):
        for m in range(-ir.l, ir.l + 1):
            table[(i, m)] = at
            at += 1
    return table


def prepare_z_rotation(irreps):
    """Entries ``(x index, cs index, output, scale)`` of a rotation about z (reference ``:460-521``):
    ``x'[m] = cos(m phi) x[m] - sign(m) sin(|m| phi) x[-m]`` with ``cs = [1, sin phi, cos phi, sin 2 phi, ...]``;
    ``m = 0`` components are copied."""
    where = _component_index(irreps)
    index1, index2, index_out, scales = [], [], [], []
    for (i, m), M in where.items():
        if m == 0:
            index_out.append(M); scales.append(1.0); index1.append(M); index2.append(0)
        else:
            index_out.append(M); scales.append(1.0); index1.append(M); index2.append(2 * abs(m))
            index_out.append(M); scales.append(-(float(m > 0) - float(m < 0)))
            index1.append(where[(i, -m)]); index2.append(2 * abs(m) - 1)
    return index1, index2, index_out, scales, 1 + 2 * max((ir.l for ir in irreps), default=0)


def z_rotation_infos(irreps):
    """``(forward, gradient of x, gradient of cs)`` product tables of the z rotation (reference ``:536-585``)."""
    irreps = check_irreps(irreps)
    index1, index2, index_out, scales, cs_dim = prepare_z_rotation(irreps)
    return sparse_product_infos(index1=index1, index2=index2, index=index_out, scale=scales, out_size=irreps.dim,
                                in1_size=irreps.dim, in2_size=cs_dim)


def j_matrix_info(irreps) -> SparseScaleInfo:
    """Block-diagonal ``J`` as a sparse scale table; entries below 1e-9 are dropped (reference ``:587-636``)."""
    irreps = check_irreps(irreps)
    index_in, index_out, scales, offset = [], [], [], 0
    for ir in irreps:
        block = j_matrix(ir.l)
        for row in range(ir.dim):
            for col in range(ir.dim):
                if abs(block[row, col]) > 1e-9:
                    index_out.append(offset + row)
                    index_in.append(offset + col)
                    scales.append(float(block[row, col]))
        offset += ir.dim
    return sparse_scale_info(index=index_in, index_out=index_out, scale=scales, out_size=irreps.dim)


def wigner_d_info(irreps) -> WignerRotationInfo:
    """Reference ``:638-654``.  ``sign`` holds ``p^l`` twice per irrep, as the reference's comprehension over the
    ``(l, p)`` pair of every irrep produces it."""
    irreps = check_irreps(irreps)
    fwd, bwd_x, bwd_cs = z_rotation_infos(irreps)
    sign = [ir.p ** ir.l for ir in irreps for _ in range(2)]
    return WignerRotationInfo(j_matrix_info=j_matrix_info(irreps), rotate_z_info_fwd=fwd,
                              rotate_z_info_bwd_input=bwd_x, rotate_z_info_bwd_cs=bwd_cs,
                              max_m=max(ir.l for ir in irreps), sign=tensor(sign))


# ---- SO(2) linear layer (features in the frame where the edge points along z) -----------------------------------
def prepare_so2_linear(irreps_out, irreps_in, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """Entries of ``SO2Linear`` (reference ``:674-778``).  A path ``(k, i)`` carries one weight for ``m = 0`` and two
    (``w_-``, ``w_+``) for every ``0 < m <= min(l_k, l_i)``:

        out[+m] += s (w_+ x[+m] - w_- x[-m]),      out[-m] += s (w_+ x[-m] + w_- x[+m]),     s = 1 / sqrt(2 n),

    ``out[0] += x[0] w_0 / sqrt(n0)``, where ``n0`` counts the paths into ``(k, 0)`` and — following the reference's
    bookkeeping, which looks the running count up under ``(k, -m)`` while storing it under ``(k, m)`` — ``n`` is 1
    for every ``m > 0``."""
    if path is None:
        path = [(k, i) for k in range(len(irreps_out)) for i in range(len(irreps_in))]
    where_in, where_out = _component_index(irreps_in), _component_index(irreps_out)
    weight_of, count = {}, {}
    for k, i in path:
        for m in range(min(irreps_out[k].l, irreps_in[i].l) + 1):
            if m == 0:
                weight_of[(k, i, 0)] = len(weight_of)
                count[(k, 0)] = count.get((k, 0), 0) + 1
            else:
                weight_of[(k, i, -m)] = len(weight_of)
                weight_of[(k, i, m)] = len(weight_of)
                count[(k, m)] = count.get((k, -m), 0) + 1
    index1, index2, index_out, scales = [], [], [], []

    def entry(out, inp, w, s):
        index_out.append(out); index1.append(inp); index2.append(w); scales.append(s)

    for k, i in path:
        for m in range(min(irreps_out[k].l, irreps_in[i].l) + 1):
            if m == 0:
                entry(where_out[(k, 0)], where_in[(i, 0)], weight_of[(k, i, 0)],
                      count[(k, 0)] ** (-0.5) if path_norm else 1.0)
                continue
            s = (count[(k, m)] * 2) ** (-0.5) if path_norm else 2 ** (-0.5)
            entry(where_out[(k, m)], where_in[(i, m)], weight_of[(k, i, m)], s)
            entry(where_out[(k, -m)], where_in[(i, -m)], weight_of[(k, i, m)], s)
            entry(where_out[(k, m)], where_in[(i, -m)], weight_of[(k, i, -m)], -s)
            entry(where_out[(k, -m)], where_in[(i, m)], weight_of[(k, i, -m)], s)
    if channel_norm:
        scales = [s * channel_scale for s in scales]
    return index1, index2, index_out, scales, len(weight_of)


def so2_linear_infos(irreps_out, irreps_in, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """``(forward, backward1, backward2, num_weights)`` (reference ``:784-786``)."""
    irreps_out, irreps_in = check_irreps(irreps_out), check_irreps(irreps_in)
    index1, index2, index_out, scales, n = prepare_so2_linear(irreps_out, irreps_in, path, path_norm, channel_norm,
                                                              channel_scale)
    return (*sparse_product_infos(index1, index2, index_out, scales, irreps_out.dim, irreps_in.dim, n), n)


def so2_linear_info(irreps_out, irreps_in, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """``(forward table, num_weights)`` (reference ``:780-782``)."""
    irreps_out, irreps_in = check_irreps(irreps_out), check_irreps(irreps_in)
    index1, index2, index_out, scales, n = prepare_so2_linear(irreps_out, irreps_in, path, path_norm, channel_norm,
                                                              channel_scale)
    return sparse_product_info(index1, index2, index_out, scales, irreps_out.dim), n


def irreps_blocks_infos(irreps):
    """Tables of the block-diagonal action of one dense ``(2l+1, 2l+1)`` matrix per irrep on a feature
    (reference ``:656-671``): entry ``q`` multiplies matrix element ``q`` (blocks laid out one after the other,
    row-major) with input component ``M_in`` into output component ``M_out``."""
    irreps = check_irreps(irreps)
    index_in, index_out, first = [], [], 0
    for ir in irreps:
        for m_out in range(first, first + ir.dim):
            for m_in in range(first, first + ir.dim):
                index_in.append(m_in)
                index_out.append(m_out)
        first += ir.dim
    return sparse_product_infos(list(range(len(index_in))), index_in, index_out)
