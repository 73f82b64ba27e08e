"""TEST INFRASTRUCTURE ONLY: list-based restatement of the reference's constant-table construction.

Each function names the reference lines it follows.  Tables are returned as plain Python structures
(``dict`` of lists / ``None`` / ints) so a comparison against either the golden fixtures or the product's
tensors is a bit-for-bit list comparison; ``scale`` lists hold Python doubles and are rounded to fp32 by the
caller exactly as ``torch.tensor(list)`` does in the reference.

Pinned by: ``tests/golden/tp_tables.npz`` and ``tests/golden/scale_tables.npz`` (written by the reference's
own ``tp_infos`` / ``sparse_scale_infos``), closed-form path/nnz counts, and hand-checked tiny cases
(tests/test_tables.py).
"""
import bisect

from . import ref_constants

_P = {"e": 1, "o": -1, "": 0}


# ---- irreps (equitorch/irreps/__init__.py:161-207, 220-238, 558-584, 889-921) --------------------------
def parse(irreps):
    """'2x0e+1o' or (lo, hi) -> expanded list of (l, p)."""
    if isinstance(irreps, tuple):
        return [(l, 0) for l in range(irreps[0], irreps[1] + 1)]
    out = []
    for term in irreps.replace(" ", "").split("+"):
        if not term:
            continue
        mul, _, ir = term.rpartition("x")
        par = ir[-1] if ir[-1] in "eo" else ""
        l = int(ir[:-1] if par else ir)
        out.extend([(l, _P[par])] * (int(mul) if mul else 1))
    return out


def has_path(out, a, b):
    return abs(a[0] - b[0]) <= out[0] <= a[0] + b[0] and (out[1] == 0 or a[1] * b[1] == out[1])


def segments(irs):
    seg = [0]
    for l, _ in irs:
        seg.append(seg[-1] + 2 * l + 1)
    return seg


# ---- equitorch/utils/_indices.py ------------------------------------------------------------------------
def sort_columns(cols):
    """``sort_by_column_key`` (:89-138) with key == data: rows sorted as tuples (stable, lexicographic)."""
    rows = sorted(zip(*cols))
    return [list(c) for c in zip(*rows)] if rows else [[] for _ in cols]


def batch_segments(keys):
    """``extract_batch_segments`` (:12-87): run-length segmentation of already-sorted key columns."""
    if not keys or not keys[0]:
        return [], [], []
    n = len(keys[0])
    seg = [0]
    for i in range(n):
        if any(k[i] != k[seg[-1]] for k in keys):
            seg.append(i)
    seg.append(n)
    batch = [0] * n
    for b in range(len(seg) - 1):
        for i in range(seg[b], seg[b + 1]):
            batch[i] = b
    vals = [[k[s] for s in seg[:-1]] for k in keys]
    return batch, seg, vals


def scatter_indices(keys):
    """``extract_scatter_indices`` (:140-204): rank of each key tuple among the sorted unique tuples."""
    if not keys or not keys[0]:
        return [], []
    tuples = list(zip(*keys))
    uniq = sorted(set(tuples))
    idx = [bisect.bisect_left(uniq, t) for t in tuples]
    return idx, [list(c) for c in zip(*uniq)]


# ---- equitorch/utils/_structs.py ---------------------------------------------------------------------------
def _fill_segments(index_m, seg_m, out_size):
    """The ``seg_new`` loop shared by ``sparse_scale_info`` (:47-54) and ``sparse_product_info`` (:114-121)."""
    seg_new, cnt = [0], 0
    for m in range(out_size):
        if cnt < len(index_m) and index_m[cnt] == m:
            seg_new.append(seg_m[cnt + 1])
            cnt += 1
        else:
            seg_new.append(seg_new[-1])
    return seg_new


def sparse_scale_info(index=None, index_out=None, scale=None, out_size=None):
    """:22-71. Returns dict(scale, index, seg_out, index_out, out_size)."""
    assert index is not None or index_out is not None
    n = len(index or index_out)
    index = index or list(range(n))
    index_out = index_out or list(range(n))
    if scale is not None:
        index_out_s, index_s, scale_s = sort_columns([index_out, index, scale])
    else:
        index_out_s, index_s = sort_columns([index_out, index])
        scale_s = None
    _, seg_m, (index_m,) = batch_segments([index_out_s])
    if out_size is None:
        out_size = len(index_m)
    seg_new = _fill_segments(index_m, seg_m, out_size)
    if index_s == list(range(n)):
        index_s = None
    if seg_new == list(range(out_size + 1)):
        seg_new = None
    return dict(scale=scale_s, index=index_s, seg_out=seg_new, index_out=None, out_size=out_size)


def sparse_scale_infos(index=None, index_out=None, scale=None, out_size=None, in_size=None):
    """:73-77."""
    return (sparse_scale_info(index, index_out, scale, out_size),
            sparse_scale_info(index_out, index, scale, in_size))


def sparse_product_info(index1=None, index2=None, index=None, scale=None, out_size=None):
    """:79-138. Returns dict(scale, index1, index2, seg_out, gather_index, index_out, out_size)."""
    assert index1 is not None or index2 is not None or index is not None
    n = len(index1 or index2 or index)
    index1 = index1 or list(range(n))
    index2 = index2 or list(range(n))
    index = index or list(range(n))
    if scale is not None:
        index_s, index1_s, index2_s, scale_s = sort_columns([index, index1, index2, scale])
    else:
        index_s, index1_s, index2_s = sort_columns([index, index1, index2])
        scale_s = None
    _, seg_m, (index_m,) = batch_segments([index_s])
    if out_size is None:
        out_size = len(index_m)
    # :103-106 — pads for empty leading / trailing output rows *before* the seg_new loop indexes seg_m by
    # the running count; when the first output row is empty the prefix shifts that indexing (kept as is).
    if index_m[0] != 0:
        seg_m = [0] * index_m[0] + seg_m
    if index_m[-1] != out_size:
        seg_m = seg_m + [n] * (out_size - index_m[-1] - 1)
    if index1_s == list(range(n)):
        index1_s = None
    if index2_s == list(range(n)):
        index2_s = None
    seg_new = _fill_segments(index_m, seg_m, out_size)
    if seg_new == list(range(out_size + 1)):
        seg_new = None
    return dict(scale=scale_s, index1=index1_s, index2=index2_s, seg_out=seg_new, gather_index=None,
                index_out=None, out_size=out_size)


def sparse_product_infos(index1=None, index2=None, index=None, scale=None, out_size=None, in1_size=None,
                         in2_size=None):
    """:141-147: the same COO list with the three roles rotated."""
    return (sparse_product_info(index1, index2, index, scale, out_size),
            sparse_product_info(index2, index, index1, scale, in1_size),
            sparse_product_info(index, index1, index2, scale, in2_size))


def fully_connected_paths(irs_out, irs1, irs2):
    """``generate_fully_connected_tp_paths`` (:149-159)."""
    return [(k, i, j) for k, o in enumerate(irs_out) for i, a in enumerate(irs1) for j, b in enumerate(irs2)
            if has_path(o, a, b)]


def prepare_so3(irs_out, irs1, irs2, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """:162-216. COO lists (cg, M, M1, M2, k, i, j, w_idx) and the number of paths."""
    if not path:
        path = fully_connected_paths(irs_out, irs1, irs2)
    so, s1, s2 = segments(irs_out), segments(irs1), segments(irs2)
    count, cur = {}, None
    for k, _, _ in path:  # run length of consecutive equal k (:177-184)
        if k == cur:
            count[k] += 1
        else:
            count[k] = 1
            cur = k
    cols = [[] for _ in range(8)]
    for w, (k, i, j) in enumerate(path):
        l, l1, l2 = irs_out[k][0], irs1[i][0], irs2[j][0]
        cg = ref_constants.so3_cg(l, l1, l2)
        for km in range(2 * l + 1):
            norm = (count[k] ** (-0.5) if path_norm else 1.0) * (channel_scale if channel_norm else 1.0)
            for im in range(2 * l1 + 1):
                for jm in range(2 * l2 + 1):
                    v = float(cg[km][im][jm]) * norm
                    if v != 0.0:
                        for col, x in zip(cols, (v, so[k] + km, s1[i] + im, s2[j] + jm, k, i, j, w)):
                            col.append(x)
    return (*cols, len(path))


TP_FIELDS = ("info_Mij_fwd", "info_Mij_bwd1", "info_Mij_bwd2", "info_M_fwd", "info_M_bwd1", "info_M_bwd2",
             "info_kM1j_fwd", "info_kM1j_bwd1", "info_kM1j_bwd2", "info_kM1M2_fwd", "info_kM1M2_bwd1",
             "info_kM1M2_bwd2", "info_M_kM1M2_fwd", "info_M_kM1M2_bwd")


def create_tp_info(cg, M, M1, M2, k, i, j, w, out_size, in1_size, in2_size):
    """:219-291."""
    k_s, M_s, i_s, j_s, M1_s, M2_s, w_s, cg_s = sort_columns([k, M, i, j, M1, M2, w, cg])
    mij, _, (k_q, M_q, i_q, j_q, w_q) = batch_segments([k_s, M_s, i_s, j_s, w_s])
    infos_inter = sparse_product_infos(M1_s, M2_s, mij, cg_s, in1_size=in1_size, in2_size=in2_size)
    m_batch_q, _, _ = batch_segments([M_q])
    infos_m = sparse_product_infos(index2=w_q, index=m_batch_q, out_size=out_size)

    b5, (k5, i5, j5, M15, M25, w5) = scatter_indices([k_s, i_s, j_s, M1_s, M2_s, w_s])
    b4, (k4, i4, M14, j4, w4) = scatter_indices([k5, i5, M15, j5, w5])
    m_batch, _, (m_out,) = batch_segments([M_s])
    infos_km1j = sparse_product_infos(index1=M14, index2=w4, in1_size=in1_size)
    infos_km1m2 = sparse_product_infos(index1=b4, index2=M25, in2_size=in2_size)
    infos_m_km1m2 = sparse_scale_infos(index=b5, index_out=[m_out[b] for b in m_batch], scale=cg_s,
                                       out_size=out_size)
    vals = (*infos_inter, *infos_m, *infos_km1j, *infos_km1m2, *infos_m_km1m2)
    info = dict(zip(TP_FIELDS, vals))
    info["out_size"] = out_size
    return info


def tp_infos(irreps_out, irreps1, irreps2, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """:318-333: forward table and the two role-rotated backward tables, plus the number of paths."""
    io, i1, i2 = parse(irreps_out), parse(irreps1), parse(irreps2)
    cg, M, M1, M2, k, i, j, w, n_paths = prepare_so3(io, i1, i2, path, path_norm, channel_norm, channel_scale)
    do, d1, d2 = segments(io)[-1], segments(i1)[-1], segments(i2)[-1]
    return (create_tp_info(cg, M, M1, M2, k, i, j, w, do, d1, d2),
            create_tp_info(cg, M1, M2, M, i, j, k, w, d1, d2, do),
            create_tp_info(cg, M2, M, M1, j, k, i, w, d2, do, d1),
            n_paths)


# ---- irreps-preserving channel mixing (equitorch/utils/_structs.py:336-459) --------------------------------
def has_linear_path(out, a):
    """``has_path`` with two arguments (equitorch/irreps/__init__.py:237-238)."""
    return out[0] == a[0] and (out[1] == 0 or a[1] == out[1])


def prepare_irreps_linear(irs_out, irs_in, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """:346-385.  Pinned by closed forms (tests/test_tables.py): entry count ``sum over paths of 2l+1``, scale
    ``count^-1/2``, and the layer reducing to ``x @ W`` per irrep when every output irrep has one path."""
    if not path:
        path = [(i, i0) for i, o in enumerate(irs_out) for i0, a in enumerate(irs_in) if has_linear_path(o, a)]
    seg_out, seg_in = segments(irs_out), segments(irs_in)
    current, count = None, {}
    for i, _ in path:
        count[i] = count[i] + 1 if i == current else 1
        current = i
    scales, M_s, M0_s, ii0_s = [], [], [], []
    for w_idx, (i, i0) in enumerate(path):
        norm = count[i] ** (-0.5) if path_norm else 1
        if channel_norm:
            norm *= channel_scale
        for m in range(2 * irs_out[i][0] + 1):
            scales.append(norm)
            M_s.append(seg_out[i] + m)
            M0_s.append(seg_in[i0] + m)
            ii0_s.append(w_idx)
    return scales, M_s, M0_s, ii0_s, len(path)


def create_irreps_linear_info(scales, M_s, M0_s, ii0_s, out_size):
    """:387-415, as a dict with the field names of ``IrrepsLinearInfo``."""
    M_MM0, M0_MM0, ii0_MM0, scales_MM0 = sort_columns([M_s, M0_s, ii0_s, scales])
    _, M_seg, (M,) = batch_segments([M_MM0])
    ii0_k, M_k, M0_k, scales_k = sort_columns([ii0_s, M_s, M0_s, scales])
    _, ii0_seg, (_, scales_ii0) = batch_segments([ii0_k, scales_k])
    return dict(scale_MM0=scales_MM0, M_seg_MM0=M_seg, ii0_MM0=ii0_MM0, M0_MM0=M0_MM0, M_MM0=M_MM0, M_out=M,
                ii0_seg_ii0MM0=ii0_seg, M_ii0MM0=M_k, M0_ii0MM0=M0_k, scales_ii0=scales_ii0, out_size=out_size)


def irreps_linear_infos(irreps_out, irreps_in, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """:432-443 -> (forward dict, backward dict, num_paths)."""
    io, ii = parse(irreps_out), parse(irreps_in)
    scales, M_s, M0_s, ii0_s, n = prepare_irreps_linear(io, ii, path, path_norm, channel_norm, channel_scale)
    return (create_irreps_linear_info(scales, M_s, M0_s, ii0_s, segments(io)[-1]),
            create_irreps_linear_info(scales, M0_s, M_s, ii0_s, segments(ii)[-1]), n)


def irreps_info(irreps):
    """:446-459."""
    irs = parse(irreps)
    idx = [i for i, (l, _) in enumerate(irs) for _ in range(2 * l + 1)]
    return dict(rsqrt_dims=[(2 * l + 1) ** (-0.5) for l, _ in irs], rdims=[1 / (2 * l + 1) for l, _ in irs],
                irrep_index=idx, irrep_seg=segments(irs), num_irreps=len(irs))


# ---- rotations and the SO(2) linear layer (equitorch/utils/_structs.py:460-786) -----------------------------
def _components(irs):
    table, at = {}, 0
    for i, (l, _) in enumerate(irs):
        for m in range(-l, l + 1):
            table[(i, m)] = at
            at += 1
    return table


def z_rotation_infos(irreps):
    """:460-585 -> (forward, gradient-of-x, gradient-of-cs) dicts of ``sparse_product_infos``."""
    irs = parse(irreps)
    where = _components(irs)
    i1, i2, io, sc = [], [], [], []
    for (i, m), M in where.items():
        if m == 0:
            io.append(M); sc.append(1.0); i1.append(M); i2.append(0)
        else:
            io.append(M); sc.append(1.0); i1.append(M); i2.append(2 * abs(m))
            io.append(M); sc.append(-(float(m > 0) - float(m < 0))); i1.append(where[(i, -m)]); i2.append(2 * abs(m) - 1)
    dim = segments(irs)[-1]
    return sparse_product_infos(i1, i2, io, sc, dim, dim, 1 + 2 * max(l for l, _ in irs))


def j_matrix_info(irreps):
    """:587-636."""
    irs = parse(irreps)
    idx_in, idx_out, sc, off = [], [], [], 0
    for l, _ in irs:
        blk = ref_constants.j_matrix(l)
        for r in range(2 * l + 1):
            for c in range(2 * l + 1):
                if abs(blk[r][c]) > 1e-9:
                    idx_out.append(off + r); idx_in.append(off + c); sc.append(float(blk[r][c]))
        off += 2 * l + 1
    return sparse_scale_info(index=idx_in, index_out=idx_out, scale=sc, out_size=off)


def so2_linear_infos(irreps_out, irreps_in, path=None, path_norm=True, channel_norm=False, channel_scale=1.0):
    """:674-786 -> (forward, backward1, backward2 dicts, num_weights).  The count for ``m > 0`` is read under the key
    ``(k, -m)``, which is never written, so it is always 1 — as in the reference."""
    io_, ii_ = parse(irreps_out), parse(irreps_in)
    if path is None:
        path = [(k, i) for k in range(len(io_)) for i in range(len(ii_))]
    w_in, w_out = _components(ii_), _components(io_)
    widx, cnt = {}, {}
    for k, i in path:
        for m in range(min(io_[k][0], ii_[i][0]) + 1):
            if m == 0:
                widx[(k, i, 0)] = len(widx)
                cnt[(k, 0)] = cnt.get((k, 0), 0) + 1
            else:
                widx[(k, i, -m)] = len(widx)
                cnt[(k, m)] = cnt.get((k, -m), 0) + 1
                widx[(k, i, m)] = len(widx)
                cnt[(k, m)] = cnt.get((k, -m), 0) + 1
    i1, i2, io, sc = [], [], [], []
    for k, i in path:
        for m in range(min(io_[k][0], ii_[i][0]) + 1):
            if m == 0:
                sc.append(cnt[(k, 0)] ** (-0.5) if path_norm else 1.0)
                io.append(w_out[(k, 0)]); i1.append(w_in[(i, 0)]); i2.append(widx[(k, i, 0)])
                continue
            s = (cnt[(k, m)] * 2) ** (-0.5) if path_norm else 2 ** (-0.5)
            for out_m, in_m, w_m, sign in ((m, m, m, 1), (-m, -m, m, 1), (m, -m, -m, -1), (-m, m, -m, 1)):
                sc.append(sign * s)
                io.append(w_out[(k, out_m)]); i1.append(w_in[(i, in_m)]); i2.append(widx[(k, i, w_m)])
    if channel_norm:
        sc = [s * channel_scale for s in sc]
    n = len(widx)
    return (*sparse_product_infos(i1, i2, io, sc, segments(io_)[-1], segments(ii_)[-1], n), n)
