"""Irreps-preserving channel mixing (``IrrepsLinear`` / ``IrrepWiseLinear``).  With a shared weight the layer runs on
the hand-written matrix-core kernels of the fully connected product (bf16: compiled tables; fp32: table-driven) as a
product with the scalar 1; per-sample weights, fp64, higher-order gradients and shapes those kernels do not take run
as library GEMMs on strided views:

The reference runs these layers on its table-driven vector-matrix kernels (``indexed_vecmat_scale_segment`` plus
a scatter, ``equitorch/nn/functional/linears.py:494-571``).  The tables have a simple structure: a path couples
the ``2l+1`` consecutive components of one input irrep with those of one output irrep through one ``(C_in, C_out)``
matrix and one scale.  So every path is a plain GEMM, and this module issues it as such — the one place where a
library GEMM (``torch.baddbmm`` / ``torch.bmm`` -> rocBLAS / hipBLASLt) is the right kernel:

* shared weight ``(P, C_in, C_out)``: a batch of ``2l+1`` GEMMs ``(N, C_in) @ (C_in, C_out)``, one per component,
  reading ``x[:, M0, :]`` and writing ``out[:, M, :]`` in place through their row strides (no gather, no scatter,
  no intermediate);
* per-sample weight ``(N, P, C_in, C_out)``: a batch of ``N`` GEMMs ``(2l+1, C_in) @ (C_in, C_out)``.

Gradients are the same two primitives again (``mix`` with the transposed weight and exchanged row ranges for the
input, ``outer`` for the weight), each a :class:`torch.autograd.Function` whose backward is written in terms of
the two, so gradients of every order are available as in the reference.
"""
from typing import List, NamedTuple, Tuple

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
from ...ops.kernels import cached


class Path(NamedTuple):
    w: int          # weight index
    o0: int         # first output component
    i0: int         # first input component
    k: int          # number of components (2l+1)
    scale: float


class Group(NamedTuple):
    """Consecutive paths whose output and input ranges advance together: one batched GEMM over ``rows`` components,
    component ``j`` using weight ``w_of_row[j]`` times ``scale_of_row[j]``."""
    o0: int
    i0: int
    rows: int
    w_of_row: Tuple[int, ...]
    scale_of_row: Tuple[float, ...]
    accumulate: bool      # an earlier group already wrote these output rows

    @property
    def scale(self):
        """The common scale of the rows, or None if they differ."""
        return self.scale_of_row[0] if len(set(self.scale_of_row)) == 1 else None


class LinearPlan(NamedTuple):
    paths: Tuple[Path, ...]
    n_paths: int
    out_size: int

    def groups(self) -> Tuple[Group, ...]:
        out: List[Group] = []
        written: List[Tuple[int, int]] = []
        for p in self.paths:
            g = out[-1] if out else None
            hit = any(a < p.o0 + p.k and p.o0 < b for a, b in written)
            if (g is not None and g.o0 + g.rows == p.o0 and g.i0 + g.rows == p.i0
                    and not g.accumulate and not hit):
                out[-1] = Group(g.o0, g.i0, g.rows + p.k, g.w_of_row + (p.w,) * p.k,
                                g.scale_of_row + (p.scale,) * p.k, False)
                written[-1] = (g.o0, g.o0 + g.rows + p.k)
            else:
                out.append(Group(p.o0, p.i0, p.k, (p.w,) * p.k, (p.scale,) * p.k, hit))
                written.append((p.o0, p.o0 + p.k))
        return tuple(out)


def _plan_from_entries(M, M0, ii0, scale, out_size) -> LinearPlan:
    """Group table entries ``(M, M0, path, scale)`` by path and check that each path is a pair of consecutive
    ranges with one scale — true for every table ``irreps_linear_infos`` builds."""
    by_path = {}
    for m, m0, p, s in zip(M, M0, ii0, scale):
        by_path.setdefault(int(p), []).append((int(m), int(m0), float(s)))
    paths = []
    for p in sorted(by_path):
        ent = sorted(by_path[p])
        o0, i0, s = ent[0]
        for j, (m, m0, sj) in enumerate(ent):
            if m != o0 + j or m0 != i0 + j or sj != s:
                raise _lib.CgtpError("irreps_linear: a path of the table is not a pair of consecutive component "
                                     "ranges with a single scale")
        paths.append(Path(p, o0, i0, len(ent), s))
    return LinearPlan(tuple(paths), (max(by_path) + 1) if by_path else 0, int(out_size))


def plan_of_linear_info(info) -> LinearPlan:
    return cached(info.M_MM0, "linear_plan", lambda: _plan_from_entries(
        info.M_MM0.tolist(), info.M0_MM0.tolist(), info.ii0_MM0.tolist(), info.scale_MM0.tolist(), info.out_size))


def plan_of_irreps_info(info) -> LinearPlan:
    def build():
        seg = info.irrep_seg.tolist()
        return LinearPlan(tuple(Path(i, seg[i], seg[i], seg[i + 1] - seg[i], 1.0) for i in range(len(seg) - 1)),
                          len(seg) - 1, seg[-1])
    return cached(info.irrep_seg, "irrep_wise_plan", build)


def plan_of_product_info(info, in_size: int, n_weights: int) -> LinearPlan:
    """Plan of ``out[n, M, :] = sum_t scale_t * x[n, index1_t, :] @ W[index2_t]`` for a ``SparseProductInfo`` (the
    table of ``sparse_vecmat``; ``SO2Linear('uv')``): one single-component path per entry, ordered so that entries
    on one diagonal (``M - index1`` fixed, ``M`` rising) follow each other and merge into batched GEMMs."""
    anchor = next(t for t in (info.seg_out, info.index1, info.index2, info.scale) if t is not None)

    def build():
        n = next((t.shape[0] for t in (info.index1, info.index2, info.scale) if t is not None), None)
        if n is None:
            n = int(info.seg_out[-1]) if info.seg_out is not None else in_size
        i1 = list(range(n)) if info.index1 is None else info.index1.tolist()
        i2 = list(range(n)) if info.index2 is None else info.index2.tolist()
        sc = [1.0] * n if info.scale is None else info.scale.tolist()
        if info.seg_out is None:
            out_of, n_out = list(range(n)), n
        else:
            seg = info.seg_out.tolist()
            n_out = len(seg) - 1
            out_of = [m for m in range(n_out) for _ in range(seg[m], seg[m + 1])]
        if info.out_size is not None:
            n_out = max(n_out, int(info.out_size))
        entries = sorted(zip(out_of, i1, i2, sc), key=lambda e: (e[0] - e[1], e[0]))
        return LinearPlan(tuple(Path(int(w), int(m), int(m0), 1, float(s)) for m, m0, w, s in entries), int(n_weights),
                          int(n_out))
    return cached(anchor, ("product_plan", in_size, n_weights), build)


def transposed(plan: LinearPlan, in_size: int) -> LinearPlan:
    return LinearPlan(tuple(Path(p.w, p.i0, p.o0, p.k, p.scale) for p in plan.paths), plan.n_paths, in_size)


_GROUPS = {}


def _groups(plan: LinearPlan) -> Tuple[Group, ...]:
    g = _GROUPS.get(plan)
    if g is None:
        if len(_GROUPS) > 256:
            _GROUPS.clear()
        g = _GROUPS[plan] = plan.groups()
    return g


_ROW_WEIGHTS = {}


def _row_weights(grp: Group, device) -> Tensor:
    key = (grp.w_of_row, str(device))
    t = _ROW_WEIGHTS.get(key)
    if t is None:
        if len(_ROW_WEIGHTS) > 256:
            _ROW_WEIGHTS.clear()
        t = _ROW_WEIGHTS[key] = torch.tensor(grp.w_of_row, dtype=torch.int64, device=device)
    return t


_ROW_SCALES = {}


def _row_scales(grp: Group, like: Tensor) -> Tensor:
    """``(rows, 1, 1)`` tensor of the rows' scales (only asked for when they differ)."""
    key = (grp.scale_of_row, str(like.device), like.dtype)
    t = _ROW_SCALES.get(key)
    if t is None:
        if len(_ROW_SCALES) > 256:
            _ROW_SCALES.clear()
        t = _ROW_SCALES[key] = torch.tensor(grp.scale_of_row, dtype=like.dtype, device=like.device).view(-1, 1, 1)
    return t


def _covered(plan: LinearPlan) -> bool:
    rows = sorted((p.o0, p.o0 + p.k) for p in plan.paths)
    end = 0
    for a, b in rows:
        if a > end:
            return False
        end = max(end, b)
    return end >= plan.out_size


def _mix_raw(x: Tensor, w: Tensor, plan: LinearPlan, w_t: bool) -> Tensor:
    """``out[n, o0+j, :] += scale * x[n, i0+j, :] @ W[(n,) p]`` for every path; ``w_t``: use ``W^T``."""
    n, _, cin = x.shape
    shared = w.ndim == 3
    cout = w.shape[-2] if w_t else w.shape[-1]
    out = (torch.empty if _covered(plan) else torch.zeros)((n, plan.out_size, cout), dtype=x.dtype, device=x.device)
    if n == 0:
        return out
    for grp in _groups(plan):
        xs, os_ = x[:, grp.i0:grp.i0 + grp.rows, :], out[:, grp.o0:grp.o0 + grp.rows, :]
        beta = 1.0 if grp.accumulate else 0.0
        if shared:
            # one GEMM (N, C_in) @ (C_in, C_out) per component, batched over the components of the group
            wb = w.index_select(0, _row_weights(grp, w.device))
            alpha = grp.scale
            if alpha is None:                                          # rows with different scales: fold them in
                wb, alpha = wb * _row_scales(grp, wb), 1.0
            if w_t:
                wb = wb.transpose(1, 2)
            ot = os_.transpose(0, 1)                                   # (rows, N, cout), rows strided by D_out * cout
            torch.baddbmm(ot, xs.transpose(0, 1), wb, beta=beta, alpha=alpha, out=ot)
        else:
            # per sample: (rows of one path, C_in) @ (C_in, C_out); paths of a group share nothing, so go one by one
            at = 0
            while at < grp.rows:
                pw = grp.w_of_row[at]
                k = next((j for j in range(at, grp.rows) if grp.w_of_row[j] != pw), grp.rows) - at
                wp = w[:, pw].transpose(1, 2) if w_t else w[:, pw]
                k = next((j for j in range(at, at + k) if grp.scale_of_row[j] != grp.scale_of_row[at]), at + k) - at
                dst = os_[:, at:at + k, :]
                torch.baddbmm(dst, xs[:, at:at + k, :], wp, beta=beta, alpha=grp.scale_of_row[at], out=dst)
                at += k
    return out


def _long_k_bmm(a: Tensor, b: Tensor) -> Tensor:
    """``bmm(a (B, m, K), b (B, K, n))`` for small ``m x n`` and long ``K`` (a sum over samples): the library runs one
    workgroup per output tile down the whole of ``K``, so the sum is cut into ``S`` slices that run as a larger batch
    and are added afterwards."""
    k = a.shape[-1]
    s = 1
    while s < 64 and k % (2 * s) == 0 and k // (2 * s) >= 512:
        s *= 2
    if s == 1:
        return torch.bmm(a, b)
    parts = torch.matmul(a.unflatten(2, (s, k // s)).permute(0, 2, 1, 3), b.unflatten(1, (s, k // s)))
    return parts.sum(dim=1)


def _all_rows_outer(x: Tensor, g: Tensor):
    """``prod[j] = sum_n x[n, j, :]^T (x) g[n, j, :]`` for every component ``j`` of contiguous ``x (N, D, C_in)`` and
    ``g (N, D, C_out)``, or None when ``N`` is too short to be worth cutting.  The sum over samples is cut into ``S``
    interleaved slices (sample ``n`` belongs to slice ``n mod S``): seen as ``(N/S, S*D, C)`` the tensors then have
    one batch axis ``(slice, component)`` of stride ``C``, so the ``S*D`` partial products are one batched GEMM on
    the tensors as they lie in memory, and their sum over the slices is small."""
    n, d, cin = x.shape
    cout = g.shape[-1]
    s = 1
    while s < 64 and n % (2 * s) == 0 and n // (2 * s) >= 512:
        s *= 2
    if s == 1:
        return None
    a = x.view(n // s, s * d, cin).permute(1, 2, 0)             # (S*D, C_in, N/S), a transposed operand
    b = g.view(n // s, s * d, cout).transpose(0, 1)             # (S*D, N/S, C_out)
    return torch.bmm(a, b).view(s, d, cin, cout).sum(dim=0)


def _outer_raw(x: Tensor, g: Tensor, plan: LinearPlan, shared: bool) -> Tensor:
    """``gw[(n,) p] = scale * sum_j x[n, i0+j, :]^T (x) g[n, o0+j, :]`` (summed over ``n`` when ``shared``)."""
    n, _, cin = x.shape
    cout = g.shape[-1]
    if shared:
        gw = torch.zeros((plan.n_paths, cin, cout), dtype=x.dtype, device=x.device)
        if n:
            for grp in _groups(plan):
                prod = None
                if grp.rows == x.shape[1] == g.shape[1] and x.is_contiguous() and g.is_contiguous():
                    prod = _all_rows_outer(x, g)
                if prod is None:
                    a = x[:, grp.i0:grp.i0 + grp.rows, :].permute(1, 2, 0)      # (rows, cin, N)
                    b = g[:, grp.o0:grp.o0 + grp.rows, :].transpose(0, 1)       # (rows, N, cout)
                    prod = _long_k_bmm(a, b)
                if grp.scale is None:
                    gw.index_add_(0, _row_weights(grp, x.device), prod * _row_scales(grp, prod))
                else:
                    gw.index_add_(0, _row_weights(grp, x.device), prod, alpha=grp.scale)
        return gw
    gw = torch.zeros((n, plan.n_paths, cin, cout), dtype=x.dtype, device=x.device)
    if n:
        for p in plan.paths:      # gw starts at zero and a weight may serve several paths: accumulate
            dst = gw[:, p.w]
            torch.baddbmm(dst, x[:, p.i0:p.i0 + p.k, :].transpose(1, 2), g[:, p.o0:p.o0 + p.k, :], beta=1.0,
                          alpha=p.scale, out=dst)
    return gw


class _Mix(Function):
    """out = mix(x, W): the layer itself; also the gradient with respect to x (transposed plan and weight)."""

    @staticmethod
    def forward(ctx, x: Tensor, w: Tensor, plan: LinearPlan, w_t: bool, in_size: int):
        ctx.save_for_backward(x, w)
        ctx.plan, ctx.w_t, ctx.in_size = plan, w_t, in_size
        return _mix_raw(x, w, plan, w_t)

    @staticmethod
    def backward(ctx, g: Tensor):
        x, w = ctx.saved_tensors
        plan, w_t = ctx.plan, ctx.w_t
        gx = gw = None
        if ctx.needs_input_grad[0]:
            gx = _Mix.apply(g, w, transposed(plan, ctx.in_size), not w_t, plan.out_size)
        if ctx.needs_input_grad[1]:
            if w_t:   # out = x W^T: the gradient of W is the outer product with the operands exchanged
                gw = _Outer.apply(g, x, transposed(plan, ctx.in_size), w.ndim == 3)
            else:
                gw = _Outer.apply(x, g, plan, w.ndim == 3)
        return gx, gw, None, None, None


class _Outer(Function):
    """gw = outer(x, g): gradient with respect to the weight; linear in both arguments."""

    @staticmethod
    def forward(ctx, x: Tensor, g: Tensor, plan: LinearPlan, shared: bool):
        ctx.save_for_backward(x, g)
        ctx.plan, ctx.shared = plan, shared
        return _outer_raw(x.contiguous(), g.contiguous(), plan, shared)

    @staticmethod
    def backward(ctx, ggw: Tensor):
        x, g = ctx.saved_tensors
        plan = ctx.plan
        gx = gg = None
        if ctx.needs_input_grad[0]:   # d/dx sum(ggw * gw) = mix^T(g, ggw^T)
            gx = _Mix.apply(g, ggw, transposed(plan, x.shape[1]), True, g.shape[1])
        if ctx.needs_input_grad[1]:   # d/dg = mix(x, ggw)
            gg = _Mix.apply(x, ggw, LinearPlan(plan.paths, plan.n_paths, g.shape[1]), False, x.shape[1])
        return gx, gg, None, None


def _as_tensor_product(plan: LinearPlan, in_size: int):
    """The layer as a fully connected product with the scalar 1 as second operand (``C(l; l, 0)`` is the identity):
    forward ``TensorProductInfo`` over parity-free irreps laid out like the plan's row ranges, or None if the
    plan's scales are not the path normalisation such a product would carry."""
    from ...utils import tp_infos

    def layout(blocks, size):
        irreps, index, at = [], {}, 0
        for start, k in sorted(set(blocks)):
            if start < at:
                return None, None            # overlapping ranges of different irreps
            irreps += [0] * (start - at)     # rows no path touches: scalars
            index[start] = len(irreps)
            irreps.append((k - 1) // 2)
            at = start + k
        irreps += [0] * (size - at)
        return irreps, index

    irr_out, idx_out = layout([(p.o0, p.k) for p in plan.paths], plan.out_size)
    irr_in, idx_in = layout([(p.i0, p.k) for p in plan.paths], in_size)
    if irr_out is None or irr_in is None or [p.w for p in plan.paths] != list(range(len(plan.paths))):
        return None
    path = [(idx_out[p.o0], idx_in[p.i0], 0) for p in plan.paths]
    if path != sorted(path):
        return None
    info = tp_infos(irr_out, irr_in, [0], path=path)[0]
    return info


def _matrix_core_path(x: Tensor, weight: Tensor, plan: LinearPlan, in_size: int, anchor: Tensor):
    """bf16 with a shared weight: the hand-written MFMA kernels of the fully connected product, if a table equal to
    this layer's is compiled in (cgtp_uv_find); None otherwise."""
    from . import _uvw_mfma
    if x.dtype != torch.bfloat16 or weight.ndim != 3 or x.shape[0] == 0:
        return None
    def build():
        info = _as_tensor_product(plan, in_size)
        return False if info is None else info.to(x.device)     # False: memoised "no such product"

    info = cached(anchor, ("linear_as_tp", in_size, str(x.device)), build)
    if info is False or _uvw_mfma.uv_config_of(info) < 0:
        return None
    ones = cached(anchor, ("ones", x.shape[0], str(x.device)),
                  lambda: torch.ones(x.shape[0], 1, dtype=torch.bfloat16, device=x.device))
    return _uvw_mfma.try_forward(x, ones, weight, info)


_ONES = {}


def _ones_column(n: int, dtype, device) -> Tensor:
    """``(n, 1)`` ones: one buffer per dtype and device, grown geometrically to the largest batch seen and sliced, so
    that graphs of varying size do not leave one buffer per distinct size behind."""
    key = (dtype, str(device))
    buf = _ONES.get(key)
    if buf is None or buf.shape[0] < n:
        buf = torch.ones(max(n, 2 * (0 if buf is None else buf.shape[0])), 1, dtype=dtype, device=device)
        _ONES[key] = buf
    return buf[:n]


def _table_driven_path(x: Tensor, weight: Tensor, plan: LinearPlan, in_size: int, anchor: Tensor):
    """fp32 with a shared weight: the layer as a fully connected product with the scalar 1 on the table-driven
    matrix-core kernels (``cgtp_uvt_*``: forward, grad input and grad weight in one launch each, rows read and written
    in place): every path of the plan becomes ``k`` table entries (output row, input row, 0, weight, scale).  None
    when the extents do not fit those kernels."""
    import numpy as np

    from ..._tables import TpCoo
    from ...ops import kernels
    from . import _uv_native
    if x.dtype not in (torch.float32, torch.float64) or weight.ndim != 3 or x.shape[0] == 0:
        return None

    def build():
        rows = [(p.o0 + j, p.i0 + j, p.w, p.scale) for p in plan.paths for j in range(p.k)]
        if not rows:
            return False
        m, m1, pw, sc = (np.asarray(v) for v in zip(*rows))
        zeros = np.zeros(len(rows), dtype=np.int32)
        coo = TpCoo(sc.astype(np.float64), m.astype(np.int32), m1.astype(np.int32), zeros, pw.astype(np.int32), zeros,
                    int(in_size), 1, int(plan.out_size), int(plan.n_paths))
        return _uv_native.CooTable(coo, anchor, lambda xx, yy, ww: _Mix.apply(xx, ww, plan, False, in_size) * yy[:, :, None])

    table = cached(anchor, ("linear_as_coo_table", in_size, plan.n_paths, plan.out_size), build)
    if table is False:
        return None
    ones = _ones_column(x.shape[0], x.dtype, x.device)
    if not _uv_native.u1v_supported(x, ones, weight, table):
        return None
    kernels.log_tier("irreps_linear", "table-driven matrix-core kernels")
    return _uv_native.u1v(x, ones, weight, table)


def _streaming_path(x: Tensor, weight: Tensor, plan: LinearPlan, in_size: int, anchor: Tensor):
    """A weight per sample: the streaming kernels of the fully connected products (``_psw``), with the scalar 1 as the
    second operand.  None when the plan or the extents do not fit them."""
    import numpy as np

    from ...ops import kernels
    from . import _psw

    def build():
        rows = [(p.o0 + j, p.i0 + j, p.w, p.scale) for p in plan.paths for j in range(p.k)]
        if not rows or in_size > 255:
            return False
        m, m1, pw, sc = (np.asarray(v) for v in zip(*rows))
        try:
            return _psw.PswTable(m, m1, np.zeros_like(m), pw, sc, in_size, 1, plan.out_size, plan.n_paths, x.device)
        except ValueError:
            return False

    table = cached(anchor, ("linear_as_psw_table", in_size, plan.n_paths, plan.out_size, str(x.device)), build)
    if table is False or not _psw.launchable(table, x, None, weight):
        return None
    kernels.log_tier("irreps_linear", "per-sample weight streaming kernel", str(x.dtype))
    return _psw.product(table, x, None, weight, lambda xx, _y, ww: _Mix.apply(xx, ww, plan, False, in_size))


def _adapted_path(x: Tensor, weight: Tensor, plan: LinearPlan, in_size: int, anchor: Tensor):
    """Operands the native kernels do not take as they are, adapted to them: bf16 / fp16 widened to fp32 (the result
    rounded once), channel counts of a shared weight that are not multiples of 4 filled up with zero channels (the
    result cut back).  None when the kernels still have no launch shape for the adapted operands."""
    dtype, cin, cout = x.dtype, weight.shape[-2], weight.shape[-1]
    xa, wa = x, weight
    if dtype in (torch.bfloat16, torch.float16):
        xa, wa = xa.float(), wa.float()
    elif dtype not in (torch.float32, torch.float64):
        return None
    if wa.ndim == 3 and (cin % 4 or cout % 4):
        pad = torch.nn.functional.pad
        xa, wa = pad(xa, (0, -cin % 4)), pad(wa, (0, -cout % 4, 0, -cin % 4))
    if xa is x:
        return None
    out = _table_driven_path(xa, wa, plan, in_size, anchor) if wa.ndim == 3 else _streaming_path(xa, wa, plan, in_size, anchor)
    if out is None:
        return None
    if out.shape[-1] != cout:
        out = out[..., :cout]
    return out.to(dtype).contiguous()


class _NoPaths(Function):
    """A table without a reachable entry: the result is zero whatever the operands hold, and so are their gradients.
    (The reference's builder can produce one: ``sparse_product_info``, ``equitorch/utils/_structs.py:105-123``, shifts
    its segment pointers when the first output row has no entry, e.g. ``SO2Linear('0e' -> '2e+0e')``; its kernels then
    walk no segment and return the zero-filled output.)"""

    @staticmethod
    def forward(ctx, x: Tensor, weight: Tensor, out_size: int):
        ctx.save_for_backward(x, weight)
        return x.new_zeros(x.shape[0], out_size, weight.shape[-1])

    @staticmethod
    def backward(ctx, g):
        x, weight = ctx.saved_tensors
        return torch.zeros_like(x), torch.zeros_like(weight), None


def no_paths(x: Tensor, weight: Tensor, plan: LinearPlan) -> Tensor:
    return _NoPaths.apply(x, weight, plan.out_size)


def mix(input: Tensor, weight: Tensor, plan: LinearPlan, in_size: int, anchor: Tensor = None) -> Tensor:
    """``(..., D_in, C_in) x (P, C_in, C_out) | (N, P, C_in, C_out) -> (..., D_out, C_out)``."""
    _lib.require_gpu(input, weight)
    if input.dtype != weight.dtype:
        raise _lib.CgtpError(f"input is {input.dtype} but weight is {weight.dtype}")
    if input.shape[-2] != in_size:
        raise _lib.CgtpError(f"input has {input.shape[-2]} components, the table expects {in_size}")
    if weight.ndim not in (3, 4) or weight.shape[-3] != plan.n_paths or weight.shape[-2] != input.shape[-1]:
        raise _lib.CgtpError(f"weight {tuple(weight.shape)} does not fit {plan.n_paths} paths of "
                             f"{input.shape[-1]} input channels")
    lead = input.shape[:-2]
    x = input.reshape(-1, *input.shape[-2:]).contiguous()
    if weight.ndim == 4 and weight.shape[0] != x.shape[0]:
        raise _lib.CgtpError(f"per-sample weight has {weight.shape[0]} samples, input has {x.shape[0]}")
    if not plan.paths:
        return no_paths(x, weight, plan).reshape(*lead, plan.out_size, weight.shape[-1])
    out = _matrix_core_path(x, weight, plan, in_size, anchor) if anchor is not None else None
    if out is None and anchor is not None:
        out = _table_driven_path(x, weight, plan, in_size, anchor)
    if out is None and weight.ndim == 4 and anchor is not None:
        out = _streaming_path(x, weight, plan, in_size, anchor)
    if out is None and anchor is not None and x.shape[0] > 0:
        out = _adapted_path(x, weight, plan, in_size, anchor)
    if out is None:
        out = _Mix.apply(x, weight, plan, False, in_size)
    return out.reshape(*lead, plan.out_size, out.shape[-1])
