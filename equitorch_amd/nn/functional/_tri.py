"""Autograd wrapper of the table-driven contraction kernels.

``out[r, o, (c)] = sum_t coef_t * A[r, ia_t, (c)] * B[r, ib_t, (c)] * W[r, iw_t, (c)]`` is linear in each
operand, and its gradient with respect to one operand is the same contraction with that operand's index
column exchanged with the output column and the operand replaced by the incoming gradient.  The family is
therefore closed under differentiation: ``TriContract.backward`` calls ``TriContract`` again, which gives
gradients of every order without saving any intermediate (the reference reaches the same closure through
its sibling Functions and rotated tables, ``equitorch/nn/functional/sparse_product.py``,
``equitorch/nn/functional/linears.py:44-83``).
"""
from __future__ import annotations

from typing import Optional, Sequence

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
        # rows an operand must have for every index of the table to land inside it
        self.min_rows = [0 if i is None or i.size == 0 else int(i.max()) + 1 for i in self.idx]
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


def _axes(kind) -> str:
    """Operand kind -> channel axes it carries: '' (channel-less), 'u', 'w' or 'uw'.  The integer kinds of the
    single-axis family map to 'u' (per-channel) and '' (channel-less)."""
    if kind is None or isinstance(kind, str):
        return kind
    return {OPERAND_NONE: None, OPERAND_VEC: "u", OPERAND_SCALAR: ""}[kind]


def _is_shared(t: Tensor, axes: str) -> bool:
    return t.ndim == 1 + len(axes)


def _gen_operand(t: Optional[Tensor], axes: Optional[str]) -> "_lib.GenOperand":
    op = _lib.GenOperand()
    if t is None or axes is None:
        return op
    op.present, op.data = 1, t.data_ptr()
    shared = _is_shared(t, axes)
    op.row_stride = 0 if shared else t.stride(0)
    op.idx_stride = t.stride(0 if shared else 1)
    pos = 1 if shared else 2
    for ax in axes:
        setattr(op, f"{ax}_stride", t.stride(pos))
        pos += 1
    return op


def _gen_contract(spec: "TriSpec", ops, axes, out_axes: str, out_shared: bool, n_rows: int, U: int, W: int,
                  dtype, device) -> Tensor:
    import ctypes as C
    table = spec.packed(dtype, device)
    a = _lib.GenArgs()
    a.a, a.b, a.w = (_gen_operand(t, ax) for t, ax in zip(ops, axes))
    a.coef, a.idx, a.seg = _lib.ptr(table["coef"]), table["idx"].data_ptr(), table["seg"].data_ptr()
    a.n_out, a.nnz = spec.out_size, table["idx"].shape[0]
    shape = (spec.out_size,) + ((U,) if "u" in out_axes else ()) + ((W,) if "w" in out_axes else ())
    if not out_shared:
        shape = (n_rows,) + shape
    out = torch.empty(shape, dtype=dtype, device=device)
    if n_rows == 0 or out.numel() == 0:      # empty batch: nothing to launch; a sum over no rows is zero
        return out.zero_()
    if a.nnz == 0:                           # a table without entries: a sum over no terms
        return out.zero_()
    a.out, a.n_rows, a.U, a.W = out.data_ptr(), n_rows, U, W
    a.out_has_u, a.out_has_w = int("u" in out_axes), int("w" in out_axes)
    a.reduce_rows, a.dtype = int(out_shared), _lib.dtype_code(dtype)
    _lib.check(_lib.lib.cgtp_gen_contract(C.byref(a), _lib.stream_ptr(device)), "cgtp_gen_contract")
    return out


def _matrix_core_route(spec: "TriSpec", ops, axes, out_axes: str, out_shared: bool, n_rows: int,
                       dtype) -> Optional[Tensor]:
    """Two of the two-axis contractions have matrix-core kernels (``cgtp_uvt_apply`` / ``cgtp_uvt_grad_w``, any
    table): a batched vector operand times a shared matrix operand, with or without a channel-less third operand
    (``indexed_vecmat_scale_gather`` / ``indexed_mat_t_vec_scale_gather`` with a shared ``input2``; reference
    ``ops/batched_sparse_dense_op.py:1200-1534``), and the outer product of two batched vector operands summed over
    the rows (``indexed_outer_scale_gather(..., out_accumulated=True)``, ``:436-579``: the gradient of such a shared
    matrix).  Returns None where they do not apply (other operand shapes, channel counts that are not multiples of
    4, rows of 16 samples beyond the LDS); the caller then takes the general kernel."""
    from ..._tables import TpCoo
    from . import _uv_native as nat
    if dtype not in (torch.float32, torch.float64) or n_rows <= 0:
        return None
    slot = {}
    for i, ax in enumerate(axes):
        if ax is None:
            continue
        if ax in slot:
            return None
        slot[ax] = i
    nnz = spec.out_idx.shape[0]
    if nnz == 0:
        return None
    coef = np.ones(nnz) if spec.coef is None else spec.coef
    zeros = np.zeros(nnz, dtype=np.int64)

    def rows_of(ax):           # (batched, contiguous) rows of a vector / channel-less operand
        t = ops[slot[ax]]
        return t.contiguous() if t.ndim == 2 + len(ax) else None

    def table(key, build):
        fast = spec.__dict__.setdefault("_matrix_core_tables", {})
        if key not in fast:
            fast[key] = nat.CooTable(build(), torch.empty(0), None)
        return fast[key]

    if not out_shared and "uw" in slot and len(out_axes) == 1 and set(slot) - {""} == {"uw", "uw".replace(out_axes, "")}:
        vec_ax = "uw".replace(out_axes, "")
        mat, x = ops[slot["uw"]], rows_of(vec_ax)
        y = rows_of("") if "" in slot else torch.ones((n_rows, 1), dtype=dtype, device=mat.device)
        if mat.ndim != 3 or x is None or y is None or x.data_ptr() % 16:
            return None
        n_paths, d1, d2 = mat.shape[0], x.shape[1], y.shape[1]
        k, cout = (mat.shape[1], mat.shape[2]) if vec_ax == "u" else (mat.shape[2], mat.shape[1])
        if nat.chunk_of(n_rows, d1, d2, spec.out_size, k, 0, cout, dtype) <= 0:
            return None
        tab = table(("apply", vec_ax, "" in slot), lambda: TpCoo(
            coef, spec.out_idx, spec.idx[slot[vec_ax]], spec.idx[slot[""]] if "" in slot else zeros,
            spec.idx[slot["uw"]], zeros, d1, d2, spec.out_size, n_paths))
        sp, su, sw = mat.stride()
        wp = nat.pack(mat, n_paths, k, cout, sp, *((su, sw) if vec_ax == "u" else (sw, su)))
        kernels.log_tier("sparse matrix product", "table-driven matrix-core kernel (shared matrix)", str(dtype))
        return nat.apply(x, y, wp, tab, "out", spec.out_size, cout)
    if out_shared and out_axes == "uw" and set(slot) - {""} == {"u", "w"}:
        x, g = rows_of("u"), rows_of("w")
        y = rows_of("") if "" in slot else torch.ones((n_rows, 1), dtype=dtype, device=ops[slot["u"]].device)
        if x is None or g is None or y is None or x.shape[2] % 4 or g.shape[2] % 4:
            return None
        if (x.data_ptr() | g.data_ptr()) % 16:
            return None
        tab = table(("grad_w", "" in slot), lambda: TpCoo(
            coef, spec.idx[slot["w"]], spec.idx[slot["u"]], spec.idx[slot[""]] if "" in slot else zeros,
            spec.out_idx, zeros, x.shape[1], y.shape[1], g.shape[1], spec.out_size))
        kernels.log_tier("sparse matrix product", "table-driven matrix-core kernel (outer product summed over rows)",
                         str(dtype))
        return nat.grad_w(x, y, g, tab)
    return None


class TriContract(Function):
    """forward(spec, kinds, out_kind, out_shared, a, b, w) -> out.

    ``kinds`` / ``out_kind`` name the channel axes of each operand ('' | 'u' | 'w' | 'uw', or the integer kinds
    of the single-axis family; None / OPERAND_NONE = operand absent, passed as None).  An axis the output carries
    is element-wise, the others are summed.  Half-precision inputs are computed in fp32 and rounded once."""

    @staticmethod
    def forward(ctx, spec: TriSpec, kinds, out_kind, out_shared: bool,
                a: Optional[Tensor], b: Optional[Tensor], w: Optional[Tensor]):
        axes = [_axes(k) for k in kinds]
        out_axes = _axes(out_kind)
        ops = [a, b, w]
        present = [t for t, ax in zip(ops, axes) if ax is not None]
        _lib.require_gpu(*present)
        res_dtype = present[0].dtype
        for t in present[1:]:
            res_dtype = torch.promote_types(res_dtype, t.dtype)
        dtype = res_dtype if res_dtype in (torch.float32, torch.float64) else torch.float32
        device = present[0].device
        single_axis = all(ax in (None, "", "u") for ax in axes + [out_axes])
        ops = [None if ax is None else (t.to(dtype).contiguous() if single_axis else t.to(dtype))
               for t, ax in zip(ops, axes)]
        n_rows, ext = None, {"u": None, "w": None}
        for slot, (t, ax) in enumerate(zip(ops, axes)):
            if ax is None:
                continue
            if t.ndim not in (1 + len(ax), 2 + len(ax)):
                raise _lib.CgtpError(f"operand with axes '{ax}' must have {1 + len(ax)} or {2 + len(ax)} dims, "
                                     f"got {t.ndim}")
            have = t.shape[t.ndim - len(ax) - 1]
            if have < spec.min_rows[slot]:
                raise _lib.CgtpError(f"operand {slot} has {have} rows along its indexed axis, the table reaches row "
                                     f"{spec.min_rows[slot] - 1}")
            if not _is_shared(t, ax):
                if n_rows not in (None, t.shape[0]):
                    raise _lib.CgtpError(f"batch size mismatch: {n_rows} vs {t.shape[0]}")
                n_rows = t.shape[0]
            for i, name in enumerate(ax):
                size = t.shape[t.ndim - len(ax) + i]
                if ext[name] not in (None, size):
                    raise _lib.CgtpError(f"extent mismatch on axis {name}: {ext[name]} vs {size}")
                ext[name] = size
        any_batched = n_rows is not None
        n_rows = 1 if n_rows is None else n_rows
        for name in out_axes:
            if ext[name] is None:
                raise _lib.CgtpError(f"output axis {name} is carried by no operand")
        if single_axis:
            if ext["u"] is None:
                raise _lib.CgtpError("at least one operand must carry a channel axis")
            code = {None: OPERAND_NONE, "": OPERAND_SCALAR, "u": OPERAND_VEC}
            out = kernels.tri_contract(spec.packed(dtype, device), spec.out_size,
                                       *[(t, code[ax]) for t, ax in zip(ops, axes)],
                                       n_rows, ext["u"], dtype, device,
                                       reduce_c=(out_axes == ""), reduce_rows=out_shared)
        else:
            out = _matrix_core_route(spec, ops, axes, out_axes, out_shared, n_rows, dtype) if any_batched else None
            if out is None:
                out = _gen_contract(spec, ops, axes, out_axes, out_shared, n_rows, ext["u"] or 1, ext["w"] or 1,
                                    dtype, device)
        if not out_shared and not any_batched:
            out = out.squeeze(0)  # every operand shared -> result has no batch axis either
        ctx.spec, ctx.axes, ctx.out_axes = spec, axes, out_axes
        ctx.shared = [ax is not None and _is_shared(t, ax) for t, ax in zip(ops, axes)]
        ctx.save_for_backward(*[t for t in ops if t is not None])
        ctx.present = [t is not None for t in ops]
        ctx.in_dtypes = [None if t is None else t.dtype for t in (a, b, w)]
        ctx.in_shapes = [None if t is None else t.shape for t in (a, b, w)]
        return out.to(res_dtype)

    @staticmethod
    def backward(ctx, g):
        saved = list(ctx.saved_tensors)
        ops = [saved.pop(0) if p else None for p in ctx.present]
        grads = [None, None, None]
        for s in range(3):
            if ctx.axes[s] is None or not ctx.needs_input_grad[4 + s]:
                continue
            new_ops, new_axes = list(ops), list(ctx.axes)
            new_ops[s], new_axes[s] = g, ctx.out_axes
            grads[s] = TriContract.apply(ctx.spec.grad_spec(s), tuple(new_axes), ctx.axes[s], ctx.shared[s],
                                         *new_ops).to(ctx.in_dtypes[s])
            if grads[s].shape != ctx.in_shapes[s]:
                # the output was summed over rows and every other operand is shared: the gradient of a batched
                # operand is then the same for every row
                grads[s] = grads[s].expand(ctx.in_shapes[s])
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
            # entries past the last segment are reached by no output row.  The reference's builder leaves such
            # entries behind when the first output row has none (`sparse_product_info`,
            # `equitorch/utils/_structs.py:105-123`, shifts its segment pointers by one row then); its kernels walk
            # the segments and never see them
            i1, i2 = i1[:out_idx.shape[0]], i2[:out_idx.shape[0]]
        if info.out_size is not None:
            n_out = max(n_out, int(info.out_size))
        coef = None if info.scale is None else info.scale.detach().cpu().double().numpy()[:out_idx.shape[0]]
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
