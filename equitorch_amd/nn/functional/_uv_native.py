"""Fully connected products in fp32 with a shared weight on the table-driven matrix-core kernels (``cgtp_uvt_*``):
``tensor_product_u1v`` (``SO3Linear('uv')``) and ``tensor_product_uvw`` (``TensorProduct('uvw')``) for any irreps and
normalisation, forward and first-order gradients, without the reference's ``(N, segments, C)`` intermediate
(``equitorch/nn/functional/linears.py:257-336``, ``tensor_products.py:92-172``).

The kernels walk a flat list of items (segment = (weight path, output row), chunk of the contracted channel axis)
ordered by output row; this module cuts that list from the table for each of the roles a product is used in:

    forward      out[M]   <- first operand rows M1, second operand rows M2, weight as stored
    grad first   g1[M1]   <- rows M of grad_out,   second operand rows M2, weight transposed
    ('uvw' only) g2[M2]   <- rows M of grad_out,   first operand rows M1,  weight permuted
"""
import ctypes as C
from typing import Optional

import numpy as np
import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
from ...ops import kernels

FIRST, LAST = 1, 2


class CooTable:
    """A product table given directly by its coordinates (``coo``: ``TpCoo`` fields M, M1, M2, p, coef and the extents)
    instead of a ``TensorProductInfo`` — the tables of the channel-mixing layers, whose second operand is the scalar 1.
    ``anchor``: a tensor that lives as long as the table (cache key); ``fallback(x, y, w)``: a differentiable
    evaluation of the same product for gradients of higher order."""

    def __init__(self, coo, anchor: Tensor, fallback):
        self.coo, self.anchor, self.fallback = coo, anchor, fallback


def _anchor(table) -> Tensor:
    return table.anchor if isinstance(table, CooTable) else table.info_Mij_fwd.scale
MAX_TERMS = 8      # terms of a segment the weight-gradient kernel holds in registers (kUvtTerms)


class _Coefficients:
    """The coefficients of a walk's terms as a device tensor of the launch's dtype (made on first use)."""

    def term_c(self, dtype: torch.dtype) -> Tensor:
        if dtype not in self._term_c:
            self._term_c[dtype] = torch.from_numpy(np.ascontiguousarray(self._coef, dtype=np.float64)).to(
                device=self._device, dtype=dtype)
        return self._term_c[dtype]


class _Walk(_Coefficients):
    """Item list of one role of one table: one item per segment (weight path, output row), the items of a row
    consecutive, the rows dealt to ``n_groups`` groups of about equal numbers of items (the wavefronts of a workgroup
    take one group each)."""

    def __init__(self, out_idx, a_idx, b_idx, p_idx, coef, n_out: int, n_groups: int, device):
        order = np.lexsort([b_idx, a_idx, p_idx, out_idx])
        out_idx, a_idx, b_idx, p_idx = (np.asarray(v)[order] for v in (out_idx, a_idx, b_idx, p_idx))
        coef = np.asarray(coef, dtype=np.float64)[order]
        rows = []
        t, n_terms = 0, out_idx.shape[0]
        for row in range(n_out):
            items = []
            while t < n_terms and out_idx[t] == row:
                t1 = t
                while t1 < n_terms and out_idx[t1] == row and p_idx[t1] == p_idx[t]:
                    t1 += 1
                items.append([int(p_idx[t]), 0, 0, t, t1, row, 0, 0])
                t = t1
            if not items:                                  # a row without terms is written as zeros
                items.append([0, 0, 0, 0, 0, row, 0, 0])
            items[0][6] |= FIRST
            items[-1][6] |= LAST
            rows.append(items)
        # longest rows first, each to the group with the fewest items so far
        groups = [[] for _ in range(n_groups)]
        for items in sorted(rows, key=len, reverse=True):
            min(groups, key=len).extend(items)
        flat = [it for grp in groups for it in grp]
        self.n_items = len(flat)
        self.group_ptr = np.cumsum([0] + [len(grp) for grp in groups]).tolist()
        self.items = torch.tensor(flat, dtype=torch.int32).reshape(-1, 8).to(device)
        self.term_a = torch.from_numpy(a_idx.astype(np.int32)).to(device)
        self.term_b = torch.from_numpy(b_idx.astype(np.int32)).to(device)
        self._coef, self._device, self._term_c = coef, device, {}


def _walk(tp_info, role: str, n_groups: int, device) -> _Walk:
    def build():
        c = _coo(tp_info)
        if role == "out":        # rows of the first operand, rows of the second operand
            return _Walk(c.M, c.M1, c.M2, c.p, c.coef, c.DO, n_groups, device)
        if role == "in1":        # first operand of the launch = grad_out, second = input2
            return _Walk(c.M1, c.M, c.M2, c.p, c.coef, c.D1, n_groups, device)
        if role == "in1_uvw":    # first operand of the launch = input2, second = grad_out
            return _Walk(c.M1, c.M2, c.M, c.p, c.coef, c.D1, n_groups, device)
        if role == "in2_uvw":    # first operand of the launch = grad_out, second = input1
            return _Walk(c.M2, c.M, c.M1, c.p, c.coef, c.D2, n_groups, device)
        raise ValueError(role)
    return kernels.cached(_anchor(tp_info), ("uvt_walk", role, n_groups, str(device)), build)


class _PathWalk(_Coefficients):
    """Segments (weight path, output row) of a table sorted by path, with their terms: the walk of the weight-gradient
    kernel, which owns one path per workgroup."""

    def __init__(self, coo, device):
        order = np.lexsort([coo.M2, coo.M1, coo.M, coo.p])
        p_idx, m_idx, a_idx, b_idx = (np.asarray(v)[order] for v in (coo.p, coo.M, coo.M1, coo.M2))
        coef = np.asarray(coo.coef, dtype=np.float64)[order]
        items, path_ptr = [], [0]
        t, n_terms = 0, p_idx.shape[0]
        for p in range(coo.P):
            while t < n_terms and p_idx[t] == p:
                t1 = t
                while t1 < n_terms and p_idx[t1] == p and m_idx[t1] == m_idx[t]:
                    t1 += 1
                for tb in range(t, t1, MAX_TERMS):       # the kernel keeps at most MAX_TERMS terms of an item
                    items.append([p, 0, 0, tb, min(tb + MAX_TERMS, t1), int(m_idx[t]), 0, 0])
                t = t1
            path_ptr.append(len(items))
        self.n_items, self.n_terms, self.n_paths = len(items), n_terms, coo.P
        self.items = torch.tensor(items, dtype=torch.int32).reshape(-1, 8).to(device)
        self.path_ptr = torch.tensor(path_ptr, dtype=torch.int32).to(device)
        self.term_a = torch.from_numpy(a_idx.astype(np.int32)).to(device)
        self.term_b = torch.from_numpy(b_idx.astype(np.int32)).to(device)
        self._coef, self._device, self._term_c = coef, device, {}


def grad_w(x: Tensor, y: Tensor, g: Tensor, tp_info) -> Tensor:
    """``gw[p, k, w] = sum_n sum_{(p, M)} inter[n, (p, M), k] g[n, M, w]`` (``cgtp_uvt_grad_w``): ``(P, K, C_out)`` with
    ``K = C_x`` or ``C_x * C_y``; the caller reshapes."""
    walk = kernels.cached(_anchor(tp_info), ("uvt_path_walk", str(x.device)),
                          lambda: _PathWalk(_coo(tp_info), x.device))
    n, dx, cx = x.shape
    dy = y.shape[1]
    cy = y.shape[2] if y.ndim == 3 else 0
    k = cx * cy if cy else cx
    cout = g.shape[-1]
    gw = torch.empty((walk.n_paths, k, cout), dtype=x.dtype, device=x.device)
    ws = torch.empty(max(int(_lib.lib.cgtp_uvt_grad_w_workspace_bytes(n, walk.n_paths, k, cout, _lib.dtype_code(x.dtype))), 16), dtype=torch.uint8,
                     device=x.device)
    a = _lib.UvtGwArgs()
    a.x, a.y, a.g, a.gw, a.workspace = x.data_ptr(), y.data_ptr(), g.data_ptr(), gw.data_ptr(), ws.data_ptr()
    a.items, a.path_ptr = walk.items.data_ptr(), walk.path_ptr.data_ptr()
    a.term_a, a.term_b, a.term_c = walk.term_a.data_ptr(), walk.term_b.data_ptr(), walk.term_c(x.dtype).data_ptr()
    a.n_rows, a.n_items, a.n_terms, a.n_paths = n, walk.n_items, walk.n_terms, walk.n_paths
    a.dx, a.dy, a.dg, a.cx, a.cy, a.cout, a.dtype = dx, dy, g.shape[1], cx, cy, cout, _lib.dtype_code(x.dtype)
    _lib.check(_lib.lib.cgtp_uvt_grad_w(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvt_grad_w")
    return gw


class _SegWalk(_Coefficients):
    """Segments (weight path, row of the first operand) with their terms (row of grad_out, row of the second operand):
    the walk of ``cgtp_uvt_grad_y``.  Segments are not split: the kernel forms one matrix product per segment."""

    def __init__(self, coo, device):
        order = np.lexsort([coo.M, coo.M2, coo.M1, coo.p])
        p_idx, a_idx, b_idx, m_idx = (np.asarray(v)[order] for v in (coo.p, coo.M1, coo.M2, coo.M))
        coef = np.asarray(coo.coef, dtype=np.float64)[order]
        items = []
        t, n_terms = 0, p_idx.shape[0]
        while t < n_terms:
            t1 = t
            while t1 < n_terms and p_idx[t1] == p_idx[t] and a_idx[t1] == a_idx[t]:
                t1 += 1
            items.append([int(p_idx[t]), 0, 0, t, t1, int(a_idx[t]), 0, 0])
            t = t1
        # longest segments first: the wavefront groups take segments round robin
        items.sort(key=lambda it: it[3] - it[4])
        self.n_items, self.n_terms = len(items), n_terms
        self.items = torch.tensor(items, dtype=torch.int32).reshape(-1, 8).to(device)
        self.term_m = torch.from_numpy(m_idx.astype(np.int32)).to(device)
        self.term_b = torch.from_numpy(b_idx.astype(np.int32)).to(device)
        self._coef, self._device, self._term_c = coef, device, {}


def grad_y_supported(n: int, dx: int, dy: int, cx: int, cout: int, tp_info, itemsize: int = 4) -> bool:
    """Whether the 16 staged samples of a ``cgtp_uvt_grad_y`` workgroup and its tables fit the LDS."""
    c = _coo(tp_info)
    kx = ((cx + 15) // 16 + 3) // 4 * 4 * 16
    # one 32-byte item per (weight path, row of the first operand) segment, 8 bytes + a coefficient per term
    n_items = kernels.cached(_anchor(tp_info), "uvt_seg_count",
                             lambda: len(set(zip(np.asarray(c.p).tolist(), np.asarray(c.M1).tolist()))))
    lds = (16 * (dx * kx + 4) + 8 * 16 * dy) * itemsize + n_items * 32 + len(c.coef) * (8 + itemsize) + 16
    return cx % 4 == 0 and cout % 4 == 0 and lds <= 160 * 1024


def grad_y(x: Tensor, g: Tensor, wp: Tensor, tp_info, dy: int) -> Tensor:
    """``gy[n, b] = sum_t c_t <g[n, M_t, :], x[n, a_t, :] @ W[p_t]>`` (``cgtp_uvt_grad_y``); ``wp``: the weight as packed
    for the forward."""
    walk = kernels.cached(_anchor(tp_info), ("uvt_seg_walk", str(x.device)),
                          lambda: _SegWalk(_coo(tp_info), x.device))
    n, dx, cx = x.shape
    gy = torch.empty((n, dy), dtype=x.dtype, device=x.device)
    a = _lib.UvtGyArgs()
    a.x, a.g, a.wp, a.gy = x.data_ptr(), g.data_ptr(), wp.data_ptr(), gy.data_ptr()
    a.items, a.term_m, a.term_b, a.term_c = (walk.items.data_ptr(), walk.term_m.data_ptr(), walk.term_b.data_ptr(),
                                             walk.term_c(x.dtype).data_ptr())
    a.n_rows, a.n_items, a.n_terms = n, walk.n_items, walk.n_terms
    a.dx, a.dy, a.dg, a.cx, a.cout, a.dtype = dx, dy, g.shape[1], cx, g.shape[2], _lib.dtype_code(x.dtype)
    _lib.check(_lib.lib.cgtp_uvt_grad_y(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvt_grad_y")
    return gy


def chunk_of(n_rows: int, dx: int, dy: int, dout: int, cx: int, cy: int, cout: int, dtype=torch.float32) -> int:
    """Blocks of 16 contracted channels a launch with these extents pads to; <= 0: the kernels do not take them
    (channel counts not multiples of 4, rows of 16 samples beyond the LDS)."""
    return int(_lib.lib.cgtp_uvt_chunk(n_rows, dx, dy, dout, cx, cy, cout, _lib.dtype_code(dtype)))


def pack(w: Tensor, n_paths: int, k: int, cout: int, stride_p: int, stride_k: int, stride_c: int) -> Tensor:
    """The weight viewed as ``(n_paths, k, cout)`` through element strides, in matrix-core fragment order."""
    packed = torch.empty(int(_lib.lib.cgtp_uvt_packed_elems(n_paths, k, cout)), dtype=w.dtype, device=w.device)
    _lib.check(_lib.lib.cgtp_uvt_pack_weights(w.data_ptr(), packed.data_ptr(), n_paths, k, cout, stride_p, stride_k,
                                              stride_c, _lib.dtype_code(w.dtype), _lib.stream_ptr(w.device)), "cgtp_uvt_pack_weights")
    return packed


def apply(x: Tensor, y: Tensor, wp: Tensor, tp_info, role: str, dout: int, cout: int) -> Tensor:
    """One launch of ``cgtp_uvt_apply``: ``x (N, dx, cx)``, ``y (N, dy)`` or ``(N, dy, cy)`` -> ``(N, dout, cout)``."""
    n, dx, cx = x.shape
    dy = y.shape[1]
    cy = y.shape[2] if y.ndim == 3 else 0
    k = cx * cy if cy else cx
    kbi = chunk_of(n, dx, dy, dout, cx, cy, cout, x.dtype)
    if kbi <= 0:
        raise _lib.CgtpError(f"cgtp_uvt_apply does not take these extents (status {-kbi})")
    n_groups = int(_lib.lib.cgtp_uvt_item_groups(n, dx, dy, dout, cx, cy, cout, _lib.dtype_code(x.dtype)))
    walk = _walk(tp_info, role, n_groups, x.device)
    out = torch.empty((n, dout, cout), dtype=x.dtype, device=x.device)
    if n == 0:
        return out
    a = _lib.UvtArgs()
    a.x, a.y, a.wp, a.out = x.data_ptr(), y.data_ptr(), wp.data_ptr(), out.data_ptr()
    a.items, a.term_a, a.term_b, a.term_c = (walk.items.data_ptr(), walk.term_a.data_ptr(), walk.term_b.data_ptr(),
                                             walk.term_c(x.dtype).data_ptr())
    a.n_rows, a.n_items, a.n_terms = n, walk.n_items, walk.term_a.shape[0]
    a.dx, a.dy, a.dout, a.cx, a.cy, a.cout = dx, dy, dout, cx, cy, cout
    a.kbi, a.dtype = kbi, _lib.dtype_code(x.dtype)
    a.n_groups = n_groups
    for i, v in enumerate(walk.group_ptr):
        a.group_ptr[i] = v
    _lib.check(_lib.lib.cgtp_uvt_apply(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvt_apply")
    return out


def _coo(tp_info):
    return tp_info.coo if isinstance(tp_info, CooTable) else kernels.coo_of(tp_info)


def _aligned(g: Tensor) -> Tensor:
    """The incoming gradient as the kernels want it: contiguous and on a 16-byte boundary.  Autograd may hand over a
    view into a larger buffer (the gradient of a ``cat`` or of a slice), contiguous but at any element offset."""
    g = g.contiguous()
    return g.clone() if g.data_ptr() % 16 else g


class _U1vNative(Function):
    """u1v, shared fp32 weight ``(P, U, W)``.  The gradient of the first operand is the forward kernel with the rows'
    roles exchanged and the weight read transposed; the gradients of the weight and of the second operand have
    kernels of their own (``cgtp_uvt_grad_w``, ``cgtp_uvt_grad_y``).  Under ``create_graph`` the backward is the
    differentiable two-stage route of ``_uv_gemm``."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info):
        c = _coo(tp_info)
        p, u, wc = w.shape
        out = apply(x, y, pack(w, p, u, wc, u * wc, wc, 1), tp_info, "out", c.DO, wc)
        ctx.save_for_backward(x, y, w)
        ctx.tp_info = tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        from . import _uv_gemm
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        tp_info = ctx.tp_info
        if torch.is_grad_enabled():       # higher-order derivative: the differentiable route throughout
            with torch.enable_grad():
                out = tp_info.fallback(x, y, w) if isinstance(tp_info, CooTable) else _uv_gemm.u1v(x, y, w, tp_info)
                wanted = [t for t, n in zip((x, y, w), need) if n]
                got = iter(torch.autograd.grad(out, wanted, g, create_graph=True, allow_unused=True))
            return tuple(next(got) if n else None for n in need) + (None,)
        c = _coo(tp_info)
        p, u, wc = w.shape
        gx = gy = gw = None
        g = _aligned(g)
        if need[0]:
            gx = apply(g, y, pack(w, p, wc, u, u * wc, 1, wc), tp_info, "in1", c.D1, u)
        if need[2]:
            gw = grad_w(x, y, g, tp_info)
        if need[1]:
            gy = grad_y(x, g, pack(w, p, u, wc, u * wc, wc, 1), tp_info, c.D2)
        return gx, gy, gw, None


def u1v_supported(x: Tensor, y: Tensor, w: Tensor, tp_info) -> bool:
    if not (x.dtype == y.dtype == w.dtype and x.dtype in (torch.float32, torch.float64) and x.ndim == 3 and y.ndim == 2
            and w.ndim == 3):
        return False
    if x.shape[0] == 0:
        return False
    c = _coo(tp_info)
    _, u, wc = w.shape
    n = x.shape[0]
    dt = x.dtype
    if tuple(x.shape) != (n, c.D1, u) or tuple(y.shape) != (n, c.D2) or w.shape[0] != c.P:
        raise _lib.CgtpError(f"operands {tuple(x.shape)}, {tuple(y.shape)}, {tuple(w.shape)} do not fit the table: "
                             f"expected (N, {c.D1}, U), (N, {c.D2}), ({c.P}, U, W)")
    return u1v_fits(n, u, wc, tp_info, dt) and x.data_ptr() % 16 == 0


def u1v_fits(n: int, u: int, wc: int, tp_info, dtype: torch.dtype) -> bool:
    """Whether the forward, the gradient of the channelled operand and the gradient of the second operand have a launch
    shape for ``n`` samples, ``u -> wc`` channels in ``dtype`` (float32 | float64): extents only, no tensors."""
    c = _coo(tp_info)
    size = torch.empty(0, dtype=dtype).element_size()
    return (n > 0 and chunk_of(n, c.D1, c.D2, c.DO, u, 0, wc, dtype) > 0
            and chunk_of(n, c.DO, c.D2, c.D1, wc, 0, u, dtype) > 0
            and grad_y_supported(n, c.D1, c.D2, u, wc, tp_info, size))


def u1v(x: Tensor, y: Tensor, w: Tensor, tp_info) -> Tensor:
    return _U1vNative.apply(x.contiguous(), y.contiguous(), w.contiguous(), tp_info)


# ---- 1vu: the channels on the second operand — u1v on the table with the operands' rows exchanged -------------------
def operands_exchanged(tp_info) -> CooTable:
    def build():
        from . import _uv_gemm
        c = _coo(tp_info)
        return CooTable(c._replace(M1=c.M2, M2=c.M1, D1=c.D2, D2=c.D1), torch.zeros(1),
                        lambda xx, yy, ww: _uv_gemm.one_vu(yy, xx, ww, tp_info))
    return kernels.cached(_anchor(tp_info), "1vu_table", build)


# ---- vu1: out[n, M] = sum_t c_t <y[n, b_t, :], x[n, a_t, :] @ W[p_t]> ---------------------------------------------
# With the table's output rows and second-operand rows exchanged (T'), this is the gradient of u1v_T' with respect to
# its channel-less operand for the cotangent y — the kernel cgtp_uvt_grad_y — and its own gradients are the forward
# (grad y), the input gradient (grad x) and the weight gradient of u1v_T' with the cotangent of vu1 as the channel-less
# operand.  The reference computes it in three stages, weight first (equitorch/nn/functional/linears.py:414-492).
def _swapped(tp_info) -> CooTable:
    def build():
        c = _coo(tp_info)
        return CooTable(c._replace(M=c.M2, M2=c.M, D2=c.DO, DO=c.D2), torch.zeros(1), None)
    return kernels.cached(_anchor(tp_info), "vu1_table", build)


class _Vu1Native(Function):
    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info):
        t = _swapped(tp_info)
        p, u, wc = w.shape
        out = grad_y(x, y, pack(w, p, u, wc, u * wc, wc, 1), t, t.coo.D2)
        ctx.save_for_backward(x, y, w)
        ctx.tp_info = tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        from . import _uv_gemm
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        if torch.is_grad_enabled():       # higher-order derivative: the differentiable route throughout
            with torch.enable_grad():
                out = _uv_gemm.vu1(x, y, w, ctx.tp_info)
                wanted = [v for v, n in zip((x, y, w), need) if n]
                got = iter(torch.autograd.grad(out, wanted, g, create_graph=True, allow_unused=True))
            return tuple(next(got) if n else None for n in need) + (None,)
        t = _swapped(ctx.tp_info)
        c = t.coo
        p, u, wc = w.shape
        g = _aligned(g)
        gx = apply(y, g, pack(w, p, wc, u, u * wc, 1, wc), t, "in1", c.D1, u) if need[0] else None
        gy = apply(x, g, pack(w, p, u, wc, u * wc, wc, 1), t, "out", c.DO, wc) if need[1] else None
        gw = grad_w(x, g, y, t) if need[2] else None
        return gx, gy, gw, None


def vu1_supported(x: Tensor, y: Tensor, w: Tensor, tp_info) -> bool:
    if not (x.dtype == y.dtype == w.dtype and x.dtype in (torch.float32, torch.float64) and x.ndim == 3 and y.ndim == 3
            and w.ndim == 3 and x.shape[0] > 0):
        return False
    c = _coo(tp_info)
    n, (_, u, wc) = x.shape[0], w.shape
    if tuple(x.shape) != (n, c.D1, u) or tuple(y.shape) != (n, c.D2, wc) or w.shape[0] != c.P:
        raise _lib.CgtpError(f"operands {tuple(x.shape)}, {tuple(y.shape)}, {tuple(w.shape)} do not fit the table: "
                             f"expected (N, {c.D1}, C1), (N, {c.D2}, C2), ({c.P}, C1, C2)")
    return u1v_fits(n, u, wc, _swapped(tp_info), x.dtype) and x.data_ptr() % 16 == 0 and y.data_ptr() % 16 == 0


def vu1(x: Tensor, y: Tensor, w: Tensor, tp_info) -> Tensor:
    return _Vu1Native.apply(x.contiguous(), y.contiguous(), w.contiguous(), tp_info)


class _UvwNative(Function):
    """uvw, shared fp32 weight ``(P, U, V, W)``: forward and the gradients of both operands on ``cgtp_uvt_apply``
    (with the weight permuted as the reference permutes it, ``tensor_products.py:126-150``); the weight gradient and
    higher orders from the two-stage route of ``_uvw_gemm``."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info):
        c = _coo(tp_info)
        p, u, v, wc = w.shape
        out = apply(x, y, pack(w, p, u * v, wc, u * v * wc, wc, 1), tp_info, "out", c.DO, wc)
        ctx.save_for_backward(x, y, w)
        ctx.tp_info = tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        from . import _uvw_gemm
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        tp_info = ctx.tp_info
        if torch.is_grad_enabled():
            with torch.enable_grad():
                out = _uvw_gemm.uvw(x, y, w, tp_info)
                wanted = [t for t, n in zip((x, y, w), need) if n]
                got = iter(torch.autograd.grad(out, wanted, g, create_graph=True, allow_unused=True))
            return tuple(next(got) if n else None for n in need) + (None,)
        c = _coo(tp_info)
        p, u, v, wc = w.shape
        g = _aligned(g)
        gx = gy = gw = None
        if need[0]:     # first operand of the launch: y (channels v), second: grad_out (channels w); weight (P, V, W, U)
            wt = w.permute(0, 2, 3, 1).contiguous()
            gx = apply(y, g, pack(wt, p, v * wc, u, v * wc * u, u, 1), tp_info, "in1_uvw", c.D1, u)
        if need[1]:     # first: grad_out (channels w), second: x (channels u); weight (P, W, U, V)
            wt = w.permute(0, 3, 1, 2).contiguous()
            gy = apply(g, x, pack(wt, p, wc * u, v, wc * u * v, v, 1), tp_info, "in2_uvw", c.D2, v)
        if need[2]:
            gw = grad_w(x, y, g, tp_info).view(p, u, v, wc)
        return gx, gy, gw, None


def uvw_supported(x: Tensor, y: Tensor, w: Tensor, tp_info) -> bool:
    if not (x.dtype == y.dtype == w.dtype and x.dtype in (torch.float32, torch.float64) and x.ndim == 3 and y.ndim == 3
            and w.ndim == 4):
        return False
    if x.shape[0] == 0:
        return False
    c = _coo(tp_info)
    _, u, v, wc = w.shape
    n = x.shape[0]
    dt = x.dtype
    if tuple(x.shape) != (n, c.D1, u) or tuple(y.shape) != (n, c.D2, v) or w.shape[0] != c.P:
        raise _lib.CgtpError(f"operands {tuple(x.shape)}, {tuple(y.shape)}, {tuple(w.shape)} do not fit the table: "
                             f"expected (N, {c.D1}, U), (N, {c.D2}, V), ({c.P}, U, V, W)")
    return uvw_fits(n, u, v, wc, tp_info, dt) and x.data_ptr() % 16 == 0 and y.data_ptr() % 16 == 0


def uvw_fits(n: int, u: int, v: int, wc: int, tp_info, dtype: torch.dtype) -> bool:
    """The same for the product with channels on both operands."""
    c = _coo(tp_info)
    return (n > 0 and chunk_of(n, c.D1, c.D2, c.DO, u, v, wc, dtype) > 0
            and chunk_of(n, c.D2, c.DO, c.D1, v, wc, u, dtype) > 0 and chunk_of(n, c.DO, c.D1, c.D2, wc, u, v, dtype) > 0)


def uvw(x: Tensor, y: Tensor, w: Tensor, tp_info) -> Tensor:
    return _UvwNative.apply(x.contiguous(), y.contiguous(), w.contiguous(), tp_info)
