"""Fully connected products with a weight per sample on the streaming kernels (``cgtp_psw_fwd`` / ``cgtp_psw_bwd``):
one launch forward, one backward, the weight read once and its gradient written once, the coupled operand formed in
LDS — no ``(N, segments, C_in)`` intermediate in memory and no library GEMM.

The reference takes a weight with a batch axis through the same two launches as a shared one (per-sample detection
``equitorch/nn/tensor_products.py:152-155``; ``equitorch/nn/functional/linears.py:254-412`` for u1v / 1vu,
``equitorch/nn/functional/tensor_products.py:95-158`` for uvw, ``linears.py:494-571`` for the channel mixing between
irreps).

The kernels walk the table in blocks of output rows: the row ranges of the weight paths, overlapping ranges merged.
For the tables ``tp_infos`` / ``irreps_linear_infos`` / ``irreps_info`` build a block is one output irrep; a table
whose blocks exceed ``MAX_BLOCK_ROWS`` rows is left to the library route.
"""
import ctypes as C
from typing import Callable, Optional

import numpy as np
import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
from ...ops import kernels

_END_ROW = 1 << 24
_NO_TERM = 1 << 25       # the path has no term for this row: the entry only closes the (zero) row
MAX_BLOCK_ROWS = 32      # 16 rows per pass; every further pass streams the block's weights again


class PswTable:
    """The walk of a table for the streaming kernels, as device arrays.  ``a`` / ``b``: row of the first (channelled)
    and of the second operand per table entry."""

    def __init__(self, out_row, a, b, path, coef, d1: int, d2: int, d_out: int, n_paths: int, device):
        out_row, a, b, path = (np.asarray(v, dtype=np.int64) for v in (out_row, a, b, path))
        coef = np.asarray(coef, dtype=np.float64)
        if max(d1, d2) > 255:
            raise ValueError("operand rows beyond 255")
        # blocks: row ranges of the paths, ranges that overlap merged into one (an output irrep and all paths into it;
        # for the SO(2) tables, whose weights couple the rows +m and -m, all orders of an output irrep)
        spans = sorted((int(out_row[path == p].min()), int(out_row[path == p].max()) + 1, int(p)) for p in np.unique(path))
        blocks_of = {}
        lo, hi, members = spans[0][0], spans[0][1], []
        for a0, a1, p in spans:
            if a0 >= hi:
                blocks_of[(lo, hi - lo)] = members
                lo, hi, members = a0, a1, []
            hi = max(hi, a1)
            members.append(p)
        blocks_of[(lo, hi - lo)] = members
        if max(rows for _, rows in blocks_of) > MAX_BLOCK_ROWS:
            raise ValueError("a block of more rows than the kernels take in two passes")
        words, coefs, slots, blocks = [], [], [], []
        for (m0, rows), paths in sorted(blocks_of.items()):
            q0 = len(slots)
            for p in paths:
                sel = np.nonzero(path == p)[0]
                e0 = len(words)
                for j in range(rows):
                    hit = sel[out_row[sel] == m0 + j]
                    if hit.size == 0:                      # keeps the row of the coupled operand defined: zero
                        words.append(j | _END_ROW | _NO_TERM)
                        coefs.append(0.0)
                        continue
                    for i, t in enumerate(hit):
                        words.append(j | int(a[t]) << 8 | int(b[t]) << 16 | (_END_ROW if i == hit.size - 1 else 0))
                        coefs.append(float(coef[t]))
                slots.append((p, e0, len(words)))
            blocks.append((m0, rows, q0, len(slots)))
        self.covers_output = sum(rows for _, rows, _, _ in blocks) == d_out
        # weight paths without an entry (the reference's tables can leave one out: `sparse_product_info`,
        # `equitorch/utils/_structs.py:105-123`, shifts its segments when the first output row has no entry): the
        # kernels never visit them, so their gradient is written here
        self.unwalked_paths = sorted(set(range(int(n_paths))) - set(int(p) for p in np.unique(path)))
        self.device = device
        self.entries = torch.tensor(words, dtype=torch.int64).to(torch.int32).to(device)     # bit 24 at most: fits
        self._coef64 = torch.tensor(coefs, dtype=torch.float64)
        self._coef = {}
        self.slots = torch.tensor(slots, dtype=torch.int32).reshape(-1, 3).to(device)
        self.blocks = torch.tensor(blocks, dtype=torch.int32).reshape(-1, 4).to(device)
        self.dims = (int(d1), int(d2), int(d_out), int(n_paths))
        self.max_rows = max(rows for _, rows, _, _ in blocks)
        self.launchable = {}                 # memo of launchable(): extents and dtype -> bool

    def coef(self, dtype) -> Tensor:
        if dtype not in self._coef:
            self._coef[dtype] = self._coef64.to(device=self.device, dtype=dtype)
        return self._coef[dtype]

    def c_table(self, dtype) -> _lib.PswTable:
        d1, d2, d_out, n_paths = self.dims
        return _lib.PswTable(self.entries.data_ptr(), self.coef(dtype).data_ptr(), self.slots.data_ptr(),
                             self.blocks.data_ptr(), self.entries.shape[0], self.slots.shape[0], self.blocks.shape[0],
                             self.max_rows, d1, d2, d_out, n_paths)


def table_of_coo(coo, anchor: Tensor, channelled: int, device) -> Optional[PswTable]:
    """Walk of a product table (``TpCoo`` fields); ``channelled``: which operand carries the input channels of the
    weight (1: u1v, uvw, channel mixing; 2: 1vu — the operands then change places).  None when the table does not have
    the structure the kernels walk."""
    def build():
        try:
            if channelled == 1:
                return PswTable(coo.M, coo.M1, coo.M2, coo.p, coo.coef, coo.D1, coo.D2, coo.DO, coo.P, device)
            return PswTable(coo.M, coo.M2, coo.M1, coo.p, coo.coef, coo.D2, coo.D1, coo.DO, coo.P, device)
        except ValueError:
            return False
    table = kernels.cached(anchor, ("psw_table", channelled, str(device)), build)
    return None if table is False else table


def _args(table: PswTable, x: Tensor, y: Optional[Tensor], w: Tensor):
    args = _lib.PswArgs()
    args.x, args.y, args.w = x.data_ptr(), (0 if y is None else y.data_ptr()), w.data_ptr()
    args.n_rows = x.shape[0]
    args.cx = x.shape[2]
    args.cy = 1 if y is None or y.ndim == 2 else y.shape[2]
    args.cout = w.shape[-1]
    args.dtype = _lib.dtype_code(x.dtype)
    return args


def launchable(table: Optional[PswTable], x: Tensor, y: Optional[Tensor], w: Tensor) -> bool:
    """fp32 / fp64 operands of one dtype on one GPU, a weight ``(N, P, K, C_out)`` with ``K`` the product of the
    operands' channel counts, extents the table reaches, and a launch shape the kernels have (``cgtp_psw_validate``)."""
    if table is None or not x.is_cuda or x.dtype not in (torch.float32, torch.float64):
        return False
    d1, d2, _, n_paths = table.dims
    if x.ndim != 3 or w.ndim != 4 or w.dtype != x.dtype or x.shape[0] == 0:
        return False
    if y is not None and (y.dtype != x.dtype or y.ndim not in (2, 3) or y.shape[0] != x.shape[0] or y.shape[1] != d2):
        return False
    if y is None and d2 != 1:
        return False
    cy = 1 if y is None or y.ndim == 2 else y.shape[2]
    if x.shape[1] != d1 or tuple(w.shape[:3]) != (x.shape[0], n_paths, x.shape[2] * cy):
        return False
    # the answer depends on the extents, the dtype and the 16-byte alignment of the weight only
    key = (x.dtype, x.shape[0], x.shape[2], cy, w.shape[-1], y is None, w.data_ptr() % 16)
    hit = table.launchable.get(key)
    if hit is None:
        args, c_table = _args(table, x, y, w), table.c_table(x.dtype)
        args.out = args.g = 256                # the real buffers are fresh allocations (aligned)
        hit = (_lib.lib.cgtp_psw_validate(C.byref(args), C.byref(c_table), 0) == 0
               and _lib.lib.cgtp_psw_validate(C.byref(args), C.byref(c_table), 1) == 0)
        if len(table.launchable) > 256:
            table.launchable.clear()
        table.launchable[key] = hit
    return hit


class _Product(Function):
    """``fallback(x, y, w)``: a differentiable evaluation of the same product, used when a gradient of higher order is
    asked for."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Optional[Tensor], w: Tensor, table: PswTable, fallback: Callable):
        d_out = table.dims[2]
        out = (torch.empty if table.covers_output else torch.zeros)(
            (x.shape[0], d_out, w.shape[-1]), dtype=x.dtype, device=x.device)
        args, c_table = _args(table, x, y, w), table.c_table(x.dtype)
        args.out = out.data_ptr()
        _lib.check(_lib.lib.cgtp_psw_fwd(C.byref(args), C.byref(c_table), _lib.stream_ptr(x.device)),
                   "cgtp_psw_fwd")
        ctx.save_for_backward(x, y, w)
        ctx.table, ctx.fallback = table, fallback
        return out

    @staticmethod
    def backward(ctx, g: Tensor):
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        if torch.is_grad_enabled():
            with torch.enable_grad():
                inputs = [t for t, n in zip((x, y, w), need) if n]
                grads = iter(torch.autograd.grad(ctx.fallback(x, y, w), inputs, g, create_graph=True))
            return tuple(next(grads) if n else None for n in need) + (None, None)
        g = g.contiguous()
        if g.data_ptr() % 16:
            g = g.clone()
        gx = torch.empty_like(x) if need[0] else None
        gy = torch.empty_like(y) if need[1] and y is not None else None
        gw = torch.empty_like(w) if need[2] else None
        if gw is not None:
            for p in ctx.table.unwalked_paths:
                gw[:, p].zero_()
        args, c_table = _args(ctx.table, x, y, w), ctx.table.c_table(x.dtype)
        args.g = g.data_ptr()
        args.gx, args.gy, args.gw = (0 if t is None else t.data_ptr() for t in (gx, gy, gw))
        _lib.check(_lib.lib.cgtp_psw_bwd(C.byref(args), C.byref(c_table), _lib.stream_ptr(x.device)),
                   "cgtp_psw_bwd")
        return gx, gy, gw, None, None


def product(table: PswTable, x: Tensor, y: Optional[Tensor], w: Tensor, fallback: Callable) -> Tensor:
    """``x (N, D1, U)``, ``y (N, D2) | (N, D2, V) | None``, ``w (N, P, U * V, C_out)`` -> ``(N, DO, C_out)``; call only
    after :func:`launchable`."""
    return _Product.apply(x.contiguous(), None if y is None else y.contiguous(), w.contiguous(), table, fallback)
