"""Thin, allocation-owning Python launchers over the C ABI (``include/cgtp.h``).

Everything here takes contiguous CUDA (ROCm) tensors, allocates outputs / workspaces with torch, and
enqueues on torch's current stream.
"""
from __future__ import annotations

import ctypes as C
import weakref
from typing import Optional, Tuple

import numpy as np
import torch
from torch import Tensor

from .. import _lib
from .._lib import OPERAND_NONE, OPERAND_SCALAR, OPERAND_VEC, Operand, TriArgs, UvuArgs
from .._tables import TpCoo, fingerprint, pack_tri_table, tp_coo

# ---- per-table caches (keyed by the identity of a table tensor; dropped with it) --------------------------
_CACHE = {}


def cached(anchor: Tensor, key, build):
    """Memoise ``build()`` per (anchor tensor identity, key); the entry dies with the anchor tensor."""
    k = (id(anchor), key)
    hit = _CACHE.get(k)
    if hit is not None and hit[0]() is anchor:
        return hit[1]
    val = build()
    ident = id(anchor)
    ref = weakref.ref(anchor, lambda _r, k=k: _CACHE.pop(k, None))
    _CACHE[k] = (ref, val)
    return val


def coo_of(tp_info) -> TpCoo:
    return cached(tp_info.info_Mij_fwd.scale, "coo", lambda: tp_coo(tp_info))


def uvu_config_of(tp_info) -> int:
    """Index of the compiled-in table equal to this ``tp_info`` (fp32 coefficient bits), or -1."""
    return cached(tp_info.info_Mij_fwd.scale, "cfg",
                  lambda: int(_lib.lib.cgtp_uvu_find(C.c_uint64(fingerprint(coo_of(tp_info))))))


# ---- operands ---------------------------------------------------------------------------------------------
def _operand(t: Optional[Tensor], kind: int, rows: Optional[Tensor] = None) -> Operand:
    op = Operand()
    if t is None or kind == OPERAND_NONE:
        op.kind = OPERAND_NONE
        return op
    full = 3 if kind == OPERAND_VEC else 2
    if t.ndim == full:
        op.row_stride, op.idx_stride = t.stride(0), t.stride(1)
    elif t.ndim == full - 1:
        op.row_stride, op.idx_stride = 0, t.stride(0)
    else:
        raise _lib.CgtpError(f"operand of kind {kind} must have {full} or {full - 1} dims, got {t.ndim}")
    if kind == OPERAND_VEC and t.stride(-1) != 1:
        raise _lib.CgtpError("channel axis must be contiguous")
    op.data = t.data_ptr()
    op.rows = _lib.ptr(rows)
    op.kind = kind
    return op


def tri_contract(table: dict, n_out: int, a: Tuple[Optional[Tensor], int], b: Tuple[Optional[Tensor], int],
                 w: Tuple[Optional[Tensor], int], n_rows: int, channels: int, dtype: torch.dtype, device,
                 reduce_c: bool = False, reduce_rows: bool = False,
                 rows_a: Optional[Tensor] = None, rows_b: Optional[Tensor] = None,
                 rows_w: Optional[Tensor] = None) -> Tensor:
    """``out[r,o,c] = sum_t coef_t A[r,ia_t,c] B[r,ib_t,(c)] W[r,iw_t,c]`` with the packed ``table``."""
    args = TriArgs()
    args.a, args.b, args.w = _operand(*a, rows_a), _operand(*b, rows_b), _operand(*w, rows_w)
    args.coef, args.idx, args.seg = _lib.ptr(table["coef"]), table["idx"].data_ptr(), table["seg"].data_ptr()
    args.n_out, args.nnz = n_out, table["idx"].shape[0]
    shape = ((n_out,) if reduce_c else (n_out, channels))
    if not reduce_rows:
        shape = (n_rows,) + shape
    out = torch.empty(shape, dtype=dtype, device=device)
    args.out, args.n_rows, args.C = out.data_ptr(), n_rows, channels
    args.dtype, args.reduce_c, args.reduce_rows = _lib.dtype_code(dtype), int(reduce_c), int(reduce_rows)
    ws = None
    if reduce_rows:
        nbytes = int(_lib.lib.cgtp_tri_workspace_bytes(C.byref(args)))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=device)
        args.workspace = ws.data_ptr()
    _lib.check(_lib.lib.cgtp_tri_contract(C.byref(args), _lib.stream_ptr(device)), "cgtp_tri_contract")
    return out


def segment_sum(inp: Tensor, scale: Optional[Tensor], index: Optional[Tensor], seg: Optional[Tensor],
                out_size: int) -> Tensor:
    """``out[n,m,c] = sum_{t in seg m} scale[t] * inp[n, index[t], c]`` (``seg=None``: one term per row)."""
    _lib.require_gpu(inp, scale, index, seg)
    inp = inp.contiguous()
    n, in_size, ch = inp.shape
    out = torch.empty((n, out_size, ch), dtype=inp.dtype, device=inp.device)
    n_seg = out_size if seg is None else seg.shape[0] - 1
    if n_seg < out_size:
        out.zero_()
    if scale is not None:
        scale = scale.to(inp.dtype).contiguous()
    _lib.check(_lib.lib.cgtp_segment_sum(inp.data_ptr(), _lib.ptr(scale), _lib.ptr(index), _lib.ptr(seg),
                                          out.data_ptr(), n, in_size, min(n_seg, out_size), ch,
                                          _lib.dtype_code(inp.dtype), _lib.stream_ptr(inp.device)),
               "cgtp_segment_sum")
    return out


# ---- specialised uvu ----------------------------------------------------------------------------------------
def _uvu_args(cfg: int, x: Tensor, y: Tensor, w: Tensor, n_rows: int, ptr_, perm, gather) -> UvuArgs:
    a = UvuArgs()
    a.cfg, a.dtype, a.C = cfg, _lib.dtype_code(x.dtype), x.shape[-1]
    a.w_shared = int(w.ndim == 2)
    a.n_rows, a.n_x_rows = n_rows, x.shape[0]
    a.n_seg = 0 if ptr_ is None else ptr_.shape[0] - 1
    a.ptr, a.perm, a.gather = _lib.ptr(ptr_), _lib.ptr(perm), _lib.ptr(gather)
    a.x, a.y, a.w = x.data_ptr(), y.data_ptr(), w.data_ptr()
    return a


def uvu_launchable(cfg: int, x: Tensor, y: Tensor, w: Tensor, segments: bool = False) -> bool:
    """True when both the specialised forward and backward accept these operands (dtype, channel count,
    alignment); outputs are torch allocations and therefore always aligned."""
    a = UvuArgs()
    a.cfg, a.dtype, a.C = cfg, _lib.dtype_code(x.dtype), x.shape[-1]
    a.w_shared = int(w.ndim == 2)
    a.n_rows = y.shape[0]
    dummy = 256
    if segments:
        a.n_seg, a.n_x_rows, a.ptr, a.gather = x.shape[0], x.shape[0], dummy, dummy
    else:
        a.n_x_rows = x.shape[0]
    a.x, a.y, a.w = x.data_ptr() or dummy, y.data_ptr() or dummy, w.data_ptr() or dummy
    a.out = a.grad_out = a.grad_x = a.grad_y = a.grad_w = a.workspace = dummy
    if x.shape[0] == 0 or y.shape[0] == 0:
        return False
    if _lib.lib.cgtp_uvu_validate(C.byref(a), 1) != 0:
        return False
    return True


def uvu_forward(cfg: int, dims, x: Tensor, y: Tensor, w: Tensor, ptr_: Optional[Tensor] = None,
                perm: Optional[Tensor] = None, gather: Optional[Tensor] = None) -> Optional[Tensor]:
    """Specialised forward; returns None when the launch conditions are not met (caller falls back to the
    table-driven kernel)."""
    n_rows = y.shape[0]
    a = _uvu_args(cfg, x, y, w, n_rows, ptr_, perm, gather)
    n_out_rows = a.n_seg if ptr_ is not None else n_rows
    out = torch.empty((n_out_rows, dims[2], x.shape[-1]), dtype=x.dtype, device=x.device)
    a.out = out.data_ptr()
    if _lib.lib.cgtp_uvu_validate(C.byref(a), 0) != 0:
        return None
    _lib.check(_lib.lib.cgtp_uvu_fwd(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvu_fwd")
    return out


def uvu_backward(cfg: int, dims, x: Tensor, y: Tensor, w: Tensor, g: Tensor, need, ptr_=None, perm=None,
                 gather=None):
    """Specialised backward -> (grad_x, grad_y, grad_w) (None where not needed), or None if not launchable."""
    n_rows = y.shape[0]
    a = _uvu_args(cfg, x, y, w, n_rows, ptr_, perm, gather)
    a.grad_out = g.data_ptr()
    gx = torch.empty_like(x) if need[0] else None
    gy = torch.empty_like(y) if need[1] else None
    gw = torch.empty_like(w) if need[2] else None
    a.grad_x, a.grad_y, a.grad_w = _lib.ptr(gx), _lib.ptr(gy), _lib.ptr(gw)
    ws = None
    if a.w_shared and need[2]:
        nbytes = int(_lib.lib.cgtp_uvu_bwd_workspace_bytes(C.byref(a)))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        a.workspace = ws.data_ptr()
    if _lib.lib.cgtp_uvu_validate(C.byref(a), 1) != 0:
        return None
    _lib.check(_lib.lib.cgtp_uvu_bwd(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvu_bwd")
    return gx, gy, gw


def uvu_dims(cfg: int):
    d = (C.c_int32 * 5)()
    _lib.lib.cgtp_uvu_describe(cfg, d)
    return tuple(d)


# ---- packed tables for the table-driven kernel --------------------------------------------------------------
def tp_tri_table(tp_info, role: str, dtype: torch.dtype, device) -> Tuple[dict, int]:
    """Packed table of one direction of the fused tensor product.

    role 'out': out[M]  <- a=in1[M1], b=in2[M2], w=W[p]
    role 'in1': g1[M1] <- a=g[M],   b=in2[M2], w=W[p]
    role 'in2': g2[M2] <- a=g[M],   b=in1[M1], w=W[p]
    role 'w'  : gW[p]  <- a=g[M],   b=in1[M1], w=in2[M2]
    """
    def build():
        c = coo_of(tp_info)
        if role == "out":
            o, ia, ib, iw, n = c.M, c.M1, c.M2, c.p, c.DO
        elif role == "in1":
            o, ia, ib, iw, n = c.M1, c.M, c.M2, c.p, c.D1
        elif role == "in2":
            o, ia, ib, iw, n = c.M2, c.M, c.M1, c.p, c.D2
        elif role == "w":
            o, ia, ib, iw, n = c.p, c.M, c.M1, c.M2, c.P
        else:
            raise ValueError(role)
        return pack_tri_table(o, ia, ib, iw, c.coef, n, dtype, device), n
    return cached(tp_info.info_Mij_fwd.scale, ("tri", role, dtype, str(device)), build)


def product_tri_table(scale, index1, index2, seg, n_entries: int, dtype, device) -> Tuple[dict, int]:
    """Packed table for one ``SparseProductInfo``-style operator call (already sorted by output)."""
    anchor = next(t for t in (seg, index1, index2, scale) if t is not None)

    def build():
        ident = np.arange(n_entries, dtype=np.int64)
        i1 = ident if index1 is None else index1.detach().cpu().numpy()
        i2 = ident if index2 is None else index2.detach().cpu().numpy()
        if seg is None:
            out_idx, n_out = ident, n_entries
        else:
            s = seg.detach().cpu().numpy().astype(np.int64)
            n_out = s.shape[0] - 1
            out_idx = np.repeat(np.arange(n_out, dtype=np.int64), np.diff(s))
        coef = None if scale is None else scale.detach().cpu().numpy().astype(np.float64)
        return pack_tri_table(out_idx, i1, i2, None, coef, n_out, dtype, device), n_out
    key = ("prod", id(scale), id(index1), id(index2), id(seg), n_entries, dtype, str(device))
    return cached(anchor, key, build)
