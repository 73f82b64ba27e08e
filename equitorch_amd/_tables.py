"""Kernel-side views of a ``TensorProductInfo``: the flat COO list and its packed / fingerprinted forms.

The two-stage tables of the reference (``info_Mij_fwd``: nnz -> stage-1 segment ``q``; ``info_M_fwd``:
``q`` -> weight path ``p`` and output row ``M``) determine, per non-zero ``t``, the tuple
``(coef, M, M1, M2, p)`` of the fused contraction ``out[M] += coef * x[M1] * y[M2] * W[p]``.
"""
from __future__ import annotations

from typing import Dict, NamedTuple

import numpy as np
import torch


class TpCoo(NamedTuple):
    coef: np.ndarray  # (T,) float64 copy of the table's scale values
    M: np.ndarray     # (T,) int32 output row
    M1: np.ndarray    # (T,) int32 row of input1
    M2: np.ndarray    # (T,) int32 row of input2
    p: np.ndarray     # (T,) int32 weight path
    q: np.ndarray     # (T,) int32 stage-1 segment (k, M, i, j)
    D1: int
    D2: int
    DO: int
    P: int


def _expand_seg(seg, n_rows_default: int) -> np.ndarray:
    """CSR pointer (or None = one entry per row) -> row id per entry."""
    if seg is None:
        return np.arange(n_rows_default, dtype=np.int64)
    seg = seg.detach().cpu().numpy().astype(np.int64)
    return np.repeat(np.arange(seg.shape[0] - 1, dtype=np.int64), np.diff(seg))


def tp_coo(tp_info) -> TpCoo:
    """Flatten the forward tables of one ``TensorProductInfo`` into per-non-zero arrays (table order)."""
    s1, s2 = tp_info.info_Mij_fwd, tp_info.info_M_fwd
    coef = s1.scale.detach().cpu().double().numpy()
    T = coef.shape[0]
    ident = np.arange(T, dtype=np.int64)
    M1 = ident if s1.index1 is None else s1.index1.cpu().numpy()
    M2 = ident if s1.index2 is None else s1.index2.cpu().numpy()
    q = _expand_seg(s1.seg_out, T)
    n_q = int(s1.out_size)
    p_of_q = np.arange(n_q, dtype=np.int64) if s2.index2 is None else s2.index2.cpu().numpy()
    i1_of_q = np.arange(n_q, dtype=np.int64) if s2.index1 is None else s2.index1.cpu().numpy()
    M_of_q = _expand_seg(s2.seg_out, n_q)
    # stage 2 walks q' = 0..n_q-1 reading inter[index1[q']]; map back to stage-1 segment ids
    p_by_inter = np.empty(n_q, dtype=np.int64)
    M_by_inter = np.empty(n_q, dtype=np.int64)
    p_by_inter[i1_of_q] = p_of_q
    M_by_inter[i1_of_q] = M_of_q
    i32 = lambda a: np.ascontiguousarray(a, dtype=np.int32)
    p = p_by_inter[q]
    return TpCoo(coef, i32(M_by_inter[q]), i32(M1), i32(M2), i32(p), i32(q),
                 int(tp_info.info_Mij_bwd1.out_size), int(tp_info.info_Mij_bwd2.out_size),
                 int(tp_info.out_size), int(p.max()) + 1)


def round_coefficients(coef: np.ndarray, precision: str) -> np.ndarray:
    """fp32 array of the coefficients as they read after ``tensor.to(precision)`` of the fp32 table:
    ``'f32'`` (unchanged), ``'bf16'`` or ``'f16'`` (round to nearest even from fp32)."""
    c32 = np.ascontiguousarray(coef, dtype=np.float32)
    if precision == "f32":
        return c32
    if precision == "f16":
        return c32.astype(np.float16).astype(np.float32)
    if precision == "bf16":
        u = c32.view(np.uint32).astype(np.uint64)
        u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
        return u.astype(np.uint32).view(np.float32)
    raise ValueError(precision)


def fingerprint(coo: TpCoo, precision: str = "f32") -> int:
    """64-bit FNV-1a over dims, indices and the fp32 bits of the coefficients rounded to ``precision``; identifies
    a compiled-in table (``'bf16'`` / ``'f16'``: the table of a module converted to that type)."""
    blob = b"".join([
        np.array([coo.D1, coo.D2, coo.DO, coo.P, coo.coef.shape[0]], dtype=np.int32).tobytes(),
        coo.M.tobytes(), coo.M1.tobytes(), coo.M2.tobytes(), coo.p.tobytes(),
        round_coefficients(coo.coef, precision).tobytes(),
    ])
    h = 0xCBF29CE484222325
    for b in blob:
        h = ((h ^ b) * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def pack_tri_table(out_idx, ia, ib, iw, coef, n_out: int, dtype: torch.dtype, device) -> Dict[str, torch.Tensor]:
    """Sort a COO list by output index and pack it for ``cgtp_tri_contract``.

    Returns device tensors ``coef`` (dtype), ``idx`` (int32 holding ia | ib<<10 | iw<<20) and ``seg``
    (int32 CSR pointer of length n_out+1).  ``ia`` / ``ib`` / ``iw`` may be None (operand absent -> 0).
    """
    out_idx = np.asarray(out_idx, dtype=np.int64)
    T = out_idx.shape[0]
    z = np.zeros(T, dtype=np.int64)
    ia = z if ia is None else np.asarray(ia, dtype=np.int64)
    ib = z if ib is None else np.asarray(ib, dtype=np.int64)
    iw = z if iw is None else np.asarray(iw, dtype=np.int64)
    if T and (ia.max() >= 1024 or ib.max() >= 1024 or iw.max() >= 4096):
        raise ValueError("sparse index too large for the packed table (limits 1024 / 1024 / 4096)")
    order = np.lexsort([ib, ia, iw, out_idx])
    packed = (ia | (ib << 10) | (iw << 20))[order].astype(np.uint32).view(np.int32)
    seg = np.zeros(n_out + 1, dtype=np.int64)
    np.add.at(seg, out_idx + 1, 1)
    seg = np.cumsum(seg).astype(np.int32)
    res = {
        "idx": torch.from_numpy(packed.copy()).to(device),
        "seg": torch.from_numpy(seg).to(device),
        "coef": None,
    }
    if coef is not None:
        res["coef"] = torch.from_numpy(np.asarray(coef, dtype=np.float64)[order].copy()).to(dtype).to(device)
    return res
