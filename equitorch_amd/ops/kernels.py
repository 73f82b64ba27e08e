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
from .._lib import OPERAND_NONE, OPERAND_VEC, Operand, TriArgs, UvuArgs
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
    ref = weakref.ref(anchor, lambda _r, k=k: _CACHE.pop(k, None) if _CACHE is not None else None)
    _CACHE[k] = (ref, val)
    return val


def coo_of(tp_info) -> TpCoo:
    return cached(tp_info.info_Mij_fwd.scale, "coo", lambda: tp_coo(tp_info))


class Cfg(int):
    """Index of a compiled-in table (an ``int``, -1: none), carrying how the caller's table maps onto the compiled one.

    ``path_scale`` (float64 array over the compiled paths, or None = all ones): the caller's coefficients are the
    compiled ones times one factor per weight path — what ``path_norm`` / ``channel_norm`` / ``channel_scale`` change
    (``equitorch/utils/_structs.py:177-206``).  ``w_rows`` (int array over the compiled paths, or None = identity): the
    caller's weight row of every compiled path, -1 for a path the caller's table does not have (an explicit ``path=``
    subset); such weights are expanded with zero rows before the launch (:func:`expand_paths`).  ``exact``: every
    coefficient of the caller's table is the compiled one times its path's factor to the last bit.  The tables hold
    fp32 products of coupling and normalisation, so with another normalisation the ratios of a path's entries scatter
    by an fp32 rounding (1e-7): nothing in fp32 arithmetic, but seven digits short of what float64 operands are held
    to — those take the compiled kernels for exact matches only (:func:`uvu_launchable`)."""
    path_scale: Optional[np.ndarray]
    w_rows: Optional[np.ndarray]

    def __new__(cls, value: int, path_scale=None, w_rows=None, exact=True):
        obj = super().__new__(cls, value)
        obj.path_scale, obj.w_rows, obj.exact = path_scale, w_rows, exact
        obj._dev = {}
        return obj

    def scale_tensor(self, dtype: torch.dtype, device) -> Optional[Tensor]:
        """``path_scale`` as a device tensor of ``dtype`` (cached), or None."""
        if self.path_scale is None:
            return None
        key = (dtype, str(device))
        if key not in self._dev:
            self._dev[key] = torch.from_numpy(self.path_scale).to(device=device, dtype=dtype)
        return self._dev[key]

    def rows_tensor(self, device) -> Optional[Tensor]:
        if self.w_rows is None:
            return None
        key = ("rows", str(device))
        if key not in self._dev:
            self._dev[key] = torch.from_numpy(self.w_rows.astype(np.int64)).to(device)
        return self._dev[key]


_COMPILED = {}   # family -> list of (dims, {(M, M1, M2): (p, coef)}) of every compiled configuration


def _compiled_tables(family: str):
    """The tables compiled into the library, read back through ``cgtp_uvu_table`` / ``cgtp_uv_table`` (once)."""
    if family in _COMPILED:
        return _COMPILED[family]
    L = _lib.lib
    out = []
    n = L.cgtp_uvu_num_configs() if family == "uvu" else L.cgtp_uv_num_configs()
    for cfg in range(n):
        dims = (C.c_int32 * 5)()
        if family == "uvu":
            L.cgtp_uvu_describe(cfg, dims)
        else:
            L.cgtp_uv_table(cfg, dims, None, None)
        nnz = dims[4]
        coef, idx = (C.c_float * nnz)(), (C.c_int32 * (4 * nnz))()
        got = L.cgtp_uvu_table(cfg, coef, idx) if family == "uvu" else L.cgtp_uv_table(cfg, None, coef, idx)
        assert got == nnz
        ix = np.frombuffer(idx, dtype=np.int32).reshape(nnz, 4)
        cf = np.frombuffer(coef, dtype=np.float32).astype(np.float64)
        out.append((tuple(dims), {(int(m), int(a), int(b)): (int(p), float(c)) for (m, a, b, p), c in zip(ix, cf)}))
    _COMPILED[family] = out
    return out


_RATIO_TOL = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}   # coefficient tensors converted with the module


def _match_config(tp_info, family: str) -> Cfg:
    """The compiled configuration whose table has the same entries as ``tp_info`` up to one factor per weight path
    (and, for an explicit ``path=`` subset, a subset of its paths), or ``Cfg(-1)``.  Exact equality of the fp32
    coefficients gives ``path_scale = None``."""
    coo = coo_of(tp_info)
    tol = _RATIO_TOL.get(tp_info.info_Mij_fwd.scale.dtype, 1e-6)
    nnz = coo.coef.shape[0]
    for cfg, (dims, table) in enumerate(_compiled_tables(family)):
        if dims[:3] != (coo.D1, coo.D2, coo.DO) or nnz > dims[4] or coo.P > dims[3]:
            continue
        comp_of, row_of, ratios, ok = {}, {}, {}, True      # caller path -> compiled path and back; ratios per path
        for t in range(nnz):
            hit = table.get((int(coo.M[t]), int(coo.M1[t]), int(coo.M2[t])))
            if hit is None:
                ok = False
                break
            pc, cc = hit
            pm = int(coo.p[t])
            if comp_of.setdefault(pm, pc) != pc or row_of.setdefault(pc, pm) != pm:
                ok = False
                break
            ratios.setdefault(pc, []).append(float(coo.coef[t]) / cc)
        if not ok:
            continue
        # every entry of a matched compiled path must be present (a path is either taken whole or not at all)
        count = {}
        for (_, _, _), (pc, _) in table.items():
            count[pc] = count.get(pc, 0) + 1
        if any(len(r) != count[pc] for pc, r in ratios.items()):
            continue
        scale = np.zeros(dims[3], dtype=np.float64)
        exact = True
        for pc, r in ratios.items():
            r = np.asarray(r)
            mid = float(np.median(r))
            if mid == 0.0 or np.any(np.abs(r / mid - 1.0) > tol):
                ok = False
                break
            scale[pc] = mid
            exact = exact and bool(np.all(r == mid))
        if not ok:
            continue
        full = len(ratios) == dims[3]
        identity = full and all(row_of[pc] == pc for pc in range(dims[3]))
        ones = full and np.all(np.abs(scale - 1.0) <= tol)
        rows = None if identity else np.array([row_of.get(pc, -1) for pc in range(dims[3])], dtype=np.int64)
        return Cfg(cfg, None if ones else scale, rows, exact)
    return Cfg(-1)


def uvu_config_of(tp_info) -> Cfg:
    """The compiled-in channel-wise table this ``tp_info`` runs on (see :class:`Cfg`), or ``Cfg(-1)``."""
    return cached(tp_info.info_Mij_fwd.scale, "cfg", lambda: _match_config(tp_info, "uvu"))


def uv_config_of(tp_info) -> Cfg:
    """The same among the tables of the fully connected product on the matrix cores."""
    return cached(tp_info.info_Mij_fwd.scale, "uv_cfg", lambda: _match_config(tp_info, "uv"))


def expand_paths(w: Tensor, cfg, path_dim: int) -> Tensor:
    """Weights of a table that has only some of the compiled paths (``cfg.w_rows``), laid out over all compiled
    paths with zeros for the missing ones; differentiable.  Identity when the table has all paths in order."""
    rows = getattr(cfg, "w_rows", None)
    if rows is None:
        return w
    idx = cfg.rows_tensor(w.device)
    present = idx >= 0
    full = w.index_select(path_dim, idx.clamp(min=0))
    shape = [1] * w.ndim
    shape[path_dim] = -1
    return full * present.to(w.dtype).view(shape)


def contract_paths(gw: Optional[Tensor], cfg, path_dim: int) -> Optional[Tensor]:
    """Inverse of :func:`expand_paths` for a gradient: the rows of the caller's own paths, in the caller's order."""
    rows = getattr(cfg, "w_rows", None)
    if rows is None or gw is None:
        return gw
    key = ("inverse", str(gw.device))
    if key not in cfg._dev:
        inv = np.full(int(rows.max()) + 1, -1, dtype=np.int64)
        for pc, pm in enumerate(rows):
            if pm >= 0:
                inv[pm] = pc
        cfg._dev[key] = torch.from_numpy(inv).to(gw.device)
    return gw.index_select(path_dim, cfg._dev[key]).contiguous()


_TIER_LOG = bool(__import__("os").environ.get("CGTP_LOG_TIER"))
_TIER_SEEN = set()


def log_tier(op: str, tier: str, detail: str = ""):
    """With ``CGTP_LOG_TIER=1`` in the environment: one line on stderr the first time an operator takes a kernel tier
    (compiled table / block-wise / table-driven / library GEMM), so that a slow path is visible."""
    if _TIER_LOG and (op, tier, detail) not in _TIER_SEEN:
        _TIER_SEEN.add((op, tier, detail))
        import sys
        print(f"[cgtp] {op}: {tier}{' (' + detail + ')' if detail else ''}", file=sys.stderr, flush=True)


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
    op.size = t.shape[-2] if kind == OPERAND_VEC else t.shape[-1]
    return op


def tri_contract(table: dict, n_out: int, a: Tuple[Optional[Tensor], int], b: Tuple[Optional[Tensor], int],
                 w: Tuple[Optional[Tensor], int], n_rows: int, channels: int, dtype: torch.dtype, device,
                 reduce_c: bool = False, reduce_rows: bool = False,
                 rows_a: Optional[Tensor] = None, rows_b: Optional[Tensor] = None,
                 rows_w: Optional[Tensor] = None, out: Optional[Tensor] = None,
                 static_scratch: bool = False) -> Tensor:
    """``out[r,o,c] = sum_t coef_t A[r,ia_t,c] B[r,ib_t,(c)] W[r,iw_t,c]`` with the packed ``table``.
    ``static_scratch``: launch through ``cgtp_tri_contract_static`` — no workspace is allocated here, the partial
    rows of a sum over rows live in the library's fixed per-device array (and with ``out`` given, this call allocates
    nothing at all)."""
    shape = ((n_out,) if reduce_c else (n_out, channels))
    if not reduce_rows:
        shape = (n_rows,) + shape
    if out is None:
        out = torch.empty(shape, dtype=dtype, device=device)
    elif tuple(out.shape) != shape or out.dtype != dtype or not out.is_contiguous():
        raise _lib.CgtpError(f"out must be a contiguous {dtype} tensor of shape {shape}")
    if n_rows == 0 or out.numel() == 0:      # empty batch: nothing to launch; a sum over no rows is zero
        return out.zero_()
    if table["idx"].shape[0] == 0:           # a table without entries: a sum over no terms
        return out.zero_()
    args = TriArgs()
    args.a, args.b, args.w = _operand(*a, rows_a), _operand(*b, rows_b), _operand(*w, rows_w)
    args.coef, args.idx, args.seg = _lib.ptr(table["coef"]), table["idx"].data_ptr(), table["seg"].data_ptr()
    args.n_out, args.nnz = n_out, table["idx"].shape[0]
    args.out, args.n_rows, args.C = out.data_ptr(), n_rows, channels
    args.dtype, args.reduce_c, args.reduce_rows = _lib.dtype_code(dtype), int(reduce_c), int(reduce_rows)
    if static_scratch:
        _lib.check(_lib.lib.cgtp_tri_contract_static(C.byref(args), _lib.stream_ptr(device)),
                   "cgtp_tri_contract_static")
        return out
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
    if inp.dtype not in (torch.float32, torch.float64):      # reduced precision: summed in fp32, rounded once
        return segment_sum(inp.float(), scale, index, seg, out_size).to(inp.dtype)
    inp = inp.contiguous()
    n, in_size, ch = inp.shape
    out = torch.empty((n, out_size, ch), dtype=inp.dtype, device=inp.device)
    if inp.numel() == 0 or out.numel() == 0:      # nothing to sum: every output row is an empty sum
        return out.zero_()
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


# ---- fused layer RMS normalisation ------------------------------------------------------------------------------
def _seg_array(irrep_seg: Tensor):
    """Host int32 array of the irrep boundaries (cached on the table tensor)."""
    def build():
        vals = [int(v) for v in irrep_seg.detach().cpu().tolist()]
        return (C.c_int32 * len(vals))(*vals), len(vals) - 1
    return cached(irrep_seg, "layer_rms_seg", build)


def _rdims_array(rdims: Tensor):
    """Host float array of the table's ``1 / dim`` factors (fp32, as the reference stores them)."""
    def build():
        vals = rdims.detach().to(torch.float32).cpu().tolist()
        return (C.c_float * len(vals))(*vals)
    return cached(rdims, "layer_rms_rdims", build)


def layer_rms_supported(irrep_seg: Tensor, channels: int, dtype: torch.dtype) -> bool:
    if dtype not in (torch.float32, torch.float64):
        return False
    arr, k = _seg_array(irrep_seg)
    return bool(_lib.lib.cgtp_layer_rms_supported(arr, k, channels, _lib.dtype_code(dtype)))


def layer_rms_forward(x: Tensor, weight: Optional[Tensor], irrep_seg: Tensor, rdims: Tensor, scaled: bool, eps: float,
                      want_rsigma: bool):
    """``(out, rsigma | None)`` of ``cgtp_layer_rms_forward``; ``x`` is ``(N, D, C)`` contiguous."""
    arr, k = _seg_array(irrep_seg)
    n, d, ch = x.shape
    out = torch.empty_like(x)
    rsigma = torch.empty((n, k), dtype=x.dtype, device=x.device) if want_rsigma else None
    _lib.check(_lib.lib.cgtp_layer_rms_forward(x.data_ptr(), _lib.ptr(weight), out.data_ptr(), _lib.ptr(rsigma), arr,
                                               _rdims_array(rdims), k, n, d, ch, int(scaled), float(eps),
                                               _lib.dtype_code(x.dtype),
                                               _lib.stream_ptr(x.device)), "cgtp_layer_rms_forward")
    return out, rsigma


def layer_rms_backward(x: Tensor, weight: Optional[Tensor], rsigma: Tensor, grad_out: Tensor, irrep_seg: Tensor,
                       rdims: Tensor, scaled: bool, need_x: bool, need_w: bool):
    """``(grad_x | None, grad_weight | None)`` of ``cgtp_layer_rms_backward``."""
    arr, k = _seg_array(irrep_seg)
    n, d, ch = x.shape
    gx = torch.empty_like(x) if need_x else None
    gw = ws = None
    if need_w:
        gw = torch.empty((k, ch), dtype=x.dtype, device=x.device)
        nbytes = int(_lib.lib.cgtp_layer_rms_workspace_bytes(n, k, ch, _lib.dtype_code(x.dtype)))
        ws = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.lib.cgtp_layer_rms_backward(x.data_ptr(), _lib.ptr(weight), rsigma.data_ptr(), grad_out.data_ptr(),
                                                _lib.ptr(gx), _lib.ptr(gw), _lib.ptr(ws), arr, _rdims_array(rdims), k,
                                                n, d, ch, int(scaled), _lib.dtype_code(x.dtype),
                                                _lib.stream_ptr(x.device)),
               "cgtp_layer_rms_backward")
    return gx, gw


# ---- fused Wigner rotation ----------------------------------------------------------------------------------
class RotationLayout:
    """Irrep blocks and dense J blocks recovered from the tables of a ``WignerRotationInfo``: the z-rotation table
    pairs component ``m`` with ``-m`` (so the partner of a block's first row is its last row), and the entries of the
    sparse J table fill one dense block per irrep.  ``ok`` is False when the tables do not have that structure."""

    def __init__(self, info):
        z, j = info.rotate_z_info_fwd, info.j_matrix_info
        self.ok = False
        # tables with identity columns or one term per output arrive with those fields collapsed to None
        n_z = next((t.shape[0] for t in (z.index1, z.index2, z.scale) if t is not None), None)
        if n_z is None or z.out_size is None:
            return
        dim = int(z.out_size)
        zi = list(range(n_z)) if z.index1 is None else z.index1.tolist()
        zseg = list(range(dim + 1)) if z.seg_out is None else z.seg_out.tolist()
        if len(zseg) - 1 != dim:
            return
        first, degree, at = [], [], 0
        while at < dim:
            partner = max(zi[zseg[at]:zseg[at + 1]], default=at)     # m = -l pairs with m = +l, the block's last row
            size = partner - at + 1
            if size < 1 or size % 2 == 0 or at + size > dim:
                return
            first.append(at)
            degree.append((size - 1) // 2)
            at += size
        block_of = [k for k, l in enumerate(degree) for _ in range(2 * l + 1)]
        blocks = [torch.zeros(2 * l + 1, 2 * l + 1, dtype=torch.float64) for l in degree]
        n_j = next((t.shape[0] for t in (j.index, j.scale) if t is not None), dim)
        jseg = list(range(dim + 1)) if j.seg_out is None else j.seg_out.tolist()
        jidx = list(range(n_j)) if j.index is None else j.index.tolist()
        jval = [1.0] * n_j if j.scale is None else j.scale.double().tolist()
        if len(jseg) - 1 != dim or jseg[-1] != n_j:
            return
        for row in range(dim):
            k = block_of[row]
            for t in range(jseg[row], jseg[row + 1]):
                col = jidx[t]
                if block_of[col] != k:
                    return
                blocks[k][row - first[k], col - first[k]] = jval[t]
        self.first = (C.c_int32 * len(first))(*first)
        self.degree = (C.c_int32 * len(degree))(*degree)
        self.n_irreps, self.dim, self.max_degree = len(first), dim, max(degree, default=0)
        self._flat = torch.cat([b.reshape(-1) for b in blocks]) if blocks else torch.zeros(0, dtype=torch.float64)
        self._on = {}
        self.ok = True

    def j_blocks(self, dtype, device) -> Tensor:
        key = (dtype, str(device))
        if key not in self._on:
            self._on[key] = self._flat.to(device=device, dtype=dtype)
        return self._on[key]


def rotation_layout(info) -> RotationLayout:
    return cached(info.j_matrix_info.scale, "rotation_layout", lambda: RotationLayout(info))


def wigner_rotate_supported(layout: RotationLayout, channels: int, dtype: torch.dtype) -> bool:
    return (layout.ok and dtype in (torch.float32, torch.float64) and bool(_lib.lib.cgtp_wigner_rotate_supported(
        layout.first, layout.degree, layout.n_irreps, channels, _lib.dtype_code(dtype))))


def wigner_rotate(x: Tensor, sincos_alpha: Optional[Tensor], sincos_beta: Optional[Tensor],
                  sincos_gamma: Optional[Tensor], layout: RotationLayout, transposed: bool) -> Tensor:
    """``cgtp_wigner_rotate`` on ``x (N, D, C)`` contiguous; the sincos tensors are ``(N, cs_dim)`` contiguous."""
    n, _, ch = x.shape
    out = torch.empty_like(x)
    cs_dim = next(t.shape[-1] for t in (sincos_alpha, sincos_beta, sincos_gamma) if t is not None)
    _lib.check(_lib.lib.cgtp_wigner_rotate(x.data_ptr(), out.data_ptr(), _lib.ptr(sincos_alpha), _lib.ptr(sincos_beta),
                                           _lib.ptr(sincos_gamma), layout.j_blocks(x.dtype, x.device).data_ptr(),
                                           layout.first, layout.degree, layout.n_irreps, n, ch, cs_dim,
                                           int(transposed), _lib.dtype_code(x.dtype), _lib.stream_ptr(x.device)),
               "cgtp_wigner_rotate")
    return out


def wigner_rotate_backward(x: Tensor, grad_out: Tensor, sincos, layout: RotationLayout, need_x: bool, need_cs):
    """``(grad_x | None, [grad of each sincos tensor | None])`` of ``cgtp_wigner_rotate_backward``; ``sincos`` is the
    triple (alpha, beta, gamma) with ``None`` for a skipped factor, ``need_cs`` the matching triple of flags."""
    n, _, ch = x.shape
    cs_dim = next(t.shape[-1] for t in sincos if t is not None)
    gx = torch.empty_like(x) if need_x else None
    gcs = [torch.empty_like(t) if (t is not None and want) else None for t, want in zip(sincos, need_cs)]
    _lib.check(_lib.lib.cgtp_wigner_rotate_backward(x.data_ptr(), grad_out.data_ptr(), *[_lib.ptr(t) for t in sincos],
                                                    layout.j_blocks(x.dtype, x.device).data_ptr(), layout.first,
                                                    layout.degree, layout.n_irreps, n, ch, cs_dim, _lib.ptr(gx),
                                                    *[_lib.ptr(t) for t in gcs], _lib.dtype_code(x.dtype),
                                                    _lib.stream_ptr(x.device)), "cgtp_wigner_rotate_backward")
    return gx, gcs


# ---- specialised uvu ----------------------------------------------------------------------------------------
# How the sorted edge list is cut into one range per wavefront: "aligned" (at segment boundaries, no partial rows),
# "balanced" (after equal numbers of steps), "positions" (after equal numbers of positions), or "auto": measured on the
# lmax = 2, C = 64 edge workload, the forward is fastest on aligned ranges (0.061 ms against 0.071 / 0.066) and the
# backward, whose steps are three times as long, on balanced ones (0.115 ms against 0.122 / 0.118).
_RANGE_MODE = __import__("os").environ.get("CGTP_RANGE_MODE", "auto")


class SegIndex:
    """Per-sorted-position index arrays of the segment mode (all int64, same device), and the tables that cut the
    sorted list into one range per wavefront."""

    def __init__(self, ptr: Tensor, perm: Optional[Tensor], seg_ids: Tensor, gather: Tensor,
                 positions_per_wave: int = int(__import__("os").environ.get("CGTP_POSITIONS_PER_WAVE", "32"))):
        self.ptr, self.perm, self.seg_ids, self.gather = ptr, perm, seg_ids, gather
        self.positions_per_wave = positions_per_wave
        self.wave_seg = self.aligned_ranges(ptr, positions_per_wave)
        # the step-balanced cuts for every slot count a launch can have (64 / lanes per edge), built here, where a host
        # sync is expected, and not on the first backward (inside autograd, possibly under graph capture)
        self._wave_pos = {}
        self._build_balanced(self.SLOT_COUNTS)

    SLOT_COUNTS = (1, 2, 4, 8, 16, 32, 64)

    def _build_balanced(self, slot_counts) -> None:
        import numpy as np
        ptr = self.ptr.detach().cpu().numpy()
        n_pos = int(ptr[-1]) if ptr.shape[0] else 0
        for slots in slot_counts:
            if n_pos == 0:
                self._wave_pos[slots] = None
                continue
            steps = (np.diff(ptr) + slots - 1) // slots
            last = np.cumsum(steps)                            # steps up to and including each segment
            first = last - steps
            # as many ranges as equal cuts by position would give (a launch sized for that many wavefronts stays
            # resident in one round)
            n_ranges = max(1, n_pos // self.positions_per_wave)
            per_wave = max(1, -(-int(last[-1]) // n_ranges))
            targets = np.arange(0, int(last[-1]), per_wave, dtype=np.int64)
            seg = np.searchsorted(last, targets, side="right")
            pos = ptr[:-1][seg] + (targets - first[seg]) * slots
            self._wave_pos[slots] = torch.from_numpy(np.concatenate([pos, [n_pos]]).astype(np.int64)).to(self.ptr.device)

    @staticmethod
    def aligned_ranges(ptr: Tensor, positions_per_wave: int) -> Optional[Tensor]:
        """Cut the sorted list at segment boundaries into ranges of about ``positions_per_wave`` positions:
        int32 ``[n_ranges + 1]`` segment indices (first 0, last n_seg).  Range k starts at the first segment
        whose first position is >= k * positions_per_wave.  Returns None (ranges by position are used instead)
        when a segment is so large that aligned ranges would be badly unbalanced."""
        n_seg, n_pos = ptr.shape[0] - 1, int(ptr[-1])
        if n_seg == 0:
            return None
        if n_pos and int((ptr[1:] - ptr[:-1]).max()) > 8 * positions_per_wave:
            return None
        targets = torch.arange(0, max(n_pos, 1), positions_per_wave, device=ptr.device, dtype=ptr.dtype)
        cuts = torch.searchsorted(ptr[:-1].contiguous(), targets)
        cuts = torch.unique_consecutive(torch.cat([cuts.new_zeros(1), cuts, cuts.new_full((1,), n_seg)]))
        return cuts.to(torch.int32).contiguous()

    def balanced_positions(self, slots: int) -> Optional[Tensor]:
        """Cut the sorted list after equal numbers of steps: a wavefront takes up to ``slots`` positions of one segment
        per step, so a segment of n positions costs ceil(n / slots) steps wherever it lies, and a range that holds
        whole steps only costs exactly its share.  int64 ``[n_ranges + 1]`` positions (first 0, last n_pos), cuts on
        step boundaries; as many ranges as ``positions_per_wave`` positions each would give.  The time of a wavefront follows its number of
        steps, and ranges cut at segment boundaries differ in it by a factor of up to five on a graph of average
        degree 16."""
        if slots <= 0:
            return None
        if slots not in self._wave_pos:      # a slot count outside SLOT_COUNTS: built now (reads ptr back: a host sync)
            self._build_balanced((slots,))
        return self._wave_pos[slots]


def seg_ranges(cfg: int, seg: SegIndex, dtype_code: int, channels: int, backward: bool):
    """``(wave_seg, wave_pos)``, at most one of them a tensor: how a segment-mode launch of ``cfg`` cuts the sorted list
    into one range per wavefront (``_RANGE_MODE``); both None = ranges of equal numbers of positions, which is also all
    the block-wise kernels of the large tables take."""
    if _lib.lib.cgtp_uvu_blockwise_only(int(cfg)):
        return None, None
    wave_pos = None
    if _RANGE_MODE == "balanced" or (_RANGE_MODE == "auto" and (backward or seg.wave_seg is None)):
        wave_pos = seg.balanced_positions(int(_lib.lib.cgtp_uvu_slots(int(cfg), dtype_code, channels, int(backward))))
    if wave_pos is not None:
        return None, wave_pos
    if seg.wave_seg is not None and _RANGE_MODE != "positions":
        return seg.wave_seg, None
    return None, None


class IdentitySegments:
    """A plain batch seen as an edge list in which row r is the only edge of node r: what the table-driven segment
    kernels need (``ptr``, ``perm``, ``seg_ids``, ``gather``) to run a product on a batch.  ``fwd_index`` and
    ``bwd_index`` are this object itself, as on an ``EdgePlan``."""

    def __init__(self, n: int, device):
        ids = torch.arange(n + 1, dtype=torch.int64, device=device)
        self.ptr, self.perm, self.seg_ids, self.gather = ids, None, ids[:n], ids[:n]
        self.fwd_index = self.bwd_index = self


_IDENTITY = {}


def identity_segments(n: int, device) -> IdentitySegments:
    key = (n, str(device))
    seg = _IDENTITY.get(key)
    if seg is None:
        if len(_IDENTITY) >= 8:
            _IDENTITY.pop(next(iter(_IDENTITY)))
        seg = _IDENTITY[key] = IdentitySegments(n, device)
    return seg


def _uvu_args(cfg: int, x: Tensor, y: Tensor, w: Tensor, seg: Optional[SegIndex], gather: Optional[Tensor],
              pos_per_wave: int = 0, y_vec: int = 0, backward: bool = False) -> UvuArgs:
    a = UvuArgs()
    a.y_vec = y_vec
    a.y_channels = int(y.ndim == 3)
    a.cfg, a.dtype, a.C = cfg, _lib.dtype_code(x.dtype), x.shape[-1]
    a.w_shared = int(w.ndim == 2)
    a.n_rows, a.n_x_rows = y.shape[0], x.shape[0]
    if seg is not None:
        a.n_seg = seg.ptr.shape[0] - 1
        a.ptr, a.perm, a.seg_ids, a.gather = seg.ptr.data_ptr(), _lib.ptr(seg.perm), seg.seg_ids.data_ptr(), \
            seg.gather.data_ptr()
        a.pos_per_wave = pos_per_wave
        if pos_per_wave == 0:
            wave_seg, wave_pos = seg_ranges(cfg, seg, a.dtype, a.C, backward)
            if wave_pos is not None:
                a.wave_pos, a.n_waves = wave_pos.data_ptr(), wave_pos.shape[0] - 1
            elif wave_seg is not None:
                a.wave_seg, a.n_waves = wave_seg.data_ptr(), wave_seg.shape[0] - 1
    else:
        a.gather = _lib.ptr(gather)
    a.x, a.y, a.w = x.data_ptr(), y.data_ptr(), w.data_ptr()
    scale = cfg.scale_tensor(x.dtype, x.device) if isinstance(cfg, Cfg) else None
    a.path_scale = _lib.ptr(scale)
    a._keep = scale
    return a


_GW_WORKSPACE_BYTES = 512 << 20      # largest per-row weight-gradient workspace of one row-mode backward launch


def _workspace(a: UvuArgs, backward: int, device):
    nbytes = int(_lib.lib.cgtp_uvu_workspace_bytes(C.byref(a), backward))
    if nbytes == 0:
        return None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    a.workspace = ws.data_ptr()
    return ws


_LAUNCHABLE = {}


def uvu_launchable(cfg: int, x: Tensor, y: Tensor, w: Tensor, segments: bool = False, gathered: bool = False,
                   y_vec: int = 0) -> bool:
    """True when both the specialised forward and backward accept these operands (dtype, channel count,
    alignment); outputs are torch allocations and therefore always aligned.  ``gathered``: row mode with the rows
    of ``x`` picked by an index."""
    if x.shape[0] == 0 or y.shape[0] == 0:
        return False
    if x.dtype == torch.float64 and not getattr(cfg, "exact", True):
        return False
    # the answer depends on these only (pointers enter through their 16-byte alignment)
    key = (int(cfg), x.dtype, x.shape[-1], w.ndim, y.ndim, segments, gathered, y_vec,
           x.data_ptr() % 16, y.data_ptr() % 16, w.data_ptr() % 16, x.shape[0] == y.shape[0],
           max(x.shape[0], y.shape[0]) >= 1 << 31)
    hit = _LAUNCHABLE.get(key)
    if hit is not None:
        return hit
    a = UvuArgs()
    a.cfg, a.dtype, a.C = cfg, _lib.dtype_code(x.dtype), x.shape[-1]
    a.w_shared = int(w.ndim == 2)
    a.n_rows = y.shape[0]
    a.y_vec = y_vec
    a.y_channels = int(y.ndim == 3)
    dummy = 256
    a.n_x_rows = x.shape[0]
    if segments:
        a.n_seg, a.ptr, a.gather, a.seg_ids = x.shape[0], dummy, dummy, dummy
    elif gathered:
        a.gather = a.x_gather = dummy
    a.x, a.y, a.w = x.data_ptr() or dummy, y.data_ptr() or dummy, w.data_ptr() or dummy
    a.out = a.grad_out = a.grad_x = a.grad_y = a.grad_w = dummy
    ok = _lib.lib.cgtp_uvu_validate(C.byref(a), 1) == 0
    if len(_LAUNCHABLE) < 4096:
        _LAUNCHABLE[key] = ok
    return ok


Y_HARMONICS, Y_UNIT_VECTOR, Y_RAW_VECTOR = 0, 1, 2


def uvu_forward(cfg: int, dims, x: Tensor, y: Tensor, w: Tensor, seg: Optional[SegIndex] = None,
                gather: Optional[Tensor] = None, pos_per_wave: int = 0, y_vec: int = 0) -> Tensor:
    """Compiled-table forward.  Row mode: ``out[r] = TP(x[gather[r] | r], y[r], w[r])``.  Segment mode:
    ``out[s] = sum_{q in segment s} TP(x[seg.gather[q]], y[e_q], w[e_q])``.  With ``y_vec`` (segment mode), ``y``
    holds ``(E, 3)`` edge vectors and the kernel evaluates their harmonics itself (``Y_UNIT_VECTOR``: after
    normalising them, ``Y_RAW_VECTOR``: as they are)."""
    w = expand_paths(w, cfg, -2)
    a = _uvu_args(cfg, x, y, w, seg, gather, pos_per_wave, y_vec)
    n_out_rows = a.n_seg if seg is not None else y.shape[0]
    out = torch.empty((n_out_rows, dims[2], x.shape[-1]), dtype=x.dtype, device=x.device)
    a.out = out.data_ptr()
    ws = _workspace(a, 0, x.device)
    _lib.check(_lib.lib.cgtp_uvu_fwd(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvu_fwd")
    return out


def uvu_backward(cfg: int, dims, x: Tensor, y: Tensor, w: Tensor, g: Tensor, need, seg: Optional[SegIndex] = None,
                 gather: Optional[Tensor] = None, pos_per_wave: int = 0, x_gather: Optional[Tensor] = None,
                 y_vec: int = 0):
    """Compiled-table backward -> (grad_x, grad_y, grad_w), None where ``need`` is False.  Row mode: ``gather``
    picks the row of ``g`` and ``x_gather`` the row of ``x`` of every batch row; with ``x_gather`` the returned
    grad_x is per batch row, ``(n_rows, D1, C)``."""
    w_given = w
    w = expand_paths(w, cfg, -2)
    a = _uvu_args(cfg, x, y, w, seg, gather, pos_per_wave, y_vec, backward=True)
    a.grad_out = g.data_ptr()
    a.x_gather = _lib.ptr(x_gather)
    n = y.shape[0]
    if seg is None and need[2] and w.ndim == 2 and n > 1:
        # Row mode with a shared weight: some kernels write one weight gradient per row into the workspace and sum
        # afterwards ((rows + chunks) * paths * channels elements).  Past _GW_WORKSPACE_BYTES the rows are taken in
        # equal parts, each with a workspace of its own size, and the parts' gradients are added in order.
        a.grad_w = w.data_ptr()       # any non-null pointer: the query only asks whether the gradient is wanted
        nbytes = int(_lib.lib.cgtp_uvu_workspace_bytes(C.byref(a), 1))
        if nbytes > _GW_WORKSPACE_BYTES:
            parts = min(n, -(-nbytes // _GW_WORKSPACE_BYTES))
            step = -(-n // parts)
            gx = (torch.empty((n,) + x.shape[1:], dtype=x.dtype, device=x.device) if x_gather is not None
                  else torch.empty_like(x)) if need[0] else None
            gy = torch.empty_like(y) if need[1] else None
            gw = None
            rows = lambda t, i0, i1: None if t is None else t[i0:i1]
            for i0 in range(0, n, step):
                i1 = min(i0 + step, n)
                px, py, pw = uvu_backward(cfg, dims, x if x_gather is not None else x[i0:i1], y[i0:i1], w_given,
                                          g if gather is not None else g[i0:i1], need, None, rows(gather, i0, i1),
                                          pos_per_wave, rows(x_gather, i0, i1), y_vec)
                if gx is not None:
                    gx[i0:i1] = px
                if gy is not None:
                    gy[i0:i1] = py
                gw = pw if gw is None else gw + pw
            return gx, gy, gw
    if not need[0]:
        gx = None
    elif x_gather is not None:
        gx = torch.empty((y.shape[0],) + x.shape[1:], dtype=x.dtype, device=x.device)
    else:
        gx = torch.empty_like(x)
    gy = torch.empty_like(y) if need[1] else None
    gw = torch.empty_like(w) if need[2] else None
    a.grad_x, a.grad_y, a.grad_w = _lib.ptr(gx), _lib.ptr(gy), _lib.ptr(gw)
    ws = _workspace(a, 1, x.device)
    _lib.check(_lib.lib.cgtp_uvu_bwd(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvu_bwd")
    return gx, gy, contract_paths(gw, cfg, -2)


def radial_effective_weight(w_last: Tensor, cfg) -> Tensor:
    """``w_last (R, P, C)`` of the caller's table laid out over the compiled paths with the table's per-path factors
    folded in (the kernels that produce the per-edge weights themselves take no separate ``path_scale``)."""
    w = expand_paths(w_last, cfg, -2)
    scale = cfg.scale_tensor(w.dtype, w.device) if isinstance(cfg, Cfg) else None
    if scale is not None:
        w = w * scale.view(1, -1, 1)
    return w.contiguous()


def uvu_radial_supported(cfg: int, x: Tensor, h: Tensor, w_last: Tensor) -> bool:
    """Whether the segment kernels of ``cfg`` can form the per-edge weights from ``h (E, R)`` and ``w_last (R, P, C)``
    themselves: fp32, 64 channels, R a multiple of 4 up to 16, aligned operands."""
    return (cfg >= 0 and bool(_lib.lib.cgtp_uvu_radial_supported(int(cfg))) and x.dtype == h.dtype == w_last.dtype
            and x.dtype == torch.float32 and x.shape[-1] == 64 and h.ndim == 2 and w_last.ndim == 3
            and h.shape[1] == w_last.shape[0] and h.shape[1] % 4 == 0 and 4 <= h.shape[1] <= 16
            and w_last.shape[2] == x.shape[-1]
            and 4 <= uvu_dims(int(cfg))[3] <= 16 and h.shape[0] > 0 and x.shape[0] > 0
            and x.data_ptr() % 16 == 0 and h.data_ptr() % 16 == 0)


def uvu_radial_forward(cfg: int, dims, x: Tensor, y: Tensor, h: Tensor, w_eff: Tensor, seg: SegIndex,
                       y_vec: int = 0) -> Tensor:
    """Segment-mode forward with the per-edge weights ``h @ w_eff`` formed inside the kernel (``w_eff`` from
    :func:`radial_effective_weight`)."""
    a = _uvu_args(Cfg(int(cfg)), x, y, h, seg, None, 0, y_vec)
    a.w, a.w_shared, a.path_scale = None, 0, None
    a.radial_h, a.radial_w, a.radial_r = h.data_ptr(), w_eff.data_ptr(), h.shape[1]
    out = torch.empty((a.n_seg, dims[2], x.shape[-1]), dtype=x.dtype, device=x.device)
    a.out = out.data_ptr()
    ws = _workspace(a, 0, x.device)
    _lib.check(_lib.lib.cgtp_uvu_fwd(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvu_fwd (radial)")
    return out


def uvu_radial_backward(cfg: int, dims, x: Tensor, y: Tensor, h: Tensor, w_eff: Tensor, g: Tensor, need,
                        seg: SegIndex, y_vec: int = 0):
    """-> (grad_x, grad_y, grad_h, grad_w_eff).  The segment kernel regenerates the weights and writes the per-edge
    weight gradient; ``cgtp_uvu_radial_grad`` contracts it with ``w_eff`` and ``h`` in one pass."""
    a = _uvu_args(Cfg(int(cfg)), x, y, h, seg, None, 0, y_vec, backward=True)
    a.w, a.w_shared, a.path_scale = None, 0, None
    a.radial_h, a.radial_w, a.radial_r = h.data_ptr(), w_eff.data_ptr(), h.shape[1]
    a.grad_out = g.data_ptr()
    gx = torch.empty_like(x) if need[0] else None
    gy = torch.empty_like(y) if need[1] else None
    want_w = need[2] or need[3]
    n_paths = dims[3]
    gw = torch.empty((y.shape[0], n_paths, x.shape[-1]), dtype=x.dtype, device=x.device) if want_w else None
    a.grad_x, a.grad_y, a.grad_w = _lib.ptr(gx), _lib.ptr(gy), _lib.ptr(gw)
    ws = _workspace(a, 1, x.device)
    _lib.check(_lib.lib.cgtp_uvu_bwd(C.byref(a), _lib.stream_ptr(x.device)), "cgtp_uvu_bwd (radial)")
    gh = gwl = None
    if want_w:
        r = h.shape[1]
        gh = torch.empty_like(h)
        gwl = torch.empty_like(w_eff)
        nbytes = int(_lib.lib.cgtp_uvu_radial_grad_workspace_bytes(y.shape[0], r, n_paths))
        ws2 = torch.empty(max(nbytes, 16), dtype=torch.uint8, device=x.device)
        _lib.check(_lib.lib.cgtp_uvu_radial_grad(gw.data_ptr(), h.data_ptr(), w_eff.data_ptr(), gh.data_ptr(),
                                                 gwl.data_ptr(), ws2.data_ptr(), y.shape[0], r, n_paths, _lib.F32,
                                                 _lib.stream_ptr(x.device)), "cgtp_uvu_radial_grad")
    return gx, gy, gh, gwl


# ---- channel-wise product over an edge list for a table that is not compiled in ------------------------------------
class UvuTable:
    """A ``TensorProductInfo`` as the data the table-driven segment kernels read: entries sorted by (path, output
    row), one (path, output row) segment per run; device arrays and the ``cgtp_uvu_tab`` descriptor over them."""

    def __init__(self, coo, device):
        order = np.lexsort((coo.M2, coo.M1, coo.M, coo.p))          # by path, then output row, then table order
        p, m = coo.p[order].astype(np.int64), coo.M[order].astype(np.int64)
        nnz = int(order.shape[0])
        padded = (nnz + 63) // 64 * 64 + 128         # whole 64-entry chunks, and two more the walk reads ahead into
        key = p * (int(coo.DO) + 1) + m
        last_of_seg = np.concatenate([key[1:] != key[:-1], [True]])
        last_of_path = np.concatenate([p[1:] != p[:-1], [True]])
        idx = np.zeros(padded, dtype=np.uint32)
        idx[:nnz] = (coo.M1[order].astype(np.uint32) | (coo.M2[order].astype(np.uint32) << 8)
                     | (last_of_seg.astype(np.uint32) << 16) | (last_of_path.astype(np.uint32) << 17)
                     | (m.astype(np.uint32) << 18))
        coef = np.zeros(padded, dtype=np.float32)
        coef[:nnz] = coo.coef[order]
        walk = p[np.concatenate([[True], p[1:] != p[:-1]])]          # the paths in walk order
        paths = np.concatenate([walk, [0xffff, 0xffff]]).astype(np.uint32)
        self.dims = (int(coo.D1), int(coo.D2), int(coo.DO), int(coo.P))
        self.nnz, self.n_segments = nnz, int(last_of_seg.sum())
        self.coef = torch.from_numpy(coef).to(device)
        self.idx = torch.from_numpy(idx.view(np.int32).copy()).to(device)
        self.paths = torch.from_numpy(paths.view(np.int32).copy()).to(device)
        t = _lib.UvuTab()
        t.coef, t.idx, t.paths = (v.data_ptr() for v in (self.coef, self.idx, self.paths))
        t.nnz, t.n_segments = self.nnz, self.n_segments
        t.D1, t.D2, t.DO, t.P = self.dims
        self.c = t


def uvu_table_of(tp_info, device) -> Optional[UvuTable]:
    """The table of ``tp_info`` for the table-driven segment kernels (cached on the info), or None when it does not
    fit them (a row index past 255, more than 8192 entries)."""
    def build():
        coo = coo_of(tp_info)
        if max(coo.D1, coo.D2, coo.DO) > 255 or coo.P > 65534 or coo.coef.shape[0] > 8192 \
                or coo.coef.shape[0] == 0:
            return False
        return UvuTable(coo, device)
    tab = cached(tp_info.info_Mij_fwd.scale, ("uvu_table", str(device)), build)
    return tab or None


def _uvu_tab_args(x: Tensor, y: Tensor, w: Tensor, seg: SegIndex) -> UvuArgs:
    a = UvuArgs()
    a.cfg, a.dtype, a.C = -1, _lib.dtype_code(x.dtype), x.shape[-1]
    a.w_shared = int(w.ndim == 2)
    a.n_rows, a.n_x_rows = y.shape[0], x.shape[0]
    a.n_seg = seg.ptr.shape[0] - 1
    a.ptr, a.perm, a.seg_ids, a.gather = seg.ptr.data_ptr(), _lib.ptr(seg.perm), seg.seg_ids.data_ptr(), \
        seg.gather.data_ptr()
    a.x, a.y, a.w = x.data_ptr(), y.data_ptr(), w.data_ptr()
    return a


def uvu_tab_launchable(tab: Optional[UvuTable], x: Tensor, y: Tensor, w: Tensor, need_grad_w: bool) -> bool:
    """Whether the table-driven segment kernels take these operands in both directions (fp32, up to 256 channels — 64
    unless a multiple of 4 and aligned —, per-edge weights or a shared weight that needs no gradient)."""
    if tab is None or x.dtype != torch.float32 or not (x.dtype == y.dtype == w.dtype):
        return False
    if x.shape[0] == 0 or y.shape[0] == 0 or y.ndim != 2 or (w.ndim == 2 and need_grad_w):
        return False
    a = UvuArgs()
    a.dtype, a.C, a.w_shared = _lib.F32, x.shape[-1], int(w.ndim == 2)
    a.n_rows, a.n_x_rows, a.n_seg = y.shape[0], x.shape[0], x.shape[0]
    dummy = 256
    a.ptr = a.seg_ids = a.gather = a.out = a.grad_out = a.grad_x = a.grad_y = dummy
    a.x, a.y, a.w = x.data_ptr() or dummy, y.data_ptr() or dummy, w.data_ptr() or dummy
    return all(_lib.lib.cgtp_uvu_tab_validate(C.byref(a), C.byref(tab.c), d) == 0 for d in (0, 1))


def _uvu_tab_workspace(a: UvuArgs, tab: UvuTable, backward: int, device):
    nbytes = int(_lib.lib.cgtp_uvu_tab_workspace_bytes(C.byref(a), C.byref(tab.c), backward))
    if nbytes < 0:
        _lib.check(_lib.lib.cgtp_uvu_tab_validate(C.byref(a), C.byref(tab.c), backward), "cgtp_uvu_tab_validate")
    if nbytes <= 0:
        return None
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    a.workspace = ws.data_ptr()
    return ws


def uvu_tab_forward(tab: UvuTable, x: Tensor, y: Tensor, w: Tensor, seg: SegIndex) -> Tensor:
    """``out[s] = sum_{q in segment s} TP(x[seg.gather[q]], y[e_q], w[e_q])`` for any table, one launch."""
    a = _uvu_tab_args(x, y, w, seg)
    out = torch.empty((a.n_seg, tab.dims[2], x.shape[-1]), dtype=x.dtype, device=x.device)
    a.out = out.data_ptr()
    ws = _uvu_tab_workspace(a, tab, 0, x.device)
    _lib.check(_lib.lib.cgtp_uvu_tab_fwd(C.byref(a), C.byref(tab.c), _lib.stream_ptr(x.device)), "cgtp_uvu_tab_fwd")
    return out


def uvu_tab_backward(tab: UvuTable, x: Tensor, y: Tensor, w: Tensor, g: Tensor, need, seg: SegIndex):
    """-> (grad_x, grad_y, grad_w) over the list sorted by the other end (``seg``: segments = rows of x)."""
    a = _uvu_tab_args(x, y, w, seg)
    a.grad_out = g.data_ptr()
    gx = torch.empty_like(x) if need[0] else None
    gy = torch.empty_like(y) if need[1] else None
    gw = torch.empty_like(w) if need[2] else None
    a.grad_x, a.grad_y, a.grad_w = _lib.ptr(gx), _lib.ptr(gy), _lib.ptr(gw)
    ws = _uvu_tab_workspace(a, tab, 1, x.device)
    _lib.check(_lib.lib.cgtp_uvu_tab_bwd(C.byref(a), C.byref(tab.c), _lib.stream_ptr(x.device)), "cgtp_uvu_tab_bwd")
    return gx, gy, gw


def uvu_sh_degree(cfg: int) -> int:
    """Degree L when the fused kernels of ``cfg`` can evaluate the second operand from edge vectors, else -1."""
    return int(_lib.lib.cgtp_uvu_sh_degree(cfg))


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
        coef = None if scale is None else scale.detach().cpu().double().numpy()
        return pack_tri_table(out_idx, i1, i2, None, coef, n_out, dtype, device), n_out
    key = ("prod", id(scale), id(index1), id(index2), id(seg), n_entries, dtype, str(device))
    return cached(anchor, key, build)
