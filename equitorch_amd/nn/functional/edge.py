"""Fused edge message passing: gather at the source node, channel-wise tensor product with the edge
harmonics and per-edge (or shared) weights, and scatter-sum to the destination node, in one kernel.

In reference terms this is the composition

    msg = SO3Linear('uu')(x.index_select(0, src), sh, W)                      (equitorch/nn/linears.py:145-187)
    out = indexed_scale_segment(msg.view(1, E, -1), None, perm, ptr, N)       (ops/indexed_scale_segment_op.py)

with ``perm`` / ``ptr`` the dst-sorted tables of ``sparse_scale_info(index_out=dst)``.  Neither the gathered
features nor the messages touch memory here; the backward walks the src-sorted edge list so that the
gradient with respect to the node features is a register-level segment sum as well.
"""
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
from ...ops import kernels
from ...structs import TensorProductInfo
from .linears import tensor_product_u1u
from .sparse_scale import sparse_scale
from ...structs import SparseScaleInfo


class EdgePlan:
    """Sorted views of an edge list ``(src, dst)`` over ``num_nodes`` nodes.

    ``perm_dst`` is the stable ascending sort of the edges by ``dst`` and ``ptr_dst`` its CSR pointer
    (``ptr_dst[v] .. ptr_dst[v+1]`` are the sorted positions whose edges end at ``v``) — bit for bit the
    ``index`` and ``seg_out`` of ``sparse_scale_info(index=range(E), index_out=dst, out_size=num_nodes)``
    (``equitorch/utils/_structs.py:22-71``; a tuple sort on ``(dst, e)`` is a stable sort on ``dst``).
    ``perm_src`` / ``ptr_src`` are the same for ``src``.  All tensors are int64 on ``src.device``.
    """

    def __init__(self, src: Tensor, dst: Tensor, num_nodes: int, num_src_nodes: Optional[int] = None):
        assert src.ndim == 1 and src.shape == dst.shape and src.dtype == dst.dtype == torch.int64
        self.src, self.dst = src.contiguous(), dst.contiguous()
        self.num_nodes = int(num_nodes)
        self.num_src_nodes = int(num_src_nodes if num_src_nodes is not None else num_nodes)
        self.num_edges = src.shape[0]
        self.perm_dst, self.ptr_dst = self._sorted(self.dst, self.num_nodes)
        self.perm_src, self.ptr_src = self._sorted(self.src, self.num_src_nodes)
        # per-sorted-position views for the fused kernels: segment id and the row gathered at the other end
        self.fwd_index = kernels.SegIndex(self.ptr_dst, self.perm_dst, self.dst[self.perm_dst].contiguous(),
                                          self.src[self.perm_dst].contiguous())
        self.bwd_index = kernels.SegIndex(self.ptr_src, self.perm_src, self.src[self.perm_src].contiguous(),
                                          self.dst[self.perm_src].contiguous())

    @staticmethod
    def _sorted(key: Tensor, n: int):
        perm = torch.sort(key, stable=True).indices
        ptr = torch.zeros(n + 1, dtype=torch.int64, device=key.device)
        ptr[1:] = torch.cumsum(torch.bincount(key, minlength=n), 0)
        return perm.contiguous(), ptr

    def scale_infos(self):
        """(forward, transposed) ``SparseScaleInfo`` of the scatter-sum, for ``sparse_scale``."""
        return (SparseScaleInfo(None, self.perm_dst, self.ptr_dst, None, self.num_nodes),
                SparseScaleInfo(None, self.dst, None, None, self.num_edges))


def _check_edge_operands(x: Tensor, y: Tensor, plan: EdgePlan, tp_info: TensorProductInfo, weight: Optional[Tensor] = None,
                         h: Optional[Tensor] = None, w_last: Optional[Tensor] = None, edge_vectors: bool = False) -> None:
    """Operand extents against the edge list and the table, before any kernel sees them: the fused kernels read
    ``P * C`` weights and ``D2`` (or 3) values of the second operand for every edge of the plan, and ``D1 * C`` values
    of every source node, whatever the tensors hold."""
    coo = kernels.coo_of(tp_info)
    e = plan.num_edges
    if plan.num_src_nodes != x.shape[0]:
        raise _lib.CgtpError(f"plan was built for {plan.num_src_nodes} source nodes, x has {x.shape[0]}")
    if x.ndim != 3 or x.shape[1] != coo.D1:
        raise _lib.CgtpError(f"x must be (N_src, {coo.D1}, C) for this table, got {tuple(x.shape)}")
    d2 = 3 if edge_vectors else coo.D2
    if y.ndim != 2 or y.shape[0] != e or y.shape[1] != d2:
        raise _lib.CgtpError(f"the second operand must be ({e}, {d2}) for this plan and table, got {tuple(y.shape)}")
    c = x.shape[2]
    if weight is not None:
        ok = (weight.ndim == 2 and tuple(weight.shape) == (coo.P, c)) or \
             (weight.ndim == 3 and tuple(weight.shape) == (e, coo.P, c))
        if not ok:
            raise _lib.CgtpError(f"weight must be ({coo.P}, {c}) or ({e}, {coo.P}, {c}), got {tuple(weight.shape)}")
    if h is not None:
        if h.ndim != 2 or h.shape[0] != e:
            raise _lib.CgtpError(f"h must be ({e}, R), got {tuple(h.shape)}")
        if w_last.ndim != 3 or tuple(w_last.shape) != (h.shape[1], coo.P, c):
            raise _lib.CgtpError(f"w_last must be ({h.shape[1]}, {coo.P}, {c}), got {tuple(w_last.shape)}")


def _unfused(plan: EdgePlan, tp_info: TensorProductInfo, y_vec: int = 0):
    """``expression(x, y, w)``: the same result from the three steps the fused kernels replace — gather, product on the
    batch of edges, segment sum — each of which autograd differentiates to any order (``y``: harmonics, or edge vectors
    when ``y_vec`` says so).  The fused kernels' backward evaluates it when a gradient of the gradient is asked for
    (forces in the loss), as the reference's composition of differentiable functions would be.  Holds the plan's
    tensors, not the plan."""
    src, infos, num_nodes = plan.src, plan.scale_infos(), plan.num_nodes
    d2 = int(kernels.coo_of(tp_info).D2)

    def expression(x: Tensor, y: Tensor, w: Tensor) -> Tensor:
        if y_vec:
            from .sphericals import spherical_harmonics
            y = spherical_harmonics(y, int(round(d2 ** 0.5)) - 1, normalize_input=(y_vec == kernels.Y_UNIT_VECTOR))
        msg = tensor_product_u1u(x.index_select(0, src), y, w, tp_info)
        e, d, c = msg.shape
        return sparse_scale(msg.view(1, e, d * c), *infos).view(num_nodes, d, c)
    return expression


def _higher_order(expression, inputs, need, g: Tensor):
    """Gradients of ``expression(*inputs)`` for the inputs ``need`` marks, themselves differentiable."""
    with torch.enable_grad():
        wanted = [t for t, n in zip(inputs, need) if n]
        grads = iter(torch.autograd.grad(expression(*inputs), wanted, g, create_graph=True, allow_unused=True))
    return tuple(next(grads) if n else None for n in need)


def _shim_handle(plan: EdgePlan, cfg, x: Tensor, y_vec: int, tp_info: TensorProductInfo):
    """The C++ extension's handle of this plan for one compiled table, dtype and channel count (it holds the sorted
    views and the range tables of both directions), or None when the extension is not there or the table needs the
    weights rearranged (a subset of the compiled paths)."""
    from ... import _shim
    mod = _shim.module()
    if mod is None or getattr(cfg, "w_rows", None) is not None:
        return None
    scale_np = getattr(cfg, "path_scale", None)
    key = (int(cfg), x.dtype, x.shape[-1], y_vec, None if scale_np is None else scale_np.tobytes())
    handles = plan.__dict__.setdefault("_shim_handles", {})
    if key not in handles:
        code = _lib.dtype_code(x.dtype)
        scale = cfg.scale_tensor(x.dtype, x.device) if isinstance(cfg, kernels.Cfg) else None
        views = []
        for seg, backward in ((plan.fwd_index, False), (plan.bwd_index, True)):
            wave_seg, wave_pos = kernels.seg_ranges(cfg, seg, code, x.shape[-1], backward)
            views += [seg.ptr, seg.perm, seg.seg_ids, seg.gather, wave_seg, wave_pos]
        handles[key] = mod.EdgeHandle(int(cfg), int(kernels.uvu_dims(cfg)[2]), int(y_vec), scale, *views)
        expression = _unfused(plan, tp_info, y_vec)
        handles[key].set_fallback(lambda g, x_, y_, w_, *need: _higher_order(expression, (x_, y_, w_), need, g))
    return handles[key]


class _EdgeUvuCompiled(Function):
    @staticmethod
    def forward(ctx, x: Tensor, sh: Tensor, w: Tensor, plan: EdgePlan, tp_info: TensorProductInfo, cfg: int):
        dims = kernels.uvu_dims(cfg)
        out = kernels.uvu_forward(cfg, dims, x, sh, w, seg=plan.fwd_index)
        ctx.save_for_backward(x, sh, w)
        ctx.plan, ctx.cfg, ctx.dims, ctx.tp_info = plan, cfg, dims, tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        x, sh, w = ctx.saved_tensors
        plan = ctx.plan
        if torch.is_grad_enabled():
            return (*_higher_order(_unfused(plan, ctx.tp_info), (x, sh, w), ctx.needs_input_grad[:3], g), None, None, None)
        res = kernels.uvu_backward(ctx.cfg, ctx.dims, x, sh, w, g.contiguous(), ctx.needs_input_grad[:3],
                                   seg=plan.bwd_index)
        return (*res, None, None, None)


class _EdgeUvuVectors(Function):
    """The fused kernels with the harmonics evaluated inside them: the second operand is the edge vector."""

    @staticmethod
    def forward(ctx, x: Tensor, vec: Tensor, w: Tensor, plan: EdgePlan, cfg: int, y_vec: int, tp_info: TensorProductInfo):
        dims = kernels.uvu_dims(cfg)
        out = kernels.uvu_forward(cfg, dims, x, vec, w, seg=plan.fwd_index, y_vec=y_vec)
        ctx.save_for_backward(x, vec, w)
        ctx.plan, ctx.cfg, ctx.dims, ctx.y_vec, ctx.tp_info = plan, cfg, dims, y_vec, tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        x, vec, w = ctx.saved_tensors
        if torch.is_grad_enabled():
            expression = _unfused(ctx.plan, ctx.tp_info, ctx.y_vec)
            return (*_higher_order(expression, (x, vec, w), ctx.needs_input_grad[:3], g), None, None, None, None)
        res = kernels.uvu_backward(ctx.cfg, ctx.dims, x, vec, w, g.contiguous(), ctx.needs_input_grad[:3],
                                   seg=ctx.plan.bwd_index, y_vec=ctx.y_vec)
        return (*res, None, None, None, None)


class _EdgeUvuRadial(Function):
    """The fused kernels with the per-edge weights ``h @ w_last`` formed inside them (``y_vec`` 0: the second operand
    is given as harmonics, else as edge vectors)."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, h: Tensor, w_last: Tensor, plan: EdgePlan, cfg: int, y_vec: int,
                tp_info: TensorProductInfo):
        dims = kernels.uvu_dims(cfg)
        w_eff = kernels.radial_effective_weight(w_last, cfg)       # over the compiled paths, the table's factors folded in
        out = kernels.uvu_radial_forward(cfg, dims, x, y, h, w_eff, plan.fwd_index, y_vec)
        ctx.save_for_backward(x, y, h, w_last, w_eff)
        ctx.plan, ctx.cfg, ctx.dims, ctx.y_vec, ctx.tp_info = plan, cfg, dims, y_vec, tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        x, y, h, w_last, w_eff = ctx.saved_tensors
        need = ctx.needs_input_grad[:4]
        if torch.is_grad_enabled():
            plain = _unfused(ctx.plan, ctx.tp_info, ctx.y_vec)

            def expression(x_, y_, h_, w_):
                return plain(x_, y_, (h_ @ w_.reshape(w_.shape[0], -1)).view(h_.shape[0], *w_.shape[1:]))
            return (*_higher_order(expression, (x, y, h, w_last), need, g), None, None, None, None)
        gx, gy, gh, gwe = kernels.uvu_radial_backward(ctx.cfg, ctx.dims, x, y, h, w_eff, g.contiguous(), need,
                                                      ctx.plan.bwd_index, ctx.y_vec)
        gwl = None
        if need[3]:       # back through the rearrangement of the paths (linear in w_last)
            with torch.enable_grad():
                wl = w_last.detach().requires_grad_(True)
                we = kernels.radial_effective_weight(wl, ctx.cfg)
            (gwl,) = torch.autograd.grad(we, wl, gwe)
        return gx, gy, gh, gwl, None, None, None, None


class _EdgeUvuTable(Function):
    """Gather, product and segment sum in one launch for a table that is not compiled in: the table-driven segment
    kernels (``cgtp_uvu_tab_fwd`` / ``cgtp_uvu_tab_bwd``), tables read through the scalar cache, the per-edge
    operands and the segment sums in LDS."""

    @staticmethod
    def forward(ctx, x: Tensor, sh: Tensor, w: Tensor, plan: EdgePlan, tab, tp_info: TensorProductInfo):
        out = kernels.uvu_tab_forward(tab, x, sh, w, plan.fwd_index)
        ctx.save_for_backward(x, sh, w)
        ctx.plan, ctx.tab, ctx.tp_info = plan, tab, tp_info
        return out

    @staticmethod
    def backward(ctx, g):
        x, sh, w = ctx.saved_tensors
        if torch.is_grad_enabled():
            return (*_higher_order(_unfused(ctx.plan, ctx.tp_info), (x, sh, w), ctx.needs_input_grad[:3], g), None, None, None)
        res = kernels.uvu_tab_backward(ctx.tab, x, sh, w, g.contiguous(), ctx.needs_input_grad[:3], ctx.plan.bwd_index)
        return (*res, None, None, None)


class _EdgeUvuRows(Function):
    """The same composition on the row-mode kernels, for tables the fused segment kernels do not cover: per-edge
    messages from the gathered node rows, then a segment sum over the dst-sorted list; the backward forms the
    per-edge gradient of the gathered rows and sums it over the src-sorted list."""

    @staticmethod
    def forward(ctx, x: Tensor, sh: Tensor, w: Tensor, plan: EdgePlan, tp_info: TensorProductInfo, cfg: int):
        dims = kernels.uvu_dims(cfg)
        msg = kernels.uvu_forward(cfg, dims, x, sh, w, gather=plan.src)
        e, d, c = msg.shape
        out = kernels.segment_sum(msg.view(1, e, d * c), None, plan.perm_dst, plan.ptr_dst, plan.num_nodes)
        ctx.save_for_backward(x, sh, w)
        ctx.plan, ctx.cfg, ctx.dims, ctx.tp_info = plan, cfg, dims, tp_info
        return out.view(plan.num_nodes, d, c)

    @staticmethod
    def backward(ctx, g):
        x, sh, w = ctx.saved_tensors
        plan = ctx.plan
        need = ctx.needs_input_grad[:3]
        if torch.is_grad_enabled():
            return (*_higher_order(_unfused(plan, ctx.tp_info), (x, sh, w), need, g), None, None, None)
        gxe, gy, gw = kernels.uvu_backward(ctx.cfg, ctx.dims, x, sh, w, g.contiguous(), need, gather=plan.dst,
                                           x_gather=plan.src)
        gx = None
        if need[0]:
            e, d, c = gxe.shape
            gx = kernels.segment_sum(gxe.view(1, e, d * c), None, plan.perm_src, plan.ptr_src,
                                     plan.num_src_nodes).view(plan.num_src_nodes, d, c)
        return gx, gy, gw, None, None, None


def edge_tensor_product_uu(x: Tensor, sh: Tensor, weight: Tensor, plan: EdgePlan,
                           tp_info_forward: TensorProductInfo,
                           tp_info_backward1: Optional[TensorProductInfo] = None,
                           tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``out[v] = sum_{e: dst[e]=v} TP_uu(x[src[e]], sh[e], W[e])``.

    ``x (N_src, D1, C)``, ``sh (E, D2)``, ``weight (E, P, C) | (P, C)`` -> ``(N, DO, C)``.  Uses the fused
    kernel when the table of ``tp_info_forward`` is compiled in and one wavefront slot covers the channels (large
    tables, e.g. lmax = 6: fp32 with per-edge weights); otherwise runs the same three steps as separate launches.
    """
    _lib.require_gpu(x, sh, weight)
    _check_edge_operands(x, sh, plan, tp_info_forward, weight=weight)
    cfg = kernels.uvu_config_of(tp_info_forward)
    if cfg >= 0 and x.dtype == sh.dtype == weight.dtype and x.dtype in (torch.float32, torch.float64):
        xc, yc, wc = x.contiguous(), sh.contiguous(), weight.contiguous()
        if kernels.uvu_launchable(cfg, xc, yc, wc, segments=True):
            kernels.log_tier("edge_tensor_product_uu", "fused gather / product / segment sum", f"config {int(cfg)}")
            handle = _shim_handle(plan, cfg, xc, 0, tp_info_forward)
            if handle is not None:
                from ... import _shim
                return _shim.module().edge_uvu(xc, yc, wc, handle)
            return _EdgeUvuCompiled.apply(xc, yc, wc, plan, tp_info_forward, cfg)
        if kernels.uvu_launchable(cfg, xc, yc, wc, gathered=True):
            kernels.log_tier("edge_tensor_product_uu", "block-wise row kernels + segment sums", f"config {int(cfg)}")
            return _EdgeUvuRows.apply(xc, yc, wc, plan, tp_info_forward, cfg)
    if x.dtype == sh.dtype == weight.dtype == torch.float32:
        tab = kernels.uvu_table_of(tp_info_forward, x.device)
        xc, yc, wc = x.contiguous(), sh.contiguous(), weight.contiguous()
        if kernels.uvu_tab_launchable(tab, xc, yc, wc, weight.requires_grad and torch.is_grad_enabled()):
            kernels.log_tier("edge_tensor_product_uu", "table-driven fused gather / product / segment sum",
                             f"{tab.nnz} coefficients")
            return _EdgeUvuTable.apply(xc, yc, wc, plan, tab, tp_info_forward)
    kernels.log_tier("edge_tensor_product_uu", "index_select + tensor_product_u1u + sparse_scale")
    msg = tensor_product_u1u(x.index_select(0, plan.src), sh, weight, tp_info_forward)
    e, d, c = msg.shape
    fwd, bwd = plan.scale_infos()
    return sparse_scale(msg.view(1, e, d * c), fwd, bwd).view(plan.num_nodes, d, c)


def edge_tensor_product_uu_vectors(x: Tensor, edge_vec: Tensor, weight: Tensor, plan: EdgePlan,
                                   tp_info_forward: TensorProductInfo, normalize_input: bool = True,
                                   tp_info_backward1: Optional[TensorProductInfo] = None,
                                   tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """:func:`edge_tensor_product_uu` with ``sh = SphericalHarmonics(l_max, normalize_input)(edge_vec)``
    (``equitorch/nn/sphericals.py:31-35``) evaluated inside the edge kernels: ``edge_vec (E, 3)`` replaces the
    ``(E, (l_max+1)^2)`` harmonics as an input, and its gradient the harmonics' gradient as an output.  ``l_max`` is
    the degree of the second operand of ``tp_info_forward``, which must be laid out like harmonics (degrees
    ``0..l_max`` in order).  Tables without fused kernels take the harmonics kernel followed by
    :func:`edge_tensor_product_uu`.
    """
    from .sphericals import spherical_harmonics
    _lib.require_gpu(x, edge_vec, weight)
    if edge_vec.ndim != 2 or edge_vec.shape[1] != 3:
        raise ValueError(f"edge_vec must be (E, 3), got {tuple(edge_vec.shape)}")
    _check_edge_operands(x, edge_vec, plan, tp_info_forward, weight=weight, edge_vectors=True)
    cfg = kernels.uvu_config_of(tp_info_forward)
    mode = kernels.Y_UNIT_VECTOR if normalize_input else kernels.Y_RAW_VECTOR
    if (cfg >= 0 and kernels.uvu_sh_degree(cfg) >= 0 and x.dtype == edge_vec.dtype == weight.dtype
            and x.dtype in (torch.float32, torch.float64)):
        xc, vc, wc = x.contiguous(), edge_vec.contiguous(), weight.contiguous()
        if kernels.uvu_launchable(cfg, xc, vc, wc, segments=True, y_vec=mode):
            handle = _shim_handle(plan, cfg, xc, mode, tp_info_forward)
            if handle is not None:
                from ... import _shim
                return _shim.module().edge_uvu(xc, vc, wc, handle)
            return _EdgeUvuVectors.apply(xc, vc, wc, plan, cfg, mode, tp_info_forward)
    d2 = int(kernels.coo_of(tp_info_forward).D2)
    l_max = int(round(d2 ** 0.5)) - 1
    if (l_max + 1) ** 2 != d2:
        raise ValueError(f"second operand of the table has {d2} components: not a set of harmonics 0..l_max")
    sh = spherical_harmonics(edge_vec, l_max, normalize_input=normalize_input)
    return edge_tensor_product_uu(x, sh, weight, plan, tp_info_forward, tp_info_backward1, tp_info_backward2)


def edge_tensor_product_uu_radial(x: Tensor, sh_or_vec: Tensor, h: Tensor, w_last: Tensor, plan: EdgePlan,
                                  tp_info_forward: TensorProductInfo, edge_vectors: bool = False,
                                  normalize_input: bool = True) -> Tensor:
    """:func:`edge_tensor_product_uu` (or, with ``edge_vectors``, :func:`edge_tensor_product_uu_vectors`) with the
    per-edge weights ``weight[e] = h[e] @ w_last`` — the last linear layer of the network that turns radial features
    (``BesselBasis`` with a cutoff, ``equitorch/nn/radials.py:10-58``, ``nn/cutoffs.py:7-131``, and the user's MLP) into
    tensor-product weights — formed inside the edge kernels, so that the ``(E, P, C)`` weight tensor is neither written
    nor read in the forward.  ``h (E, R)``, ``w_last (R, P, C)`` (``nn.Linear(R, P * C, bias=False).weight.T`` viewed
    that way; a bias is a constant feature).  fp32, ``C = 64``, ``R`` a multiple of 4 up to 16 on the fused path; other
    shapes form ``h @ w_last`` with a matrix product and take the plain functions.
    """
    _lib.require_gpu(x, sh_or_vec, h, w_last)
    _check_edge_operands(x, sh_or_vec, plan, tp_info_forward, h=h, w_last=w_last, edge_vectors=edge_vectors)
    cfg = kernels.uvu_config_of(tp_info_forward)
    mode = 0 if not edge_vectors else (kernels.Y_UNIT_VECTOR if normalize_input else kernels.Y_RAW_VECTOR)
    xc, yc, hc = x.contiguous(), sh_or_vec.contiguous(), h.contiguous()
    # a misaligned operand (a view at an odd offset) takes the matrix-product route below instead of an error
    if (kernels.uvu_radial_supported(cfg, xc, hc, w_last) and yc.dtype == xc.dtype and yc.data_ptr() % 16 == 0
            and (not edge_vectors or kernels.uvu_sh_degree(cfg) >= 0)):
        kernels.log_tier("edge_tensor_product_uu_radial", "fused gather / weights / product / segment sum",
                         f"config {int(cfg)}")
        return _EdgeUvuRadial.apply(xc, yc, hc, w_last, plan, cfg, mode, tp_info_forward)
    kernels.log_tier("edge_tensor_product_uu_radial", "weights by matrix product, then the plain edge product")
    weight = (h @ w_last.reshape(w_last.shape[0], -1)).view(h.shape[0], *w_last.shape[1:])
    if edge_vectors:
        return edge_tensor_product_uu_vectors(x, sh_or_vec, weight, plan, tp_info_forward, normalize_input)
    return edge_tensor_product_uu(x, sh_or_vec, weight, plan, tp_info_forward)
