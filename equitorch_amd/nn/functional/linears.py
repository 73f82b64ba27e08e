"""Channel-wise tensor products where one operand has no channel axis (the ``SO3Linear('uu')`` family).

Reference: ``equitorch/nn/functional/linears.py:16-252``.  There each product is two kernel launches with the
``(N, n_segments, C)`` intermediate ``inter`` written to memory, saved for the backward and returned as a
second output; here each product is one fused launch and nothing but the inputs is saved.

    u1u : out[n,M,c] = sum_t c_t x[n,M1_t,c] y[n,M2_t]   W[(n),p_t,c]
    1uu : out[n,M,c] = sum_t c_t x[n,M1_t]   y[n,M2_t,c] W[(n),p_t,c]
    uu1 : out[n,M]   = sum_t c_t sum_c x[n,M1_t,c] y[n,M2_t,c] W[(n),p_t,c]

and the fully connected siblings u1v / 1vu / vu1 (``SO3Linear('uv')`` family, reference ``:254-492``) at the end
of the file.

``weight`` is shared ``(P, C)`` or per-sample ``(N, P, C)``.  Only ``tp_info_forward`` is read; the two
backward tables are accepted for signature compatibility.
"""
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
S, V = "", "u"  # channel axes of an operand: none / one
from ...ops import kernels
from ...structs import TensorProductInfo
from ._tri import spec_from_tp_info, tri


class _UvuCompiled(Function):
    """u1u on the kernels with a compiled-in table (``cgtp_uvu_fwd`` / ``cgtp_uvu_bwd``)."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info: TensorProductInfo, cfg: int):
        out = kernels.uvu_forward(cfg, kernels.uvu_dims(cfg), x, y, w)
        ctx.save_for_backward(x, y, w)
        ctx.tp_info, ctx.cfg = tp_info, cfg
        return out

    @staticmethod
    def backward(ctx, g):
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        if torch.is_grad_enabled():
            # higher-order derivative requested: re-express through the differentiable contraction
            with torch.enable_grad():
                spec = spec_from_tp_info(ctx.tp_info)
                gx = tri(spec.grad_spec(0), (V, S, V), V, g, y, w) if need[0] else None
                gy = tri(spec.grad_spec(1), (V, V, V), S, x, g, w) if need[1] else None
                gw = tri(spec.grad_spec(2), (V, S, V), V, x, y, g, out_shared=(w.ndim == 2)) if need[2] else None
            return gx, gy, gw, None, None
        res = kernels.uvu_backward(ctx.cfg, kernels.uvu_dims(ctx.cfg), x, y, w, g.contiguous(), need)
        return (*res, None, None)


class _UvuTableRows(Function):
    """u1u for a table that is not compiled in, on the table-driven segment kernels (``cgtp_uvu_tab_fwd`` / ``_bwd``)
    with the batch as an edge list of one edge per node."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info: TensorProductInfo, tab):
        out = kernels.uvu_tab_forward(tab, x, y, w, kernels.identity_segments(x.shape[0], x.device))
        ctx.save_for_backward(x, y, w)
        ctx.tp_info, ctx.tab = tp_info, tab
        return out

    @staticmethod
    def backward(ctx, g):
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad[:3]
        if torch.is_grad_enabled():   # higher-order derivative requested: the differentiable contraction
            with torch.enable_grad():
                spec = spec_from_tp_info(ctx.tp_info)
                gx = tri(spec.grad_spec(0), (V, S, V), V, g, y, w) if need[0] else None
                gy = tri(spec.grad_spec(1), (V, V, V), S, x, g, w) if need[1] else None
                gw = tri(spec.grad_spec(2), (V, S, V), V, x, y, g, out_shared=(w.ndim == 2)) if need[2] else None
            return gx, gy, gw, None, None
        res = kernels.uvu_tab_backward(ctx.tab, x, y, w, g.contiguous(), need,
                                       kernels.identity_segments(x.shape[0], x.device))
        return (*res, None, None)


def _row_uvu_extension(x: Tensor, y: Tensor, w: Tensor, tp_info: TensorProductInfo, cfg):
    """The same launches issued by the C++ extension (autograd node and argument block in C++), or None: extension
    not there, a table that needs its weights rearranged, or a shared weight whose per-row gradient workspace the
    Python side would split."""
    from ... import _shim
    mod = _shim.module()
    if mod is None or getattr(cfg, "w_rows", None) is not None:
        return None
    if w.ndim == 2 and w.requires_grad and mod.row_backward_workspace(x, y, w, int(cfg)) > kernels._GW_WORKSPACE_BYTES:
        return None

    def register():
        def second_order(g, x_, y_, w_, need_x, need_y, need_w):
            with torch.enable_grad():
                spec = spec_from_tp_info(tp_info)
                gx = tri(spec.grad_spec(0), (V, S, V), V, g, y_, w_) if need_x else None
                gy = tri(spec.grad_spec(1), (V, V, V), S, x_, g, w_) if need_y else None
                gw = tri(spec.grad_spec(2), (V, S, V), V, x_, y_, g, out_shared=(w_.ndim == 2)) if need_w else None
            return gx, gy, gw
        return mod.register_fallback(second_order)
    fallback = kernels.cached(tp_info.info_Mij_fwd.scale, "row_uvu_fallback", register)
    scale = cfg.scale_tensor(x.dtype, x.device) if isinstance(cfg, kernels.Cfg) else None
    return mod.row_uvu(x, y, w, scale, int(cfg), int(kernels.uvu_dims(cfg)[2]), fallback)


def _check_batch(input1, input2, weight):
    _lib.require_gpu(input1, input2, weight)


def _widen(*tensors: Tensor) -> bool:
    """All operands in one 16-bit floating type."""
    return tensors[0].dtype in (torch.bfloat16, torch.float16) and all(t.dtype == tensors[0].dtype for t in tensors)


def tensor_product_u1u(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1, C)``, ``input2 (N, D2)``, ``weight (P, C) | (N, P, C)`` -> ``(N, DO, C)``."""
    _check_batch(input1, input2, weight)
    if (input1.ndim == 3 and input2.ndim == 2 and input1.dtype == input2.dtype == weight.dtype
            and input1.dtype in (torch.float32, torch.float64)):
        cfg = kernels.uvu_config_of(tp_info_forward)
        x, y, w = input1.contiguous(), input2.contiguous(), weight.contiguous()
        if cfg >= 0 and kernels.uvu_launchable(cfg, x, y, w):
            kernels.log_tier("tensor_product_u1u", "compiled table", f"config {int(cfg)}")
            out = _row_uvu_extension(x, y, w, tp_info_forward, cfg)
            if out is not None:
                return out
            return _UvuCompiled.apply(x, y, w, tp_info_forward, cfg)
    if (input1.ndim == 3 and input2.ndim == 2 and input1.dtype == input2.dtype == weight.dtype == torch.float32
            and input1.shape[0] == input2.shape[0] and input1.shape[0] > 0):
        # no compiled table: the table-driven segment kernels of the edge products, the batch seen as an edge list in
        # which every row is a node with one edge (entries walked from registers, operands in LDS: about a third of the
        # time of the general contraction kernel below, which reads every operand of every coefficient from memory)
        tab = kernels.uvu_table_of(tp_info_forward, input1.device)
        x, y, w = input1.contiguous(), input2.contiguous(), weight.contiguous()
        if kernels.uvu_tab_launchable(tab, x, y, w, weight.requires_grad and torch.is_grad_enabled()):
            kernels.log_tier("tensor_product_u1u", "table-driven segment kernels on the batch", f"{tab.nnz} coefficients")
            return _UvuTableRows.apply(x, y, w, tp_info_forward, tab)
    kernels.log_tier("tensor_product_u1u", "table-driven kernel", str(input1.dtype))
    return tri(spec_from_tp_info(tp_info_forward), (V, S, V), V, input1, input2, weight)


so3_linear_uu = tensor_product_u1u


def tensor_product_1uu(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1)``, ``input2 (N, D2, C)`` -> ``(N, DO, C)``."""
    _check_batch(input1, input2, weight)
    return tri(spec_from_tp_info(tp_info_forward), (S, V, V), V, input1, input2, weight)


def tensor_product_uu1(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1, C)``, ``input2 (N, D2, C)`` -> ``(N, DO)`` (summed over channels)."""
    _check_batch(input1, input2, weight)
    return tri(spec_from_tp_info(tp_info_forward), (V, V, V), S, input1, input2, weight)


# ---- fully connected in the channels: weight (P, C_in, C_out) or (N, P, C_in, C_out) ---------------------------
def tensor_product_u1v(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``out[n,M,w] = sum_t c_t y[n,M2_t] sum_u x[n,M1_t,u] W[(n),p_t,u,w]`` — ``input1 (N, D1, C_in)``,
    ``input2 (N, D2)`` -> ``(N, DO, C_out)`` (reference ``linears.py:254-336``)."""
    _check_batch(input1, input2, weight)
    from . import _uv_gemm, _uvw_mfma
    fast = _uvw_mfma.try_forward(input1, input2, weight, tp_info_forward)
    if fast is not None:
        kernels.log_tier("tensor_product_u1v", "matrix-core kernel (compiled table)")
        return fast
    from . import _uv_native
    if _uv_native.u1v_supported(input1, input2, weight, tp_info_forward):
        kernels.log_tier("tensor_product_u1v", "fp32 matrix-core kernel (table-driven)")
        return _uv_native.u1v(input1, input2, weight, tp_info_forward)
    if (weight.ndim == 3 and input1.ndim == 3 and input2.ndim == 2 and input1.dtype == input2.dtype == weight.dtype
            and input1.dtype in (torch.float32, torch.float64) and (weight.shape[1] % 4 or weight.shape[2] % 4)):
        # channel counts that are not multiples of 4 (the kernels move 16 bytes per lane): zero channels appended to
        # the operand and the weight, the result cut back
        u, wc = weight.shape[1:]
        u4, w4 = -(-u // 4) * 4, -(-wc // 4) * 4
        if _uv_native.u1v_fits(input1.shape[0], u4, w4, tp_info_forward, input1.dtype):
            kernels.log_tier("tensor_product_u1v", "channel counts padded to multiples of 4", f"{u} -> {wc}")
            pad = torch.nn.functional.pad
            out = tensor_product_u1v(pad(input1, (0, u4 - u)), input2, pad(weight, (0, w4 - wc, 0, u4 - u)),
                                     tp_info_forward)
            return out[..., :wc].contiguous()
    if _widen(input1, input2, weight) and input1.ndim == 3 and input2.ndim == 2 and (
            weight.ndim == 4 or (weight.ndim == 3 and _uv_native.u1v_fits(
                input1.shape[0], weight.shape[1], weight.shape[2], tp_info_forward, torch.float32))):
        # 16-bit operands on a table without compiled matrix-core kernels: the table-driven kernels in fp32
        # arithmetic on widened copies (at 4096 samples, 64 channels, 0e+1e+2e+3e: 0.10 against 0.78 ms for the
        # library route in bf16), the result rounded once
        kernels.log_tier("tensor_product_u1v", "operands widened to fp32", str(input1.dtype))
        return tensor_product_u1v(input1.float(), input2.float(), weight.float(), tp_info_forward).to(input1.dtype)
    if weight.ndim == 4:
        from . import _psw
        table = _psw.table_of_coo(kernels.coo_of(tp_info_forward), tp_info_forward.info_Mij_fwd.scale, 1, input1.device)
        if _psw.launchable(table, input1, input2, weight):
            kernels.log_tier("tensor_product_u1v", "per-sample weight streaming kernel", str(input1.dtype))
            return _psw.product(table, input1, input2, weight,
                                lambda x, y, w: _uv_gemm.u1v(x, y, w, tp_info_forward))
    if input1.ndim == 3 and input2.ndim == 2 and _uv_gemm.supported(input1, input2, weight):
        kernels.log_tier("tensor_product_u1v", "library GEMM + table-driven kernel", str(input1.dtype))
        return _uv_gemm.u1v(input1, input2, weight, tp_info_forward)
    kernels.log_tier("tensor_product_u1v", "general two-axis kernel", str(input1.dtype))
    return tri(spec_from_tp_info(tp_info_forward), ("u", "", "uw"), "w", input1, input2, weight)


so3_linear_uv = tensor_product_u1v


def tensor_product_1vu(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``input1 (N, D1)``, ``input2 (N, D2, C_in)`` -> ``(N, DO, C_out)`` (reference ``:338-412``)."""
    _check_batch(input1, input2, weight)
    from . import _uv_gemm
    if weight.ndim == 4 and input1.ndim == 2 and input2.ndim == 3:
        from . import _psw
        table = _psw.table_of_coo(kernels.coo_of(tp_info_forward), tp_info_forward.info_Mij_fwd.scale, 2, input1.device)
        if _psw.launchable(table, input2, input1, weight):
            kernels.log_tier("tensor_product_1vu", "per-sample weight streaming kernel", str(input1.dtype))
            return _psw.product(table, input2, input1, weight,
                                lambda x, y, w: _uv_gemm.one_vu(y, x, w, tp_info_forward))
    if input1.ndim == 2 and input2.ndim == 3 and weight.ndim == 3:
        from . import _uv_native
        table = _uv_native.operands_exchanged(tp_info_forward)
        if _uv_native.u1v_supported(input2, input1, weight, table):
            kernels.log_tier("tensor_product_1vu", "fp32 matrix-core kernel (table-driven)")
            return _uv_native.u1v(input2, input1, weight, table)
    if input1.ndim == 2 and input2.ndim == 3 and _uv_gemm.supported(input1, input2, weight):
        kernels.log_tier("tensor_product_1vu", "library GEMM + table-driven kernel", str(input1.dtype))
        return _uv_gemm.one_vu(input1, input2, weight, tp_info_forward)
    return tri(spec_from_tp_info(tp_info_forward), ("", "u", "uw"), "w", input1, input2, weight)


def tensor_product_vu1(input1: Tensor, input2: Tensor, weight: Tensor,
                       tp_info_forward: TensorProductInfo,
                       tp_info_backward1: Optional[TensorProductInfo] = None,
                       tp_info_backward2: Optional[TensorProductInfo] = None) -> Tensor:
    """``out[n,M] = sum_t c_t sum_{u,w} x[n,M1_t,u] W[(n),p_t,u,w] y[n,M2_t,w]`` — ``input1 (N, D1, C1)``,
    ``input2 (N, D2, C2)``, ``weight (P, C1, C2)`` -> ``(N, DO)`` (reference ``:414-492``)."""
    _check_batch(input1, input2, weight)
    from . import _uv_gemm
    if weight.ndim == 4 and input1.ndim == 3 and input2.ndim == 3:
        # a weight per sample: the uvw product with one output channel, W read as (N, P, C1 * C2, 1)
        from . import _psw
        table = _psw.table_of_coo(kernels.coo_of(tp_info_forward), tp_info_forward.info_Mij_fwd.scale, 1, input1.device)
        w4 = weight.contiguous().flatten(2, 3).unsqueeze(-1)
        if _psw.launchable(table, input1, input2, w4):
            kernels.log_tier("tensor_product_vu1", "per-sample weight streaming kernel", str(input1.dtype))
            shape = weight.shape
            return _psw.product(table, input1, input2, w4, lambda x, y, w: _uv_gemm.vu1(
                x, y, w.reshape(shape), tp_info_forward).unsqueeze(-1)).squeeze(-1)
    from . import _uv_native
    if _uv_native.vu1_supported(input1, input2, weight, tp_info_forward):
        kernels.log_tier("tensor_product_vu1", "fp32 matrix-core kernel (table-driven)")
        return _uv_native.vu1(input1, input2, weight, tp_info_forward)
    if input1.ndim == 3 and input2.ndim == 3 and _uv_gemm.supported(input1, input2, weight):
        kernels.log_tier("tensor_product_vu1", "library GEMM + table-driven kernel", str(input1.dtype))
        return _uv_gemm.vu1(input1, input2, weight, tp_info_forward)
    return tri(spec_from_tp_info(tp_info_forward), ("u", "w", "uw"), "", input1, input2, weight)


# ---- irreps-preserving channel mixing (reference :494-571) ------------------------------------------------------
def irreps_linear(input: Tensor, weight: Tensor, irreps_linear_info_forward, irreps_linear_info_backward=None):
    r"""``out[n, M, :] = sum_{(M, M0, p)} scale * input[n, M0, :] @ weight[(n,) p]`` over the entries of the table
    (``IrrepsLinear.forward``, reference ``:528-571``): channel mixing between input and output irreps of equal
    degree and parity.  ``weight`` is ``(P, C_in, C_out)`` or ``(N, P, C_in, C_out)``.  Runs as library GEMMs on
    the strided component rows (``_irreps_gemm``); only the forward table is read."""
    from . import _irreps_gemm as G
    plan = G.plan_of_linear_info(irreps_linear_info_forward)
    in_size = (irreps_linear_info_backward.out_size if irreps_linear_info_backward is not None
               else input.shape[-2])
    return G.mix(input, weight, plan, in_size, anchor=irreps_linear_info_forward.M_MM0)


def irrep_wise_linear(input: Tensor, weight: Tensor, irreps_info):
    r"""``out[n, M, :] = input[n, M, :] @ weight[(n,) irrep_of(M)]`` (``IrrepWiseLinear.forward``, reference
    ``:494-526``): one channel-mixing matrix per irrep, the irreps themselves unchanged."""
    from . import _irreps_gemm as G
    plan = G.plan_of_irreps_info(irreps_info)
    return G.mix(input, weight, plan, plan.out_size, anchor=irreps_info.irrep_seg)


# ---- SO(2) linear maps are plain sparse products with the table of ``so2_linear_infos`` (reference :576-577) ----
from .sparse_product import sparse_mul as so2_linear_uu, sparse_vecmat as so2_linear_uv  # noqa: E402
