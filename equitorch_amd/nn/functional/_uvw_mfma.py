"""Dispatch of the fully connected ("uv") product to the bf16 matrix-core kernel (``cgtp_uv_apply``)."""
import ctypes as C
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib
from ...ops import kernels
from ._tri import spec_from_tp_info, tri


uv_config_of = kernels.uv_config_of


def pack_weights(direction: int, w: Tensor, cfg) -> Tensor:
    """W as stored by the module, (P, C_in, C_out), rewritten in the fragment order the kernel reads, with the
    per-path factors of ``cfg`` folded in (fp32 product, rounded to bf16 once).  Packed anew on every call: one small
    launch, and no cached copy that an in-place update through ``w.data`` could leave stale."""
    w = kernels.expand_paths(w, cfg, 0).contiguous()
    cin, cout = (w.shape[1], w.shape[2]) if direction == 0 else (w.shape[2], w.shape[1])
    packed = torch.empty_like(w)
    scale = cfg.scale_tensor(torch.float32, w.device) if isinstance(cfg, kernels.Cfg) else None
    _lib.check(_lib.lib.cgtp_uv_pack_weights(direction, w.data_ptr(), packed.data_ptr(), w.shape[0], cin, cout,
                                             _lib.BF16, _lib.ptr(scale), _lib.stream_ptr(w.device)),
               "cgtp_uv_pack_weights")
    return packed


def _apply(cfg: int, direction: int, x: Tensor, y: Tensor, wp: Tensor, d_out: int) -> Tensor:
    """``wp`` = ``pack_weights(direction, W)``."""
    n, _, cin = x.shape
    cout = wp.numel() // (wp.shape[0] * cin)
    out = torch.empty((n, d_out, cout), dtype=x.dtype, device=x.device)
    _lib.check(_lib.lib.cgtp_uv_apply(cfg, direction, x.data_ptr(), y.data_ptr(), wp.data_ptr(), out.data_ptr(), n,
                                      cin, cout, _lib.BF16, _lib.stream_ptr(x.device)), "cgtp_uv_apply")
    return out


def _grad_y(cfg: int, x: Tensor, g: Tensor, wp: Tensor, d2: int) -> Tensor:
    """Gradient w.r.t. the harmonics; ``wp`` = ``pack_weights(0, W)``."""
    n, _, cin = x.shape
    cout = g.shape[-1]
    gy = torch.empty((n, d2), dtype=x.dtype, device=x.device)
    _lib.check(_lib.lib.cgtp_uv_grad_y(cfg, x.data_ptr(), g.data_ptr(), wp.data_ptr(), gy.data_ptr(), n, cin, cout,
                                       _lib.BF16, _lib.stream_ptr(x.device)), "cgtp_uv_grad_y")
    return gy


def _grad_w(cfg: int, x: Tensor, y: Tensor, g: Tensor) -> Tensor:
    """Gradient w.r.t. the shared weight, (P, C_in, C_out) over the caller's own paths."""
    n, _, cin = x.shape
    cout = g.shape[-1]
    n_paths = kernels._compiled_tables("uv")[int(cfg)][0][3]
    gw = torch.empty((n_paths, cin, cout), dtype=x.dtype, device=x.device)
    scale = cfg.scale_tensor(torch.float32, x.device) if isinstance(cfg, kernels.Cfg) else None
    ws_bytes = int(_lib.lib.cgtp_uv_grad_w_workspace_bytes(cfg, n, cin, cout))
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=x.device)
    _lib.check(_lib.lib.cgtp_uv_grad_w(cfg, x.data_ptr(), y.data_ptr(), g.data_ptr(), gw.data_ptr(), ws.data_ptr(), n,
                                       cin, cout, _lib.BF16, _lib.ptr(scale), _lib.stream_ptr(x.device)),
               "cgtp_uv_grad_w")
    return kernels.contract_paths(gw, cfg, 0)


class _UvMfma(Function):
    """u1v with a shared weight on the matrix cores: forward and the three first-order gradients.  Under
    ``create_graph`` the gradients are formed by the general contraction kernel, which is differentiable again."""

    @staticmethod
    def forward(ctx, x: Tensor, y: Tensor, w: Tensor, tp_info, cfg: int):
        coo = kernels.coo_of(tp_info)
        out = _apply(cfg, 0, x, y, pack_weights(0, w, cfg), coo.DO)
        ctx.save_for_backward(x, y, w)
        ctx.tp_info, ctx.cfg, ctx.d1 = tp_info, cfg, coo.D1
        return out

    @staticmethod
    def backward(ctx, g):
        x, y, w = ctx.saved_tensors
        need = ctx.needs_input_grad
        spec = spec_from_tp_info(ctx.tp_info)
        gx = gy = gw = None
        with torch.enable_grad() if torch.is_grad_enabled() else torch.no_grad():
            if need[0]:
                if torch.is_grad_enabled():
                    gx = tri(spec.grad_spec(0), ("w", "", "uw"), "u", g, y, w)
                else:
                    gx = _apply(ctx.cfg, 1, g.contiguous(), y, pack_weights(1, w, ctx.cfg), ctx.d1)
            if need[1]:
                if torch.is_grad_enabled() or g.shape[-1] > 128:
                    gy = tri(spec.grad_spec(1), ("u", "w", "uw"), "", x, g, w)
                else:
                    gy = _grad_y(ctx.cfg, x, g.contiguous(), pack_weights(0, w, ctx.cfg), y.shape[-1])
            if need[2]:
                if torch.is_grad_enabled():
                    gw = tri(spec.grad_spec(2), ("u", "", "w"), "uw", x, y, g, out_shared=True)
                else:
                    gw = _grad_w(ctx.cfg, x, y, g.contiguous())
        return gx, gy, gw, None, None


def try_forward(input1: Tensor, input2: Tensor, weight: Tensor, tp_info) -> Optional[Tensor]:
    """The product on the MFMA kernel, or None if the operands are outside its domain (bf16, shared weight,
    C_in in {32, 64, 128} both ways, C_out a multiple of 32, table compiled in, input rows fit in LDS)."""
    if not (input1.dtype == input2.dtype == weight.dtype == torch.bfloat16):
        return None
    if input1.ndim != 3 or input2.ndim != 2 or weight.ndim != 3 or input1.shape[0] == 0:
        return None
    cin, cout = weight.shape[-2:]
    if cin not in (32, 64, 128) or cout not in (32, 64, 128):
        return None
    cfg = uv_config_of(tp_info)
    if cfg < 0:
        return None
    x, y = input1.contiguous(), input2.contiguous()
    dummy = 256
    for direction, (ci, co) in enumerate(((cin, cout), (cout, cin))):
        if _lib.lib.cgtp_uv_validate(cfg, direction, dummy, dummy, dummy, dummy, x.shape[0], ci, co, _lib.BF16) != 0:
            return None
    return _UvMfma.apply(x, y, weight, tp_info, cfg)
