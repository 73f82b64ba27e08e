"""Bessel basis and cutoff envelopes on one kernel each way (``cgtp_bessel`` / ``cgtp_bessel_grad`` / ``cgtp_cutoff``)
for fp32 / fp64 tensors on the GPU.  The reference writes them as tensor expressions (``equitorch/nn/radials.py:46-58``,
``equitorch/nn/functional/cutoffs.py:4-80``): six to ten launches each and as many again in the backward, over tensors
of a few MB — in a message-passing layer they were a fifth of the step.  Other dtypes and CPU tensors keep the
expressions; so does the gradient of the gradient (forces in the loss), which differentiates the expression."""
from typing import Callable

import torch
from torch import Tensor
from torch.autograd import Function

from ... import _lib

POLYNOMIAL, COSINE, MOLLIFIER = 0, 1, 2


def fused(*tensors: Tensor) -> bool:
    first = tensors[0]
    return (first.is_cuda and first.dtype in (torch.float32, torch.float64)
            and all(t.dtype == first.dtype and t.device == first.device for t in tensors[1:]))


class _Bessel(Function):
    @staticmethod
    def forward(ctx, r: Tensor, freq: Tensor, r_max: float, expression: Callable):
        r, freq = r.contiguous(), freq.contiguous()
        out = torch.empty(r.shape + freq.shape, dtype=r.dtype, device=r.device)
        _lib.check(_lib.lib.cgtp_bessel(r.data_ptr(), freq.data_ptr(), out.data_ptr(), r.numel(), freq.numel(), r_max,
                                        _lib.dtype_code(r.dtype), _lib.stream_ptr(r.device)), "cgtp_bessel")
        ctx.save_for_backward(r, freq)
        ctx.r_max, ctx.expression = r_max, expression
        return out

    @staticmethod
    def backward(ctx, g: Tensor):
        r, freq = ctx.saved_tensors
        need = ctx.needs_input_grad[:2]
        if torch.is_grad_enabled():
            with torch.enable_grad():
                inputs = [t for t, n in zip((r, freq), need) if n]
                grads = iter(torch.autograd.grad(ctx.expression(r, freq), inputs, g, create_graph=True))
            return tuple(next(grads) if n else None for n in need) + (None, None)
        g = g.contiguous()
        gr = torch.empty_like(r) if need[0] else None
        rows = torch.empty_like(g) if need[1] else None
        _lib.check(_lib.lib.cgtp_bessel_grad(r.data_ptr(), freq.data_ptr(), g.data_ptr(), _lib.ptr(gr), _lib.ptr(rows),
                                             r.numel(), freq.numel(), ctx.r_max, _lib.dtype_code(r.dtype),
                                             _lib.stream_ptr(r.device)), "cgtp_bessel_grad")
        gf = rows.reshape(-1, freq.numel()).sum(0) if need[1] else None
        return gr, gf, None, None


def bessel(r: Tensor, freq: Tensor, r_max: float, expression: Callable) -> Tensor:
    """``(2 / r_max) sin(freq r / r_max) / r`` with a trailing axis over ``freq``; ``expression(r, freq)``: the same as
    a tensor expression, differentiated when a gradient of higher order is asked for."""
    return _Bessel.apply(r, freq, float(r_max), expression)


class _Cutoff(Function):
    @staticmethod
    def forward(ctx, r: Tensor, kind: int, r_min: float, span: float, param: float, expression: Callable):
        r = r.contiguous()
        out = torch.empty_like(r)
        _lib.check(_lib.lib.cgtp_cutoff(kind, r.data_ptr(), 0, out.data_ptr(), r.numel(), r_min, span, param,
                                        _lib.dtype_code(r.dtype), _lib.stream_ptr(r.device)), "cgtp_cutoff")
        ctx.save_for_backward(r)
        ctx.args, ctx.expression = (kind, r_min, span, param), expression
        return out

    @staticmethod
    def backward(ctx, g: Tensor):
        (r,) = ctx.saved_tensors
        if not ctx.needs_input_grad[0]:
            return (None,) * 6
        if torch.is_grad_enabled():
            with torch.enable_grad():
                (gr,) = torch.autograd.grad(ctx.expression(r), (r,), g, create_graph=True)
            return (gr,) + (None,) * 5
        g = g.contiguous()
        gr = torch.empty_like(r)
        kind, r_min, span, param = ctx.args
        _lib.check(_lib.lib.cgtp_cutoff(kind, r.data_ptr(), g.data_ptr(), gr.data_ptr(), r.numel(), r_min, span, param,
                                        _lib.dtype_code(r.dtype), _lib.stream_ptr(r.device)), "cgtp_cutoff")
        return (gr,) + (None,) * 5


def cutoff(r: Tensor, kind: int, r_min: float, span: float, param: float, expression: Callable) -> Tensor:
    """Envelope ``kind`` of ``clamp((r - r_min) / span, 0, 1)``; ``param``: the order ``p`` (polynomial) or ``eps``
    (mollifier); ``expression(r)``: the same as a tensor expression."""
    return _Cutoff.apply(r, kind, float(r_min), float(span), float(param), expression)
