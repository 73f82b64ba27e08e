"""Rotations of equivariant features (``equitorch/nn/functional/wigner_d.py``).

A rotation with Euler angles ``(alpha, beta, gamma)`` acts as ``Z(alpha) J Z(beta) J Z(gamma)``: ``Z`` rotates about z
and only mixes the ``+-m`` pair of every irrep with ``cos(m a)``, ``sin(m a)`` (a table-driven vector-times-scalar
product, ``sparse_vecsca``), ``J`` is a constant sparse matrix (``sparse_scale``).  Every step is one launch of the
table-driven kernels of this library; no dense Wigner matrix is formed unless asked for."""
from typing import Optional

import torch
from torch import Tensor
from torch.autograd import Function

from ...ops import kernels
from ...structs import WignerRotationInfo
from .angular import sincos
from .sparse_product import sparse_vecsca
from .sparse_scale import sparse_scale
from .sphericals import xyz_to_spherical


def _z(x: Tensor, cs: Tensor, info: WignerRotationInfo) -> Tensor:
    return sparse_vecsca(x, cs, info.rotate_z_info_fwd, info.rotate_z_info_bwd_input, info.rotate_z_info_bwd_cs)


def _composed_rotation(input: Tensor, sincos_alpha, sincos_beta, sincos_gamma, info: WignerRotationInfo) -> Tensor:
    """The reference's five launches (``:14-56``); differentiable in every argument to any order."""
    x = input
    if sincos_gamma is not None:
        x = _z(x, sincos_gamma, info)
    if sincos_beta is not None:
        x = sparse_scale(x, info.j_matrix_info, info.j_matrix_info)      # J is symmetric: its own transpose
        x = _z(x, sincos_beta, info)
        x = sparse_scale(x, info.j_matrix_info, info.j_matrix_info)
    if sincos_alpha is not None:
        x = _z(x, sincos_alpha, info)
    return x


class _FusedRotation(Function):
    """One launch (``cgtp_wigner_rotate``).  The gradient of the features alone is the transposed rotation, again one
    launch; with gradients of the sincos tensors it is ``cgtp_wigner_rotate_backward``, which recomputes the
    intermediate features in registers.  Gradients of higher order go through the composition."""

    @staticmethod
    def forward(ctx, x: Tensor, sa, sb, sg, info: WignerRotationInfo, layout):
        ctx.save_for_backward(x, sa, sb, sg)
        ctx.info, ctx.layout = info, layout
        return kernels.wigner_rotate(x, sa, sb, sg, layout, transposed=False)

    @staticmethod
    def backward(ctx, g):
        x, sa, sb, sg = ctx.saved_tensors
        need_cs = [t is not None and ctx.needs_input_grad[1 + i] for i, t in enumerate((sa, sb, sg))]
        if torch.is_grad_enabled():          # a gradient of this gradient is wanted
            with torch.enable_grad():
                out = _composed_rotation(x, sa, sb, sg, ctx.info)
                wanted = [(i, t) for i, t in enumerate((x, sa, sb, sg)) if t is not None and ctx.needs_input_grad[i]]
                grads = torch.autograd.grad(out, [t for _, t in wanted], g, create_graph=True)
            res = [None] * 4
            for (i, _), gr in zip(wanted, grads):
                res[i] = gr
            return (*res, None, None)
        if not any(need_cs):                 # the transposed rotation; nothing to recompute
            return kernels.wigner_rotate(g.contiguous(), sa, sb, sg, ctx.layout, transposed=True), None, None, None, None, None
        gx, gcs = kernels.wigner_rotate_backward(x, g.contiguous(), (sa, sb, sg), ctx.layout, ctx.needs_input_grad[0],
                                                 need_cs)
        return (gx, *gcs, None, None)


def sparse_wigner_rotation(input: Tensor, sincos_alpha: Optional[Tensor], sincos_beta: Optional[Tensor],
                           sincos_gamma: Optional[Tensor], info: WignerRotationInfo) -> Tensor:
    """``D(alpha, beta, gamma) input`` for ``input (N, irreps.dim, C)`` and ``sincos_* (N, 1 + 2 max_m)`` (reference
    ``:14-56``); an angle given as ``None`` is zero and its factor is skipped.  fp32 / fp64 features with one sincos
    row per sample and irreps up to l = 6 take the fused kernels; other cases the composition."""
    cs = [t for t in (sincos_alpha, sincos_beta, sincos_gamma) if t is not None]
    if (cs and input.is_cuda and input.ndim == 3 and input.dtype in (torch.float32, torch.float64)
            and all(t.ndim == 2 and t.shape[0] == input.shape[0] and t.dtype == input.dtype
                    and t.shape[1] == cs[0].shape[1] for t in cs)):
        layout = kernels.rotation_layout(info)
        if (layout.ok and layout.dim == input.shape[1] and cs[0].shape[1] >= 1 + 2 * layout.max_degree
                and kernels.wigner_rotate_supported(layout, input.shape[2], input.dtype)):
            c = lambda t: None if t is None else t.contiguous()
            return _FusedRotation.apply(input.contiguous(), c(sincos_alpha), c(sincos_beta), c(sincos_gamma), info,
                                        layout)
    return _composed_rotation(input, sincos_alpha, sincos_beta, sincos_gamma, info)


def dense_wigner_rotation(input: Tensor, wigner_d: Tensor) -> Tensor:
    """``wigner_d @ input`` (reference ``:58-72``)."""
    return wigner_d @ input


def wigner_d_matrix(eye: Tensor, alpha: Optional[Tensor] = None, beta: Optional[Tensor] = None,
                    gamma: Optional[Tensor] = None, sincos_alpha: Optional[Tensor] = None,
                    sincos_beta: Optional[Tensor] = None, sincos_gamma: Optional[Tensor] = None,
                    info: Optional[WignerRotationInfo] = None) -> Tensor:
    """Dense ``D(alpha, beta, gamma)``: the sparse rotation applied to the identity, its columns playing the role of
    channels (reference ``:74-140``).  Angles ``(N,)`` or their ``sincos`` embeddings ``(N, 1 + 2 max_m)``; the result
    is ``(N, dim, dim)``, or ``(dim, dim)`` when no angle carries a batch of more than one."""
    assert info is not None
    sc = [s if s is not None or a is None else sincos(a, info.max_m)
          for s, a in ((sincos_alpha, alpha), (sincos_beta, beta), (sincos_gamma, gamma))]
    given = [s for s in sc if s is not None]
    dim = eye.shape[0]
    if dim == 0:
        return torch.empty((given[0].shape[0] if given else 1, 0, 0), device=eye.device, dtype=eye.dtype)
    n = max((s.shape[0] if s.ndim > 1 else 1 for s in given), default=1)
    sc = [None if s is None else s.reshape(-1, s.shape[-1]).expand(n, -1).contiguous() for s in sc]
    out = sparse_wigner_rotation(eye.unsqueeze(0).expand(n, -1, -1).contiguous(), *sc, info)
    batched = any(s is not None and s.ndim > 1 and s.shape[0] > 1 for s in given)
    return out if batched else out.squeeze(0)


def align_to_z_wigner_d(eye: Tensor, xyz: Tensor, max_m: int, info: WignerRotationInfo, normalized: bool = True,
                        eps: float = 1e-14) -> Tensor:
    """``D(0, -theta, -phi)`` for the polar angles ``(theta, phi)`` of every vector of ``xyz (N, 3)``: the rotation
    that takes the vector to the z axis (reference ``:142-204``).  ``normalized``: the vectors already have unit
    length."""
    theta, phi = xyz_to_spherical(xyz, normalize_input=not normalized, with_r=False, eps=eps, dim=-1)
    return wigner_d_matrix(eye=eye, sincos_beta=sincos(-theta, max_m), sincos_gamma=sincos(-phi, max_m), info=info)
