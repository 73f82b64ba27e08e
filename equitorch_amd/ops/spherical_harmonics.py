"""``spherical_harmonics`` (``equitorch/ops/spherical_harmonics.py:68-640``) on the HIP kernels ``cgtp_sh_forward`` /
``cgtp_sh_backward``: one kernel per direction instead of a TorchScript chain of tensor expressions."""
import torch
from torch import Tensor

from .. import _lib

MAX_DEGREE = 17


def _expression(xyz: Tensor, l_max: int, normalize: bool, scale: float) -> Tensor:
    """The same function as a tensor expression that autograd differentiates to any order (as the reference's
    TorchScript polynomials are, ``equitorch/ops/spherical_harmonics.py:68-640``): the Clebsch-Gordan recursion
    ``Y_l ~ C(l; l-1, 1) Y_(l-1) (x) Y_1``, whose degree-l block is the harmonic polynomial homogeneous of degree l."""
    from ..utils._sh import spherical_harmonics as recursion
    v = xyz / xyz.norm(dim=-1, keepdim=True).clamp_min(1e-12) if normalize else xyz
    out = recursion(v, l_max, dtype=xyz.dtype)
    return out if scale == 1.0 else out * scale


class _SphericalHarmonics(torch.autograd.Function):
    """``(n, 3) -> (n, (l_max+1)^2)``; optional fused normalisation of the input and overall scale."""

    @staticmethod
    def forward(ctx, xyz: Tensor, l_max: int, normalize: bool, scale: float):
        out = torch.empty(xyz.shape[0], (l_max + 1) ** 2, dtype=xyz.dtype, device=xyz.device)
        _lib.check(_lib.lib.cgtp_sh_forward(_lib.ptr(xyz), _lib.ptr(out), xyz.shape[0], l_max, int(normalize),
                                            float(scale), _lib.dtype_code(xyz.dtype), _lib.stream_ptr(xyz.device)),
                   "cgtp_sh_forward")
        ctx.save_for_backward(xyz)
        ctx.args = (l_max, normalize, scale)
        return out

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        (xyz,) = ctx.saved_tensors
        l_max, normalize, scale = ctx.args
        if torch.is_grad_enabled():   # a gradient of the gradient is wanted (forces in the loss): the tensor expression
            with torch.enable_grad():
                (grad,) = torch.autograd.grad(_expression(xyz, l_max, normalize, scale), (xyz,), grad_out,
                                              create_graph=True)
            return grad, None, None, None
        grad_out = grad_out.contiguous()
        grad = torch.empty_like(xyz)
        _lib.check(_lib.lib.cgtp_sh_backward(_lib.ptr(xyz), _lib.ptr(grad_out), _lib.ptr(grad), xyz.shape[0], l_max,
                                             int(normalize), float(scale), _lib.dtype_code(xyz.dtype),
                                             _lib.stream_ptr(xyz.device)), "cgtp_sh_backward")
        return grad, None, None, None


def spherical_harmonics(input: Tensor, l_max: int, dim: int = -1, normalize: bool = False,
                        scale: float = 1.0) -> Tensor:
    r"""Real spherical harmonics of degrees ``0..l_max`` of the 3-vectors stored along ``dim``.

    The result has ``(l_max+1)^2`` entries along ``dim``, index ``l^2 + l + m``; ``Y_1 = sqrt(3) (y, z, x)`` and
    ``|Y_l|^2 = 2l+1`` on the unit sphere.  Like the reference's polynomials the harmonics are homogeneous of
    degree ``l``: no normalisation of ``input`` is implied unless ``normalize`` is set, which applies
    ``input / max(|input|, 1e-12)`` inside the kernel.  ``scale`` multiplies the result.
    """
    if not 0 <= l_max <= MAX_DEGREE:
        raise ValueError(f"l_max must be in 0..{MAX_DEGREE}, got {l_max}")
    if input.shape[dim] != 3:
        raise ValueError(f"expected 3 components along dim {dim}, got shape {tuple(input.shape)}")
    _lib.require_gpu(input)
    if not input.dtype.is_floating_point:
        raise _lib.CgtpError(f"spherical_harmonics: unsupported dtype {input.dtype}")
    moved = input.movedim(dim, -1)
    flat = moved.reshape(-1, 3).contiguous()
    if flat.dtype in (torch.float32, torch.float64):
        out = _SphericalHarmonics.apply(flat, l_max, normalize, scale)
    else:   # half precisions: evaluated in fp32, rounded once
        out = _SphericalHarmonics.apply(flat.float(), l_max, normalize, scale).to(input.dtype)
    return out.reshape(*moved.shape[:-1], (l_max + 1) ** 2).movedim(-1, dim)
