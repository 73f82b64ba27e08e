"""GPU parity of the radial basis and cutoff kernels (``cgtp_bessel``, ``cgtp_bessel_grad``, ``cgtp_cutoff``) behind
``BesselBasis`` and the cutoff modules, against ``oracle/ref_radial.py`` (float64): values, gradients with respect to
the edge length and the trainable frequencies, shapes with leading axes, the clamped ends, and the gradient of the
gradient (which differentiates the tensor expression).

Tolerances: fp64 1e-12, fp32 1e-5 element-wise (``|a - b| <= tol (1 + |b|)``) on edge lengths in [0.2, 1.2 r_max]; the
gradient with respect to a frequency sums 3000 edges and is compared norm-wise with its fp32 restatement alongside."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_radial

pytestmark = pytest.mark.gpu


@pytest.fixture
def device():
    return torch.device("cuda:0")


def _lengths(n, r_max, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return (torch.rand(n, generator=g, dtype=torch.float64) * (1.2 * r_max - 0.2) + 0.2).to(dtype)


@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-12), (torch.float32, 1e-5)])
@pytest.mark.parametrize("trainable", [False, True])
def test_bessel_basis(device, dtype, tol, trainable):
    from equitorch_amd.nn import BesselBasis
    r_max, nb = 3.5, 8
    mod = BesselBasis(r_max, nb, trainable=trainable).to(device=device, dtype=dtype)
    r = _lengths(3000, r_max, 1, dtype)
    ct = torch.randn(3000, nb, generator=torch.Generator().manual_seed(2), dtype=torch.float64).to(dtype)
    rd = r.to(device).requires_grad_(True)
    out = mod(rd)
    assert out.shape == (3000, nb) and type(out.grad_fn).__name__ == "_BesselBackward"
    wrt = [rd] + ([mod.bessel_weights] if trainable else [])
    grads = torch.autograd.grad(out, wrt, ct.to(device))
    w64 = mod.bessel_weights.detach().double().cpu().requires_grad_(True)
    r64 = r.double().requires_grad_(True)
    ref = ref_radial.bessel(r64, r_max, nb, weights=w64)
    ref_g = torch.autograd.grad(ref, [r64, w64], ct.double())
    assert_close(out, ref.detach(), tol, f"bessel {dtype} values")
    assert_close(grads[0], ref_g[0], tol * 10, f"bessel {dtype} grad r")      # a sum of 8 terms of either sign
    if trainable:
        r32, w32 = r.float().requires_grad_(True), mod.bessel_weights.detach().float().cpu().requires_grad_(True)
        g32 = torch.autograd.grad(ref_radial.bessel(r32, r_max, nb, weights=w32), [w32], ct.float())[0]
        assert_close(grads[1], ref_g[1], tol, f"bessel {dtype} grad frequencies (sum over 3000 edges)", norm="max",
                     fp32_ref=g32 if dtype == torch.float32 else None)
    # leading axes are kept, an empty tensor is an empty result
    assert mod(rd.detach().view(30, 100)).shape == (30, 100, nb)
    torch.testing.assert_close(mod(rd.detach().view(30, 100)).view(3000, nb), out.detach())
    assert mod(rd.detach()[:0]).shape == (0, nb)


@pytest.mark.parametrize("dtype,tol", [(torch.float64, 1e-12), (torch.float32, 1e-5)])
@pytest.mark.parametrize("kind,make,param", [
    ("polynomial", lambda nn: nn.PolynomialCutoff(4.0, 1.0, 6), 6.0),
    ("polynomial", lambda nn: nn.PolynomialCutoff(4.0, 0.0, 3), 3.0),
    ("cosine", lambda nn: nn.CosineCutoff(4.0, 1.0), None),
    ("mollifier", lambda nn: nn.MollifierCutoff(4.0, 0.5, 1e-7), 1e-7),
])
def test_cutoffs(device, dtype, tol, kind, make, param):
    from equitorch_amd import nn as enn
    mod = make(enn)
    r = torch.cat([_lengths(2000, 4.0, 3, dtype), torch.tensor([0.0, mod.r_min, 4.0, 7.0], dtype=dtype)])
    ct = torch.randn(r.shape[0], generator=torch.Generator().manual_seed(4), dtype=torch.float64).to(dtype)
    rd = r.to(device).requires_grad_(True)
    out = mod(rd)
    assert type(out.grad_fn).__name__ == "_CutoffBackward"
    (gr,) = torch.autograd.grad(out, rd, ct.to(device))
    r64 = r.double().requires_grad_(True)
    ref = ref_radial.cutoff(kind, r64, 4.0, mod.r_min, param)
    (ref_g,) = torch.autograd.grad(ref, r64, ct.double())
    assert_close(out, ref.detach(), tol, f"{kind} cutoff {dtype} values")
    # the mollifier's slope grows like 1 / (1 - u^2)^2 towards r_max: compare where the envelope is not yet negligible
    keep = (ref.detach() > 1e-6) | (ref_g == 0)
    assert_close(gr.cpu()[keep], ref_g[keep], tol * 10, f"{kind} cutoff {dtype} grad r")
    assert float(out.detach()[-1]) == 0 or kind == "mollifier" and float(out.detach()[-1]) < 1e-30
    assert float(gr[-1]) == 0 and float(gr[-4]) == 0 or mod.r_min == 0          # outside the interval: no slope


def test_gradient_of_the_gradient_and_other_dtypes(device):
    """Forces in the loss differentiate the radial functions twice: the backward under ``create_graph`` evaluates the
    tensor expression, so ``gradgradcheck`` holds; bf16 tensors keep the tensor expressions altogether."""
    from equitorch_amd import nn as enn
    basis = enn.BesselBasis(3.0, 4, trainable=True).to(device).double()
    cut = enn.PolynomialCutoff(3.0, 0.5, 5)
    r = _lengths(6, 2.4, 5, torch.float64).to(device).requires_grad_(True)
    from equitorch_amd.nn.functional import _radial
    fn = lambda x, w: _radial.bessel(x, w, 3.0, basis._expression) * cut(x)[:, None]
    assert torch.autograd.gradcheck(fn, (r, basis.bessel_weights), eps=1e-6, atol=1e-7)
    assert torch.autograd.gradgradcheck(fn, (r, basis.bessel_weights), eps=1e-6, atol=1e-6)
    half = enn.BesselBasis(3.0, 4).to(device).bfloat16()
    out = half(r.detach().bfloat16())
    assert out.dtype == torch.bfloat16 and "Bessel" not in type(out.grad_fn).__name__
