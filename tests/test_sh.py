"""The spherical-harmonics oracle pinned on the CPU against what the reference's polynomial text fixes
(equitorch/ops/spherical_harmonics.py:80-640) and against textbook closed forms."""
import math

import numpy as np
import torch

from oracle import ref_sh


def _vectors(n, seed=0, unit=True):
    g = torch.Generator().manual_seed(seed)
    v = torch.randn(n, 3, generator=g, dtype=torch.float64)
    return v / v.norm(dim=-1, keepdim=True) if unit else v


def test_degrees_up_to_three_are_the_reference_polynomials():
    """Lines :80-114 expanded by hand: the familiar real harmonics with all leading signs positive."""
    v = _vectors(40, unit=False)
    x, y, z = v.unbind(-1)
    s = math.sqrt
    expect = torch.stack([
        torch.ones_like(x),
        s(3) * y, s(3) * z, s(3) * x,
        s(15) * x * y, s(15) * y * z, s(5) / 2 * (2 * z * z - x * x - y * y), s(15) * x * z,
        s(15) / 2 * (x * x - y * y),
        s(70) / 4 * y * (3 * x * x - y * y), s(105) * x * y * z, s(42) / 4 * y * (4 * z * z - x * x - y * y),
        s(7) / 2 * z * (2 * z * z - 3 * x * x - 3 * y * y), s(42) / 4 * x * (4 * z * z - x * x - y * y),
        s(105) / 2 * z * (x * x - y * y), s(70) / 4 * x * (x * x - 3 * y * y)], dim=-1)
    torch.testing.assert_close(ref_sh.spherical_harmonics(v, 3), expect, rtol=1e-12, atol=1e-12)


def test_matches_textbook_closed_form_for_every_l_m():
    u = _vectors(64, seed=1)
    y = ref_sh.spherical_harmonics(u, 12).numpy()
    np.testing.assert_allclose(y, ref_sh.closed_form(u.numpy(), 12), rtol=0, atol=2e-12)


def test_north_pole_and_sectoral_recursion():
    """sh_l_l(0,0,1) = +sqrt(2l+1); the sh_l_0 / sh_l_{2l} lines of every degree:
    Y_{l,-l} = c (x Y_{l-1,-(l-1)} + y Y_{l-1,l-1}),  Y_{l,l} = c (x Y_{l-1,l-1} - y Y_{l-1,-(l-1)}),  c = sqrt((2l+1)/(2l))."""
    L = 17
    pole = torch.tensor([[0.0, 0.0, 1.0]], dtype=torch.float64)
    yp = ref_sh.spherical_harmonics(pole, L)[0]
    v = _vectors(16, seed=2, unit=False)
    x, y, _ = v.unbind(-1)
    Y = ref_sh.spherical_harmonics(v, L)
    for l in range(L + 1):
        blk = yp[l * l:(l + 1) ** 2]
        assert abs(float(blk[l]) - math.sqrt(2 * l + 1)) < 1e-11 and float(blk.abs().sum() - blk[l].abs()) < 1e-11
        if l >= 2:
            c = math.sqrt((2 * l + 1) / (2 * l))
            lo, hi = Y[:, (l - 1) ** 2], Y[:, l * l - 1]
            torch.testing.assert_close(Y[:, l * l], c * (x * lo + y * hi), rtol=1e-11, atol=1e-11)
            torch.testing.assert_close(Y[:, (l + 1) ** 2 - 1], c * (x * hi - y * lo), rtol=1e-11, atol=1e-11)


def test_norm_addition_theorem_and_homogeneity():
    L = 9
    a, b = _vectors(30, seed=3), _vectors(30, seed=4)
    ya, yb = ref_sh.spherical_harmonics(a, L), ref_sh.spherical_harmonics(b, L)
    cos = (a * b).sum(-1).numpy()
    raw = _vectors(30, seed=3, unit=False)
    r = raw.norm(dim=-1)
    yr = ref_sh.spherical_harmonics(raw, L)
    for l in range(L + 1):
        s = slice(l * l, (l + 1) ** 2)
        torch.testing.assert_close((ya[:, s] ** 2).sum(-1), torch.full((30,), 2.0 * l + 1, dtype=torch.float64))
        pl = np.polynomial.legendre.legval(cos, [0] * l + [1])
        np.testing.assert_allclose((ya[:, s] * yb[:, s]).sum(-1).numpy(), (2 * l + 1) * pl, atol=1e-11)
        torch.testing.assert_close(yr[:, s], ya[:, s] * r[:, None] ** l, rtol=1e-11, atol=1e-11)


def test_gradient_oracle_against_central_differences():
    v = _vectors(6, seed=5, unit=False).requires_grad_(True)
    ct = torch.randn(6, 25, generator=torch.Generator().manual_seed(6), dtype=torch.float64)
    (ref_sh.spherical_harmonics(ref_sh.normalize(v), 4) * ct).sum().backward()
    h = 1e-6
    for k in range(3):
        d = torch.zeros(3, dtype=torch.float64)
        d[k] = h
        f = lambda w: (ref_sh.spherical_harmonics(ref_sh.normalize(w), 4) * ct).sum(-1)
        fd = (f(v.detach() + d) - f(v.detach() - d)) / (2 * h)
        torch.testing.assert_close(v.grad[:, k], fd, rtol=1e-7, atol=1e-7)
