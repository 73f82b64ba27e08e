"""Radial basis and cutoff envelopes (plain tensor expressions, as in the reference) against what their definitions
fix: boundary values, vanishing derivatives, known points, orthogonality of the Bessel functions."""
import math

import torch

from equitorch_amd.nn.radials import BesselBasis
from equitorch_amd.nn.cutoffs import CosineCutoff, MollifierCutoff, PolynomialCutoff


def test_bessel_basis_values_and_orthogonality():
    basis = BesselBasis(r_max=4.0, num_basis=6, trainable=False).double()
    r = torch.tensor([0.5, 1.0, 2.0, 3.9], dtype=torch.float64)
    out = basis(r)
    n = torch.arange(1, 7, dtype=torch.float64)
    torch.testing.assert_close(out, 0.5 * torch.sin(n * math.pi * r[:, None] / 4.0) / r[:, None])
    # int_0^R b_n b_m r^2 dr = (2 / R) delta_nm for these functions (midpoint rule on a fine grid)
    grid = (torch.arange(20000, dtype=torch.float64) + 0.5) * (4.0 / 20000)
    b = basis(grid)
    gram = (b[:, :, None] * b[:, None, :] * grid[:, None, None] ** 2).sum(0) * (4.0 / 20000)
    torch.testing.assert_close(gram, 0.5 * torch.eye(6, dtype=torch.float64), atol=1e-6, rtol=0)
    assert isinstance(BesselBasis(4.0).bessel_weights, torch.nn.Parameter)


def test_cutoffs_boundary_behaviour():
    r = torch.tensor([0.0, 1.0, 2.5, 4.0, 5.0], dtype=torch.float64, requires_grad=True)
    poly = PolynomialCutoff(r_max=4.0, r_min=1.0, p=6)(r).detach()
    assert poly[0] == 1 and poly[1] == 1 and abs(float(poly[3])) < 1e-12 and poly[4] == 0
    u = torch.tensor(0.5, dtype=torch.float64)
    expect = 1 - 28 * u ** 6 + 48 * u ** 7 - 21 * u ** 8
    torch.testing.assert_close(poly[2], expect)
    # first and second derivative vanish at both ends of the interval
    x = torch.tensor([1.0 + 1e-9, 4.0 - 1e-9], dtype=torch.float64, requires_grad=True)
    y = PolynomialCutoff(4.0, 1.0, 6)(x)
    (g1,) = torch.autograd.grad(y.sum(), x, create_graph=True)
    (g2,) = torch.autograd.grad(g1.sum(), x)
    assert g1.abs().max() < 1e-6 and g2.abs().max() < 1e-5
    cos = CosineCutoff(r_max=4.0)(r.detach())
    torch.testing.assert_close(cos[:4], 0.5 * (1 + torch.cos(math.pi * r.detach()[:4] / 4.0)))
    assert cos[4] == 0
    mol = MollifierCutoff(r_max=4.0, eps=1e-7)(r.detach())
    assert abs(float(mol[0]) - 1) < 1e-6 and float(mol[3]) < 1e-12 and float(mol[2]) == math.exp(1 - 1 / (1 - 0.625 ** 2 + 1e-7))


def test_oracle_of_the_radial_functions_is_pinned_by_what_their_definitions_fix():
    """``oracle/ref_radial.py`` against values, zeros, derivatives and integrals that follow from the definitions."""
    from oracle import ref_radial as R
    f64 = torch.float64
    rmax = 3.5
    # Bessel: zeros at r_max, the n = 1 value at r_max / 2, orthogonality with weight r^2
    assert R.bessel(torch.tensor([rmax], dtype=f64), rmax, 6).abs().max() < 1e-14
    assert abs(float(R.bessel(torch.tensor([rmax / 2], dtype=f64), rmax, 1)) - 4 / rmax ** 2) < 1e-14
    grid = (torch.arange(20000, dtype=f64) + 0.5) * (rmax / 20000)
    b = R.bessel(grid, rmax, 5)
    gram = (b[:, :, None] * b[:, None, :] * grid[:, None, None] ** 2).sum(0) * (rmax / 20000)
    torch.testing.assert_close(gram, (2 / rmax) * torch.eye(5, dtype=f64), atol=1e-6, rtol=0)
    # polynomial envelope: boundary values, vanishing first and second derivatives at both ends, the p = 6 expansion
    for p in (2.0, 6.0, 9.0):
        u = torch.tensor([0.0, 1.0], dtype=f64, requires_grad=True)
        y = R.polynomial(u, p)
        assert y[0] == 1 and abs(float(y[1])) < 1e-12
        (g1,) = torch.autograd.grad(y.sum(), u, create_graph=True)
        assert g1.abs().max() < 1e-10
        if p > 2:          # at p = 2 the second derivative at 0 is -(p+1)(p+2)/2 * 2: the envelope's order condition
            (g2,) = torch.autograd.grad(g1.sum(), u)
            assert g2.abs().max() < 1e-9
    u = torch.tensor(0.37, dtype=f64)
    torch.testing.assert_close(R.polynomial(u, 6.0), 1 - 28 * u ** 6 + 48 * u ** 7 - 21 * u ** 8)
    torch.testing.assert_close(R.cosine(torch.tensor([0.0, 0.5, 1.0], dtype=f64)), torch.tensor([1.0, 0.5, 0.0], dtype=f64),
                               atol=1e-15, rtol=0)
    assert abs(float(R.mollifier(torch.tensor(0.5, dtype=f64), 0.0)) - math.exp(-1 / 3)) < 1e-15
    assert float(R.mollifier(torch.tensor(1.0, dtype=f64), 1e-12)) < 1e-300
    # the composition is constant outside [r_min, r_max]
    r = torch.tensor([0.0, 0.9, 1.0, 4.0, 4.1, 9.0], dtype=f64)
    for kind in ("polynomial", "cosine", "mollifier"):
        c = R.cutoff(kind, r, 4.0, 1.0)
        assert c[0] == c[1] == c[2] and c[3] == c[4] == c[5] and float(c[3]) < 1e-12 and abs(float(c[0]) - 1) < 1e-9
    # and the modules of the package (tensor expressions on the CPU) are the same functions
    r = torch.rand(50, dtype=f64) * 5
    basis = BesselBasis(4.0, 7, trainable=False).double()      # its frequencies are float32 values of n pi, as the reference's
    torch.testing.assert_close(basis(r + 0.1), R.bessel(r + 0.1, 4.0, 7, weights=basis.bessel_weights))
    torch.testing.assert_close(PolynomialCutoff(4.0, 1.0, 5)(r), R.cutoff("polynomial", r, 4.0, 1.0, 5.0))
    torch.testing.assert_close(CosineCutoff(4.0, 1.0)(r), R.cutoff("cosine", r, 4.0, 1.0))
    torch.testing.assert_close(MollifierCutoff(4.0, 1.0, 1e-7)(r), R.cutoff("mollifier", r, 4.0, 1.0, 1e-7))


def test_edge_operand_extents_are_checked_before_any_launch():
    """The fused edge kernels read P * C weights, D2 harmonics (or 3 vector components) and R radial features for
    every edge of the plan whatever the tensors hold, so a short operand has to be a Python error, not a read past
    the allocation.  The check runs on the host; no GPU is needed to see it refuse."""
    import types

    import pytest
    import torch
    from equitorch_amd import _lib
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn.functional import edge
    from equitorch_amd.utils._structs import tp_infos

    irreps = Irreps("0e+1o+2e")
    info = tp_infos(irreps, irreps, irreps)[0]
    n, e, c, r, p = 5, 12, 64, 8, 11
    plan = types.SimpleNamespace(num_edges=e, num_src_nodes=n, num_nodes=n)
    x, sh, vec = torch.zeros(n, 9, c), torch.zeros(e, 9), torch.zeros(e, 3)
    h, w_last, w = torch.zeros(e, r), torch.zeros(r, p, c), torch.zeros(e, p, c)
    edge._check_edge_operands(x, sh, plan, info, weight=w)
    edge._check_edge_operands(x, sh, plan, info, weight=w[0])
    edge._check_edge_operands(x, vec, plan, info, h=h, w_last=w_last, edge_vectors=True)
    bad = [dict(x=x[:4]), dict(x=x[:, :8]), dict(y=sh[:-1]), dict(y=sh[:, :8]), dict(weight=w[:-1]),
           dict(weight=w[:, :10]), dict(weight=w[..., :32]), dict(h=h[:-1], w_last=w_last, weight=None),
           dict(h=h, w_last=w_last[:-1], weight=None), dict(h=h, w_last=w_last[:, :10], weight=None),
           dict(h=h, w_last=w_last[..., :32], weight=None), dict(y=vec)]
    for change in bad:
        kw = dict(x=x, y=sh, weight=w, h=None, w_last=None)
        kw.update(change)
        with pytest.raises(_lib.CgtpError):
            edge._check_edge_operands(kw["x"], kw["y"], plan, info, weight=kw["weight"], h=kw["h"], w_last=kw["w_last"])
    with pytest.raises(_lib.CgtpError):
        edge._check_edge_operands(x, sh, plan, info, h=h, w_last=w_last, edge_vectors=True)
