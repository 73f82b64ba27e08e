"""Gradients of the gradient through the functions whose backward is a kernel of its own: the spherical harmonics and
the fused edge products.  With forces in the loss (``F = -dE/d positions`` computed with ``create_graph=True``) the
optimiser's backward differentiates those backward passes once more; the reference gets that for free from its
composition of differentiable functions (``equitorch/ops/spherical_harmonics.py:68-640`` is a tensor expression,
``equitorch/nn/functional/linears.py:18-83`` is closed under differentiation).  Here the backward, when it runs with
gradient mode on, evaluates the same result through functions autograd can differentiate again.  Checked against
finite differences (harmonics) and against the float64 dense oracle differentiated twice (edge products)."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_ops, ref_sh

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("l_max,normalize", [(3, True), (4, False), (1, True)])
def test_spherical_harmonics_differentiate_twice(device, l_max, normalize):
    from equitorch_amd.nn.functional import spherical_harmonics
    g = torch.Generator().manual_seed(l_max)
    v = (torch.randn(7, 3, generator=g, dtype=torch.float64) * 1.3).to(device).requires_grad_(True)
    fn = lambda t: spherical_harmonics(t, l_max, normalize_input=normalize)
    assert torch.autograd.gradcheck(fn, (v,), eps=1e-6, atol=1e-8)
    assert torch.autograd.gradgradcheck(fn, (v,), eps=1e-6, atol=1e-7)
    # the same against the oracle's harmonics, differentiated twice by autograd in float64 on the CPU
    ct, cf = torch.randn(7, (l_max + 1) ** 2, generator=g, dtype=torch.float64), torch.randn(7, 3, generator=g, dtype=torch.float64)
    vr = v.detach().cpu().requires_grad_(True)
    ref = ref_sh.spherical_harmonics(ref_sh.normalize(vr) if normalize else vr, l_max)
    (rf,) = torch.autograd.grad(ref, vr, ct, create_graph=True)
    (rgg,) = torch.autograd.grad((rf * cf).sum(), vr)
    (f,) = torch.autograd.grad(fn(v), v, ct.to(device), create_graph=True)
    (gg,) = torch.autograd.grad((f * cf.to(device)).sum(), v)
    assert_close(f, rf, 1e-12, f"harmonics l_max {l_max}: gradient under create_graph", norm="max")
    assert_close(gg, rgg, 1e-11, f"harmonics l_max {l_max}: gradient of the gradient", norm="max")


@pytest.mark.parametrize("use_shim", [True, False])
@pytest.mark.parametrize("mode,dtype", [("harmonics", torch.float64), ("vectors", torch.float64), ("vectors", torch.float32),
                                        ("radial", torch.float32), ("radial vectors", torch.float32)])
def test_forces_in_the_loss_through_the_fused_edge_products(device, monkeypatch, mode, dtype, use_shim):
    """``E = <out, ct>``, ``F = dE / d(second operand)`` under ``create_graph``, loss ``<F, cf> + <out, ct2>``: its
    gradient with respect to every operand against the dense oracle (gather, dense product, scatter-sum; harmonics of
    the oracle) differentiated the same way in float64.  fp32: norm-wise 1e-5 (sums over the edges of a node and over
    the paths).  Run through the C++ autograd node and through the Python Functions."""
    from equitorch_amd import _shim
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import (EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_radial,
                                             edge_tensor_product_uu_vectors)
    from equitorch_amd.ops import kernels
    if use_shim:
        assert _shim.module() is not None
    else:
        monkeypatch.setattr(_shim, "_module", None)
    irreps, l_max, ch, n_nodes, n_edges, R = "0e+1o+2e", 2, 64, 40, 500, 8
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    P = mod.num_paths
    gen = torch.Generator().manual_seed(len(mode) + 10 * use_shim)
    src, dst = torch.randint(0, n_nodes, (n_edges,), generator=gen), torch.randint(0, n_nodes, (n_edges,), generator=gen)
    rd = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64).to(dtype).double()
    x, ct, ct2 = rd(n_nodes, 9, ch), rd(n_nodes, 9, ch), rd(n_nodes, 9, ch)
    vectors, radial = "vectors" in mode, "radial" in mode
    second = rd(n_edges, 3) * 1.2 if vectors else rd(n_edges, 9)
    cf = rd(*second.shape)
    weights = (rd(n_edges, R), rd(R, P, ch) / R ** 0.5) if radial else (rd(n_edges, P, ch),)
    T = ref_ops.dense_coupling(irreps, irreps, irreps).float().double()

    def reference(x, second, *weights):      # in the precision of its operands
        sh = ref_sh.spherical_harmonics(ref_sh.normalize(second), l_max) if vectors else second
        w = (weights[0] @ weights[1].reshape(R, -1)).view(n_edges, P, ch) if radial else weights[0]
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w, dtype=x.dtype), dst, n_nodes)

    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))

    def product(x, second, *weights):
        if radial:
            return edge_tensor_product_uu_radial(x, second, *weights, plan, mod.tp_info_forward, edge_vectors=vectors)
        if vectors:
            return edge_tensor_product_uu_vectors(x, second, *weights, plan, mod.tp_info_forward)
        return edge_tensor_product_uu(x, second, *weights, plan, mod.tp_info_forward)

    def twice(fn, inputs, cts):
        ct, cf, ct2 = cts
        out = fn(*inputs)
        (force,) = torch.autograd.grad(out, inputs[1], ct, create_graph=True)
        return out, force, torch.autograd.grad((force * cf).sum() + (out * ct2).sum(), inputs)

    ref_in = [t.clone().requires_grad_(True) for t in (x, second, *weights)]
    ref_out, ref_force, ref_gg = twice(reference, ref_in, (ct, cf, ct2))
    dev_in = [t.to(device, dtype).requires_grad_(True) for t in (x, second, *weights)]
    out, force, gg = twice(product, dev_in, [t.to(device, dtype) for t in (ct, cf, ct2)])
    if radial:
        assert "fused gather / weights / product / segment sum" in seen[0], seen
    elif not vectors:
        assert "fused gather / product / segment sum" in seen[0], seen
    assert ("Cpp" in type(out.grad_fn).__name__) == (use_shim and not radial), type(out.grad_fn).__name__
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    # fp32: the same computation restated in fp32 arithmetic beside every norm-wise comparison
    r32 = (None, None, (None,) * len(ref_gg))
    if dtype == torch.float32:
        r32 = twice(reference, [t.float().requires_grad_(True) for t in (x, second, *weights)],
                    [t.float() for t in (ct, cf, ct2)])
    assert_close(out, ref_out, tol, f"{mode}: out", norm="max", fp32_ref=r32[0])
    assert_close(force, ref_force, tol, f"{mode}: gradient under create_graph", norm="max", fp32_ref=r32[1])
    names = ("x", "second operand", "h", "w_last") if radial else ("x", "second operand", "w")
    for name, a, b, b32 in zip(names, gg, ref_gg, r32[2]):
        assert_close(a, b, tol, f"{mode}: d loss / d {name} with the force in the loss", norm="max", fp32_ref=b32)


@pytest.mark.parametrize("case", ["shared weight", "table that is not compiled in", "row kernels + segment sums"])
def test_forces_in_the_loss_on_the_other_routes_of_the_edge_product(device, monkeypatch, case):
    """The same check where ``edge_tensor_product_uu`` takes another route: a shared weight (its gradient is a sum over
    the edges), a table without compiled kernels (table-driven fused kernels) and a table whose fused kernels do not
    take 128 channels (row kernels followed by segment sums)."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    io, i1, i2, ch, dtype, want = {
        "shared weight": ("0e+1o+2e", "0e+1o+2e", "0e+1o+2e", 64, torch.float64, "fused gather / product / segment sum"),
        "table that is not compiled in": ("1o+2e+1e", "0e+1o+2e", "0e+1o", 32, torch.float32, "table-driven fused"),
        "row kernels + segment sums": ("0e+1o+2e+3o+4e",) * 3 + (128, torch.float32, "block-wise row kernels"),
    }[case]
    n_nodes, n_edges = 30, 300
    mod = SO3Linear(i1, i2, io, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    gen = torch.Generator().manual_seed(len(case))
    src, dst = torch.randint(0, n_nodes, (n_edges,), generator=gen), torch.randint(0, n_nodes, (n_edges,), generator=gen)
    rd = lambda *s: torch.randn(*s, generator=gen, dtype=torch.float64).to(dtype).double()
    d1, d2, do = Irreps(i1).dim, Irreps(i2).dim, Irreps(io).dim
    x, sh, ct, ct2, cf = rd(n_nodes, d1, ch), rd(n_edges, d2), rd(n_nodes, do, ch), rd(n_nodes, do, ch), rd(n_edges, d2)
    w = rd(mod.num_paths, ch) if case == "shared weight" else rd(n_edges, mod.num_paths, ch)
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))

    def twice(fn, inputs, cts):
        ct, cf, ct2 = cts
        out = fn(*inputs)
        (force,) = torch.autograd.grad(out, inputs[1], ct, create_graph=True)
        return out, force, torch.autograd.grad((force * cf).sum() + (out * ct2).sum(), inputs)

    reference = lambda x, sh, w: ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w, dtype=x.dtype),
                                                     dst, n_nodes)
    ref = twice(reference, [t.clone().requires_grad_(True) for t in (x, sh, w)], (ct, cf, ct2))
    r32 = (None, None, (None,) * 3)
    if dtype == torch.float32:
        r32 = twice(reference, [t.float().requires_grad_(True) for t in (x, sh, w)], [t.float() for t in (ct, cf, ct2)])
    got = twice(lambda x, sh, w: edge_tensor_product_uu(x, sh, w, plan, mod.tp_info_forward),
                [t.to(device, dtype).requires_grad_(True) for t in (x, sh, w)], [t.to(device, dtype) for t in (ct, cf, ct2)])
    assert want in seen[0], seen
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    assert_close(got[0], ref[0], tol, f"{case}: out", norm="max", fp32_ref=r32[0])
    assert_close(got[1], ref[1], tol, f"{case}: gradient under create_graph", norm="max", fp32_ref=r32[1])
    for name, a, b, b32 in zip(("x", "harmonics", "w"), got[2], ref[2], r32[2]):
        assert_close(a, b, tol, f"{case}: d loss / d {name} with the force in the loss", norm="max", fp32_ref=b32)
