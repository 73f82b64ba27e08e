"""GPU parity of the edge product whose per-edge weights are formed inside the kernels from per-edge features and a
shared matrix (``edge_tensor_product_uu_radial``, ``cgtp_uvu_radial_grad``): output and all gradients against the
dense float64 oracle with the weights formed by an explicit einsum (``W[e] = h[e] @ w_last``), gathered at src and
summed at dst."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_ops, ref_sh

pytestmark = pytest.mark.gpu

SH = {l: "+".join(f"{k}{'e' if k % 2 == 0 else 'o'}" for k in range(l + 1)) for l in range(5)}


def _case(lmax, n_nodes, n_edges, r, seed, hub=False):
    g = torch.Generator().manual_seed(seed)
    d = (lmax + 1) ** 2
    src = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst[dst == 3] = 4                                           # an empty segment
    if hub:
        dst[50:400] = 11
        src[200:500] = 2
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).float().double()
    return src, dst, rd(n_nodes, d, 64), rd(n_edges, r), rd(n_nodes, d, 64), rd, g


@pytest.mark.parametrize("lmax,r,vectors,hub", [(2, 16, False, False), (2, 8, False, True), (2, 16, True, False),
                                                (2, 4, True, True), (1, 12, False, False), (1, 16, True, True)])
def test_edge_product_with_weights_formed_in_the_kernel(device, lmax, r, vectors, hub):
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu_radial
    from equitorch_amd.ops import kernels
    n_nodes, n_edges = 70, 1303
    irr = SH[lmax]
    mod = SO3Linear(irr, irr, irr, internal_weights=False, feature_mode="uu").to(device)
    src, dst, x, h, ct, rd, g = _case(lmax, n_nodes, n_edges, r, 300 + 10 * lmax + r, hub)
    w_last = rd(r, mod.num_paths, 64) / r ** 0.5
    d2 = (lmax + 1) ** 2
    y = (rd(n_edges, 3) * (0.5 + torch.rand(n_edges, 1, generator=g, dtype=torch.float64))).float().double() if vectors \
        else rd(n_edges, d2)
    T = ref_ops.dense_coupling(irr, irr, irr)

    def oracle(dt):     # (out, grad_x, grad_y, grad_h, grad_w_last) in ``dt``: float64 the arbiter, float32 the yardstick
        xr, yr, hr, wr = (t.detach().to(dt).clone().requires_grad_(True) for t in (x, y, h, w_last))
        sh = ref_sh.spherical_harmonics(ref_sh.normalize(yr), lmax) if vectors else yr
        weights = torch.einsum("er,rpc->epc", hr, wr)
        ref = ref_ops.scatter_sum(ref_ops.dense_u1u(T, xr[src], sh, weights, dtype=dt), dst, n_nodes)
        (ref * ct.to(dt)).sum().backward()
        return ref.detach(), xr.grad, yr.grad, hr.grad, wr.grad
    want, want32 = oracle(torch.float64), oracle(torch.float32)

    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, yd, hd, wd = (t.to(device, torch.float32).requires_grad_(True) for t in (x, y, h, w_last))
    assert kernels.uvu_radial_supported(kernels.uvu_config_of(mod.tp_info_forward), xd, hd, wd)
    out = edge_tensor_product_uu_radial(xd, yd, hd, wd, plan, mod.tp_info_forward, edge_vectors=vectors)
    (out * ct.to(device, torch.float32)).sum().backward()
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_h", "grad_w_last"),
                               (out, xd.grad, yd.grad, hd.grad, wd.grad), want, want32):
        # grad_h sums over all paths and channels, grad_w_last over all edges, grad of vectors through the harmonics:
        # norm-wise, and within three times what the same computation loses in fp32
        long_sum = name in ("grad_h", "grad_w_last") or (vectors and name == "grad_y")
        assert_close(a, b, tol=1e-5, what=f"radial lmax={lmax} R={r} vec={vectors} {name}",
                     norm="max" if long_sum else "element", fp32_ref=b32)


def test_radial_with_other_normalisation_and_fallback(device):
    """A table that differs from the compiled one by per-path factors (path_norm off) keeps the fused kernels (the
    factors are folded into the shared matrix); shapes the fused kernels do not take (R = 6) give the same numbers
    through the plain functions."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu_radial
    n_nodes, n_edges, lmax = 40, 500, 2
    irr = SH[lmax]
    mod = SO3Linear(irr, irr, irr, internal_weights=False, feature_mode="uu", path_norm=False).to(device)
    T = ref_ops.dense_coupling(irr, irr, irr, path_norm=False)
    for r in (8, 6):
        src, dst, x, h, ct, rd, g = _case(lmax, n_nodes, n_edges, r, 77 + r)
        w_last, y = rd(r, mod.num_paths, 64) / r ** 0.5, rd(n_edges, 9)
        def oracle(dt):
            xr, yr, hr, wr = (t.detach().to(dt).clone().requires_grad_(True) for t in (x, y, h, w_last))
            ref = ref_ops.scatter_sum(ref_ops.dense_u1u(T, xr[src], yr, torch.einsum("er,rpc->epc", hr, wr), dtype=dt),
                                      dst, n_nodes)
            (ref * ct.to(dt)).sum().backward()
            return ref.detach(), xr.grad, yr.grad, hr.grad, wr.grad
        want, want32 = oracle(torch.float64), oracle(torch.float32)
        plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
        xd, yd, hd, wd = (t.to(device, torch.float32).requires_grad_(True) for t in (x, y, h, w_last))
        out = edge_tensor_product_uu_radial(xd, yd, hd, wd, plan, mod.tp_info_forward)
        (out * ct.to(device, torch.float32)).sum().backward()
        for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_h", "grad_w_last"),
                                   (out, xd.grad, yd.grad, hd.grad, wd.grad), want, want32):
            assert_close(a, b, tol=1e-5, what=f"radial path_norm=False R={r} {name}",
                         norm="max" if name in ("grad_h", "grad_w_last") else "element", fp32_ref=b32)


def test_weights_formed_in_the_kernel_at_3_2_million_edges(device):
    """3.2 million edges (the weight tensor that is never formed would have 2.25e9 elements; the per-edge weight
    gradient, which is written, has): harmonics and weights both produced inside the edge kernels, all five gradients,
    against the composition harmonics kernel -> matrix product -> plain fused edge product.  1e-4 of each tensor's
    scale (sums over 32 to 3.2 million terms in different orders)."""
    from equitorch_amd.nn import SO3Linear, SphericalHarmonics
    from equitorch_amd.nn.functional import (EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_radial)
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 60 GB of device memory")
    irreps, ch, n_nodes, n_edges, r = "0e+1o+2e", 64, 100_000, 3_200_000, 16
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    g = torch.Generator(device=device).manual_seed(7)
    src = torch.randint(0, n_nodes, (n_edges,), generator=g, device=device)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g, device=device)
    plan = EdgePlan(src, dst, n_nodes)
    x = torch.randn(n_nodes, 9, ch, generator=g, device=device).requires_grad_(True)
    vec = torch.randn(n_edges, 3, generator=g, device=device).requires_grad_(True)
    h = torch.randn(n_edges, r, generator=g, device=device).requires_grad_(True)
    wl = (torch.randn(r, 11, ch, generator=g, device=device) / 4).requires_grad_(True)
    ct = torch.randn(n_nodes, 9, ch, generator=g, device=device)
    out = edge_tensor_product_uu_radial(x, vec, h, wl, plan, mod.tp_info_forward, edge_vectors=True)
    grads = torch.autograd.grad(out, (x, vec, h, wl), ct)
    sh = SphericalHarmonics(2)(vec)
    w = (h @ wl.view(r, -1)).view(n_edges, 11, ch)
    assert w.numel() > 2 ** 31
    out2 = edge_tensor_product_uu(x, sh, w, plan, mod.tp_info_forward)
    grads2 = torch.autograd.grad(out2, (x, vec, h, wl), ct)
    for name, a, b in zip(("out", "grad_x", "grad_vec", "grad_h", "grad_w_last"), (out, *grads), (out2, *grads2)):
        assert (a - b).abs().max().item() <= 1e-4 * max(1.0, b.abs().max().item()), name
    del w, sh, out, out2, grads, grads2
    torch.cuda.empty_cache()
