"""GPU parity of the spherical-harmonics kernels (cgtp_sh_forward / cgtp_sh_backward) against the oracle."""
import math

import pytest
import torch

from helpers import assert_close
from oracle import ref_sh

pytestmark = pytest.mark.gpu


def _vectors(n, seed, spread=True):
    g = torch.Generator().manual_seed(seed)
    v = torch.randn(n, 3, generator=g, dtype=torch.float64)
    v = v / v.norm(dim=-1, keepdim=True)
    if spread:   # lengths in [0.6, 1.4]: the polynomials are homogeneous, so this exercises r^l
        v = v * (0.6 + 0.8 * torch.rand(n, 1, generator=g, dtype=torch.float64))
    return v


@pytest.mark.parametrize("l_max", [0, 1, 2, 3, 4, 6, 7, 8, 11, 17])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_forward_matches_oracle(device, l_max, dtype):
    """Four, two or one wavefront tiles in LDS by degree; fp64 at degree 17 addresses global memory directly; n is not
    a multiple of 64."""
    from equitorch_amd.ops import spherical_harmonics
    v = _vectors(1000 + l_max, seed=l_max)
    ref = ref_sh.spherical_harmonics(v, l_max)
    out = spherical_harmonics(v.to(device, dtype), l_max)
    assert out.dtype == dtype and out.shape == ref.shape
    if dtype == torch.float64:
        assert_close(out, ref, tol=1e-12, what=f"Y lmax={l_max}")
    else:
        # fp32 parity bar: rel/abs 1e-5; inputs rounded to fp32 first so that only arithmetic differs
        ref32 = ref_sh.spherical_harmonics(v.float().double(), l_max)
        # degrees above 8 are polynomials with alternating terms larger than the value (not normalised inputs of
        # length up to 1.5: terms of order |v|^l): element-wise up to degree 8, norm-wise beyond
        assert_close(out, ref32, tol=1e-5, what=f"Y lmax={l_max}", norm="element" if l_max <= 8 else "max")


@pytest.mark.parametrize("l_max", [1, 2, 3, 6, 9])
@pytest.mark.parametrize("normalize", [False, True])
@pytest.mark.parametrize("dtype", [torch.float64, torch.float32])
def test_backward_matches_oracle_autograd(device, l_max, normalize, dtype):
    from equitorch_amd.ops import spherical_harmonics
    n = 333
    v = _vectors(n, seed=50 + l_max).to(dtype).double().requires_grad_(True)
    ct = torch.randn(n, (l_max + 1) ** 2, generator=torch.Generator().manual_seed(7), dtype=torch.float64)
    ct = ct.to(dtype).double()
    scale = 0.37
    ref = scale * ref_sh.spherical_harmonics(ref_sh.normalize(v) if normalize else v, l_max)
    (ref * ct).sum().backward()
    vd = v.detach().to(device, dtype).requires_grad_(True)
    out = spherical_harmonics(vd, l_max, normalize=normalize, scale=scale)
    (out * ct.to(device, dtype)).sum().backward()
    tol = 1e-11 if dtype == torch.float64 else 1e-5
    assert_close(out, ref, tol=tol, what="Y")
    # the gradient sums (l_max + 1)^2 polynomial derivatives per component: norm-wise above degree 8 in fp32, and
    # within three times what the oracle's own recursion loses when it runs in fp32
    long_sum = l_max > 8 and dtype == torch.float32
    g32 = None
    if long_sum:
        v32 = v.detach().float().requires_grad_(True)
        (scale * ref_sh.spherical_harmonics(ref_sh.normalize(v32) if normalize else v32, l_max) * ct.float()).sum().backward()
        g32 = v32.grad
    assert_close(vd.grad, v.grad, tol=tol, what="grad_xyz", norm="max" if long_sum else "element", fp32_ref=g32)


def test_module_layout_options_and_edge_cases(device):
    from equitorch_amd.nn import SphericalHarmonics
    from equitorch_amd.nn.functional import spherical_harmonics
    v = _vectors(24, seed=3).reshape(2, 3, 4, 3)
    mod = SphericalHarmonics(3, normalize_input=True, integral_normalize=True)
    ref = ref_sh.spherical_harmonics(ref_sh.normalize(v.reshape(-1, 3)), 3).reshape(2, 3, 4, 16) / math.sqrt(4 * math.pi)
    assert_close(mod(v.to(device)), ref, tol=1e-12, what="module")
    # vectors stored along another dimension
    out = spherical_harmonics(v.permute(0, 3, 1, 2).to(device), 3, dim=1)
    assert out.shape == (2, 16, 3, 4)
    assert_close(out.permute(0, 2, 3, 1), ref_sh.spherical_harmonics(v.reshape(-1, 3), 3).reshape(2, 3, 4, 16),
                 tol=1e-12, what="dim=1")
    # empty batch, single vector, the zero vector under normalisation (F.normalize maps it to zero: only Y_0 survives)
    assert spherical_harmonics(torch.zeros(0, 3, device=device), 2).shape == (0, 9)
    z = torch.zeros(1, 3, device=device, dtype=torch.float64, requires_grad=True)
    y0 = SphericalHarmonics(2)(z)
    assert_close(y0, torch.tensor([[1.0] + [0.0] * 8], dtype=torch.float64), tol=1e-12, what="zero vector")
    y0.sum().backward()
    assert torch.isfinite(z.grad).all()
    # half precision: evaluated in fp32 and rounded once; gradients flow back in the input's dtype
    vb = _vectors(10, seed=4).to(device, torch.bfloat16).requires_grad_(True)
    yb = spherical_harmonics(vb, 2, normalize_input=True)
    assert yb.dtype == torch.bfloat16
    assert_close(yb.float(), ref_sh.spherical_harmonics(ref_sh.normalize(vb.detach().double().cpu()), 2), tol=1e-2,
                 what="bf16")
    yb.sum().backward()
    assert vb.grad.dtype == torch.bfloat16 and torch.isfinite(vb.grad).all()
    with pytest.raises(ValueError):
        spherical_harmonics(torch.zeros(4, 2, device=device), 2)
    with pytest.raises(ValueError):
        spherical_harmonics(torch.zeros(4, 3, device=device), 18)


def test_full_size_properties(device):
    """One million vectors, lmax = 6: |Y_l|^2 = 2l+1 for every vector and degree, and the result does not depend on
    where in the batch a vector sits (rows of a permuted batch are the permuted rows)."""
    from equitorch_amd.ops import spherical_harmonics
    n = 1_000_003
    g = torch.Generator(device=device).manual_seed(0)
    v = torch.randn(n, 3, generator=g, device=device)
    y = spherical_harmonics(v, 6, normalize=True)
    for l in range(7):
        nrm = (y[:, l * l:(l + 1) ** 2] ** 2).sum(-1)
        assert float((nrm - (2 * l + 1)).abs().max()) < 1e-4 * (2 * l + 1)
    perm = torch.randperm(n, generator=g, device=device)
    assert torch.equal(spherical_harmonics(v[perm], 6, normalize=True), y[perm])


SH = {1: "0e+1o", 2: "0e+1o+2e", 3: "0e+1o+2e+3o", 4: "0e+1o+2e+3o+4e"}


@pytest.mark.parametrize("lmax,channels,dtype,normalize", [
    (2, 64, torch.float32, True), (2, 64, torch.float32, False), (3, 32, torch.float32, True),
    (2, 20, torch.float64, True), (1, 64, torch.float32, True), (4, 32, torch.float32, True)])
def test_edge_product_with_harmonics_evaluated_in_the_kernel(device, lmax, channels, dtype, normalize):
    """edge_tensor_product_uu_vectors(x, edge_vec, W) against the dense oracle applied to the oracle's harmonics of
    the (normalised) edge vectors, gathered at src and summed at dst: output and the gradients with respect to the
    node features, the edge vectors and the per-edge weights.  lmax = 4 has no fused kernels and takes the
    harmonics kernel followed by the row-mode kernels."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu_vectors
    from oracle import ref_ops
    n_nodes, n_edges = 50, 600
    g = torch.Generator().manual_seed(100 + lmax)
    irr = SH[lmax]
    mod = SO3Linear(irr, irr, irr, internal_weights=False, feature_mode="uu").to(device)
    d = (lmax + 1) ** 2
    src = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst[dst == 7] = 8                                            # an empty segment
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
    vec = (rd(n_edges, 3) * (0.5 + torch.rand(n_edges, 1, generator=g, dtype=torch.float64))).to(dtype).double()
    T = ref_ops.dense_coupling(irr, irr, irr)
    if dtype == torch.float64:
        T = T.float().double()          # the compiled tables hold the reference's fp32 coefficients
    x, ct, w = rd(n_nodes, d, channels), rd(n_nodes, d, channels), rd(n_edges, mod.num_paths, channels)
    def oracle(dt):
        xs, vs, ws = (t.detach().to(dt).clone().requires_grad_(True) for t in (x, vec, w))
        ys = ref_sh.spherical_harmonics(ref_sh.normalize(vs) if normalize else vs, lmax)
        res = ref_ops.scatter_sum(ref_ops.dense_u1u(T, xs[src], ys, ws, dtype=dt), dst, n_nodes)
        (res * ct.to(dt)).sum().backward()
        return res.detach(), xs.grad, vs.grad, ws.grad
    want = oracle(torch.float64)
    gv32 = oracle(torch.float32)[2] if dtype == torch.float32 else None
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, vd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, vec, w))
    out = edge_tensor_product_uu_vectors(xd, vd, wd, plan, mod.tp_info_forward, normalize_input=normalize)
    (out * ct.to(device, dtype)).sum().backward()
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    for name, a, b in zip(("out", "grad_x", "grad_vec", "grad_w"), (out, xd.grad, vd.grad, wd.grad), want):
        # grad_vec: a sum over all channels and coefficients pushed through the harmonics' derivative — norm-wise, and
        # within three times what the oracle's own chain loses in fp32
        assert_close(a, b, tol=tol, what=f"lmax={lmax} {name}", norm="max" if name == "grad_vec" else "element",
                     fp32_ref=gv32 if name == "grad_vec" else None)


def test_add_spherical_harmonics_transform(device):
    """``transforms.AddSphericalHarmonics`` on a plain attribute container: the harmonics of the raw edge vectors
    (``r^l`` scaling kept, as in the reference's transform), with and without the ``1 / sqrt(4 pi)`` factor."""
    from types import SimpleNamespace

    from equitorch_amd.transforms import AddSphericalHarmonics, AddVectorNorm
    v = _vectors(257, seed=21)
    data = SimpleNamespace(edge_vec=v.to(device))
    out = AddVectorNorm()(AddSphericalHarmonics(3)(data))
    assert out.edge_sh.shape == (257, 16) and not hasattr(data, "edge_sh")
    assert_close(out.edge_sh, ref_sh.spherical_harmonics(v, 3), tol=1e-12, what="edge_sh")
    assert_close(out.edge_norm, v.norm(dim=-1), tol=1e-12, what="edge_norm")
    scaled = AddSphericalHarmonics(2, sh_attr="y", integral_normalize=True)(data)
    assert_close(scaled.y, ref_sh.spherical_harmonics(v, 2) / math.sqrt(4 * math.pi), tol=1e-12, what="scaled")


def test_harmonics_past_two_to_the_31_elements(device):
    """44 million vectors x 49 components (lmax = 6) = 2.16e9 output elements: the first and the last thousand rows and
    their gradients must be bit-equal to the same vectors evaluated as a batch of their own."""
    from equitorch_amd.nn import SphericalHarmonics
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 30 GB of device memory")
    n = 44_000_000
    g = torch.Generator(device=device).manual_seed(4)
    v = torch.randn(n, 3, generator=g, device=device).requires_grad_(True)
    sh = SphericalHarmonics(6).to(device)
    out = sh(v)
    assert out.numel() > 2 ** 31
    idx = torch.cat([torch.arange(0, 1000, device=device), torch.arange(n - 1000, n, device=device)])
    ct = torch.randn(2000, 49, generator=g, device=device)
    full_ct = torch.zeros_like(out)
    full_ct[idx] = ct
    (gv,) = torch.autograd.grad(out, v, full_ct)
    vs = v.detach()[idx].clone().requires_grad_(True)
    outs = sh(vs)
    (gvs,) = torch.autograd.grad(outs, vs, ct)
    assert torch.equal(out[idx], outs) and torch.equal(gv[idx], gvs)
    del out, full_ct, gv, v
    torch.cuda.empty_cache()
