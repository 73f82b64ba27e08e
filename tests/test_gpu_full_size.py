"""GPU parity at the full sizes of the benchmark configurations: the fused edge tensor product at
N = 4096 / E = 65536 (lmax = 2, C = 64) and the large-table edge product at N = 20000 / E = 200000 (lmax = 6,
C = 32), forward and all gradients.

The dense float64 oracle cannot run at these sizes in seconds, so it is run on sub-problems that are exact for a
strided subset of the result rows: an output row depends only on the in-edges of its node, a ``grad_x`` row only on
the out-edges of its node, ``grad_sh`` / ``grad_W`` rows only on their own edge.  The subsets are spread over the
whole index range so that every wavefront range, every XCD share and the tail of the launch contribute rows.
Inputs follow the benchmark's recipe (one CPU generator seeded 0; src, dst, x, unit vectors -> harmonics, W,
cotangent, in that order)."""
import pytest
import torch

from helpers import assert_close, unit_vectors
from oracle import ref_ops

pytestmark = pytest.mark.gpu


def _sh_irreps(lmax):
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


def _inputs(n_nodes, n_edges, lmax, channels, n_paths, hubs=0):
    from equitorch_amd.utils._sh import spherical_harmonics
    gen = torch.Generator().manual_seed(0)
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    if hubs:
        # a few nodes of very high in- and out-degree (several wavefront ranges each), the rest stay uniform
        for h in range(hubs):
            dst[1000 + 3000 * h: 1000 + 3000 * h + 700 * (h + 1)] = 97 * (h + 1)
            src[20000 + 3000 * h: 20000 + 3000 * h + 500 * (h + 1)] = 11 * (h + 1)
    d = (lmax + 1) ** 2
    x = torch.randn(n_nodes, d, channels, generator=gen)
    sh = spherical_harmonics(unit_vectors(n_edges, gen), lmax)
    w = torch.randn(n_edges, n_paths, channels, generator=gen)
    ct = torch.randn(n_nodes, d, channels, generator=gen)
    return src, dst, x, sh, w, ct


def _check_subsets(T, src, dst, x, sh, w, ct, got, n_dst, n_src, n_edge, tol=1e-5, tag=""):
    """Compare ``got = (out, grad_x, grad_sh, grad_w)`` (device tensors) with the dense oracle on strided subsets."""
    out, gx, gsh, gw = (t.detach().cpu() for t in got)
    n_nodes, n_edges = x.shape[0], src.shape[0]
    # output rows: all in-edges of a strided set of nodes (+ the first and the last node)
    nodes = torch.unique(torch.cat([torch.arange(3, n_nodes, max(1, n_nodes // n_dst)), torch.tensor([0, n_nodes - 1])]))
    mask = torch.zeros(n_nodes, dtype=torch.bool)
    mask[nodes] = True
    e_in = torch.nonzero(mask[dst]).flatten()
    def out_rows(dt):   # float64: the arbiter; float32: what the same sums lose in the reference's own arithmetic
        msg = ref_ops.dense_u1u(T, x[src[e_in]], sh[e_in], w[e_in], dtype=dt)
        return ref_ops.scatter_sum(msg, dst[e_in], n_nodes)[nodes]
    # rows summed over ~16 (up to hundreds at a hub) edges x all coefficients: norm-wise, and within three times the fp32
    # restatement's own error
    assert_close(out[nodes], out_rows(torch.float64), tol, f"{tag} out rows", norm="max",
                 fp32_ref=out_rows(torch.float32))
    # grad_x rows: all out-edges of a strided set of nodes; grad_sh / grad_w: those edges and a strided set of edges
    nodes = torch.unique(torch.cat([torch.arange(5, n_nodes, max(1, n_nodes // n_src)), torch.tensor([0, n_nodes - 1])]))
    mask = torch.zeros(n_nodes, dtype=torch.bool)
    mask[nodes] = True
    emask = mask[src]
    emask[torch.arange(7, n_edges, max(1, n_edges // n_edge))] = True
    emask[0] = emask[n_edges - 1] = True
    e_sub = torch.nonzero(emask).flatten()
    def grads(dt):
        xr = x.detach().to(dt).clone().requires_grad_(True)
        shr, wr = sh[e_sub].detach().to(dt).clone().requires_grad_(True), w[e_sub].detach().to(dt).clone().requires_grad_(True)
        loss = (ref_ops.dense_u1u(T, xr[src[e_sub]], shr, wr, dtype=dt) * ct[dst[e_sub]].to(dt)).sum()
        return torch.autograd.grad(loss, (xr, shr, wr))
    rgx, rgsh, rgw = grads(torch.float64)
    gx32, gsh32, _ = grads(torch.float32)
    assert_close(gx[nodes], rgx[nodes], tol, f"{tag} grad_x rows", norm="max", fp32_ref=gx32[nodes])
    assert_close(gsh[e_sub], rgsh, tol, f"{tag} grad_sh rows", norm="max", fp32_ref=gsh32)
    assert_close(gw[e_sub], rgw, tol, f"{tag} grad_w rows")


@pytest.mark.parametrize("graph", ["uniform", "hubs"])
def test_edge_fused_full_size_lmax2(device, graph):
    """BASELINE configs[1] / configs[2] shapes through the public autograd path (segment-aligned ranges on the
    uniform graph; the graph with hub nodes takes ranges cut by position, partial rows and the fix-up kernel)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    irr = _sh_irreps(2)
    n_nodes, n_edges, ch = 4096, 65536, 64
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    src, dst, x, sh, w, ct = _inputs(n_nodes, n_edges, 2, ch, mod.num_paths, hubs=3 if graph == "hubs" else 0)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    if graph == "uniform":
        assert plan.fwd_index.wave_seg is not None and plan.bwd_index.wave_seg is not None
    else:
        assert plan.fwd_index.wave_seg is None and plan.bwd_index.wave_seg is None
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
    out = edge_tensor_product_uu(xd, shd, wd, plan, mod.tp_info_forward)
    (out * ct.to(device)).sum().backward()
    T = ref_ops.dense_coupling(irr, irr, irr)
    _check_subsets(T, src, dst, x, sh, w, ct, (out, xd.grad, shd.grad, wd.grad), 64, 64, 512, tag=f"lmax=2 {graph}")


def test_edge_fused_full_size_by_position(device):
    """The same uniform graph with the ranges cut by position (32 per wavefront) instead of at segment boundaries:
    2048 ranges, almost every one starting and ending inside a segment."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan
    from equitorch_amd.ops import kernels
    irr = _sh_irreps(2)
    n_nodes, n_edges, ch = 4096, 65536, 64
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    src, dst, x, sh, w, ct = _inputs(n_nodes, n_edges, 2, ch, mod.num_paths)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd, ctd = (t.to(device) for t in (x, sh, w, ct))
    out = kernels.uvu_forward(cfg, dims, xd, shd, wd, seg=plan.fwd_index, pos_per_wave=32)
    gx, gy, gw = kernels.uvu_backward(cfg, dims, xd, shd, wd, ctd, (True, True, True), seg=plan.bwd_index,
                                      pos_per_wave=32)
    T = ref_ops.dense_coupling(irr, irr, irr)
    _check_subsets(T, src, dst, x, sh, w, ct, (out, gx, gy, gw), 64, 64, 512, tag="lmax=2 by position")


def test_edge_fused_full_size_vectors(device):
    """Full size with the harmonics evaluated inside the kernels (edge vectors in, gradient of the vectors out):
    output and node / weight gradients against the same oracle; the vector gradient against the harmonics' own
    backward applied to the oracle's ``grad_sh`` on the subset."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_vectors
    irr = _sh_irreps(2)
    n_nodes, n_edges, ch = 4096, 65536, 64
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    src, dst, x, _, w, ct = _inputs(n_nodes, n_edges, 2, ch, mod.num_paths)
    vec = torch.randn(n_edges, 3, generator=torch.Generator().manual_seed(1)) * 1.7
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, vd, wd = (t.to(device).requires_grad_(True) for t in (x, vec, w))
    out = edge_tensor_product_uu_vectors(xd, vd, wd, plan, mod.tp_info_forward)
    (out * ct.to(device)).sum().backward()
    from oracle import ref_sh
    T = ref_ops.dense_coupling(irr, irr, irr)
    e_sub = torch.arange(7, n_edges, 128)
    nodes = torch.arange(3, n_nodes, 64)
    mask = torch.zeros(n_nodes, dtype=torch.bool)
    mask[nodes] = True
    e_in = torch.nonzero(mask[dst]).flatten()

    def oracle(dt):     # (grad_vec rows, out rows) with the harmonics of the oracle, in float64 and restated in float32
        vr = vec.detach().to(dt).clone().requires_grad_(True)
        shr = ref_sh.spherical_harmonics(vr / vr.norm(dim=-1, keepdim=True), 2)
        loss = (ref_ops.dense_u1u(T, x.to(dt)[src[e_sub]], shr[e_sub], w[e_sub], dtype=dt) * ct[dst[e_sub]].to(dt)).sum()
        (rgv,) = torch.autograd.grad(loss, vr)
        msg = ref_ops.dense_u1u(T, x[src[e_in]], shr.detach()[e_in], w[e_in], dtype=dt)
        return rgv[e_sub], ref_ops.scatter_sum(msg, dst[e_in], n_nodes)[nodes]
    rgv, rout = oracle(torch.float64)
    gv32, out32 = oracle(torch.float32)
    assert_close(vd.grad.cpu()[e_sub], rgv, 1e-5, "grad_vec rows", norm="max", fp32_ref=gv32)
    assert_close(out.detach().cpu()[nodes], rout, 1e-5, "out rows (vectors)", norm="max", fp32_ref=out32)


def test_edge_full_size_lmax6(device):
    """BASELINE configs[4] shapes: N = 20000, E = 200000, lmax = 6, C = 32, per-edge weights (2.7 GB), forward and
    all gradients through the public autograd path (block-wise kernels in segment mode: 4082 ranges of 49 sorted
    positions, segment sums in LDS)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    irr = _sh_irreps(6)
    n_nodes, n_edges, ch = 20000, 200000, 32
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    src, dst, x, sh, w, ct = _inputs(n_nodes, n_edges, 6, ch, mod.num_paths)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
    out = edge_tensor_product_uu(xd, shd, wd, plan, mod.tp_info_forward)
    (out * ct.to(device)).sum().backward()
    T = ref_ops.dense_coupling(irr, irr, irr)
    _check_subsets(T, src, dst, x, sh, w, ct, (out, xd.grad, shd.grad, wd.grad), 12, 12, 96, tag="lmax=6")


def test_row_mode_full_size_shared_weight(device):
    """BASELINE configs[0] module (``SO3Linear('uu')``, shared weight) at 65536 rows, lmax = 2, C = 64: out / grad_x /
    grad_sh rows on a strided subset; the shared weight's gradient (a sum over all rows) through linearity — the
    gradient for a cotangent that is zero outside the subset equals the oracle's sum over the subset."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.utils._sh import spherical_harmonics
    irr = _sh_irreps(2)
    n, ch = 65536, 64
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    gen = torch.Generator().manual_seed(0)
    x = torch.randn(n, 9, ch, generator=gen)
    sh = spherical_harmonics(unit_vectors(n, gen), 2)
    w = torch.randn(mod.num_paths, ch, generator=gen)
    ct = torch.randn(n, 9, ch, generator=gen)
    sub = torch.arange(11, n, 257)
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
    out = mod(xd, shd, wd)
    gx, gsh, gw = torch.autograd.grad(out, (xd, shd, wd), ct.to(device))
    T = ref_ops.dense_coupling(irr, irr, irr)
    ref_out, (rgx, rgsh, rgw_sub) = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x[sub], sh[sub], w), ct[sub])
    _, (_, gsh32, gw32) = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x[sub], sh[sub], w), ct[sub], dtype=torch.float32)
    assert_close(out[sub.to(device)], ref_out, 1e-5, "row mode out")
    assert_close(gx[sub.to(device)], rgx, 1e-5, "row mode grad_x")
    # sums over 64 channels x 83 terms: norm-wise, and within three times the fp32 contraction's own loss
    assert_close(gsh[sub.to(device)], rgsh, 1e-5, "row mode grad_sh", norm="max", fp32_ref=gsh32)
    masked = torch.zeros_like(ct)
    masked[sub] = ct[sub]
    (gw_sub,) = torch.autograd.grad(mod(xd, shd, wd), (wd,), masked.to(device))
    assert_close(gw_sub, rgw_sub, 1e-5, "row mode grad_w of the subset", norm="max", fp32_ref=gw32)   # sum over 256 rows
    # the full gradient is additive over two halves of the batch
    half = n // 2
    parts = []
    for lo, hi in ((0, half), (half, n)):
        ws = wd.detach().requires_grad_(True)
        (gp,) = torch.autograd.grad(mod(xd[lo:hi].detach(), shd[lo:hi].detach(), ws), (ws,), ct[lo:hi].to(device))
        parts.append(gp)
    assert_close(gw, parts[0] + parts[1], 1e-5, "row mode grad_w additivity", norm="max")  # sums over 65536 rows


def test_edge_radial_full_size(device):
    """BASELINE configs[1] / configs[2] shapes with the per-edge weights formed inside the kernels (R = 16): output
    rows, node gradients and per-edge gradients of seeded subsets against the float64 oracle evaluated on exactly the
    edges those rows depend on; the gradient of the shared matrix (a sum over all edges) through additivity over two
    halves of the edge list."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu_radial
    n_nodes, n_edges, ch, r = 4096, 65536, 64, 16
    irr = "0e+1o+2e"
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    g = torch.Generator().manual_seed(23)
    src = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g)
    x = torch.randn(n_nodes, 9, ch, generator=g)
    sh = torch.randn(n_edges, 9, generator=g)
    h = torch.randn(n_edges, r, generator=g)
    wl = torch.randn(r, mod.num_paths, ch, generator=g) / r ** 0.5
    ct = torch.randn(n_nodes, 9, ch, generator=g)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, hd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, h, wl))
    out = edge_tensor_product_uu_radial(xd, shd, hd, wd, plan, mod.tp_info_forward)
    gx, gsh, gh, gwl = torch.autograd.grad(out, (xd, shd, hd, wd), ct.to(device))
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    nodes = torch.arange(11, n_nodes, 173)
    # output rows of the chosen nodes: all edges that end there
    e_in = torch.nonzero(torch.isin(dst, nodes)).flatten()
    e_out = torch.nonzero(torch.isin(src, nodes)).flatten()

    def oracle(dt):     # out rows, grad_x rows, grad_sh and grad_h of the edges that start at the chosen nodes, in ``dt``
        w_in = torch.einsum("er,rpc->epc", h[e_in].to(dt), wl.to(dt))
        msg = ref_ops.dense_u1u(T, x[src[e_in]], sh[e_in], w_in, dtype=dt)
        rows = ref_ops.scatter_sum(msg, dst[e_in], n_nodes)[nodes]
        # gradients: node rows of grad_x need all edges that start there; per-edge gradients their own edge only
        xr = x.detach().to(dt).clone().requires_grad_(True)
        shr, hr = sh[e_out].detach().to(dt).clone().requires_grad_(True), h[e_out].detach().to(dt).clone().requires_grad_(True)
        w_out = torch.einsum("er,rpc->epc", hr, wl.to(dt))
        loss = (ref_ops.dense_u1u(T, xr[src[e_out]], shr, w_out, dtype=dt) * ct[dst[e_out]].to(dt)).sum()
        rgx, rgsh, rgh = torch.autograd.grad(loss, (xr, shr, hr))
        return rows, rgx[nodes], rgsh, rgh
    ref_rows, rgx, rgsh, rgh = oracle(torch.float64)
    rows32, gx32, gsh32, gh32 = oracle(torch.float32)
    # sums over ~16 edges (rows), 64 channels x coefficients (grad_sh), 11 paths x 64 channels (grad_h): norm-wise, and
    # within three times what the same computation loses in fp32
    assert_close(out[nodes.to(device)], ref_rows, 1e-5, "radial full size out rows", norm="max", fp32_ref=rows32)
    assert_close(gx[nodes.to(device)], rgx, 1e-5, "radial full size grad_x rows", norm="max", fp32_ref=gx32)
    assert_close(gsh[e_out.to(device)], rgsh, 1e-5, "radial full size grad_sh rows", norm="max", fp32_ref=gsh32)
    assert_close(gh[e_out.to(device)], rgh, 1e-5, "radial full size grad_h rows", norm="max", fp32_ref=gh32)
    # grad of the shared matrix: additivity over two halves of the edge list (each half its own plan)
    parts = []
    for lo, hi in ((0, n_edges // 2), (n_edges // 2, n_edges)):
        pl = EdgePlan(src[lo:hi].to(device), dst[lo:hi].to(device), n_nodes)
        ws = wd.detach().requires_grad_(True)
        o = edge_tensor_product_uu_radial(xd.detach(), shd[lo:hi].detach(), hd[lo:hi].detach(), ws, pl, mod.tp_info_forward)
        parts.append(torch.autograd.grad(o, (ws,), ct.to(device))[0].double())
    assert_close(gwl.double(), parts[0] + parts[1], 1e-5, "radial full size grad_w_last additivity", norm="max")


@pytest.mark.parametrize("lmax,ch,n_nodes,n_edges", [(2, 64, 100_000, 3_200_000), (6, 32, 50_000, 700_000)])
def test_edge_kernels_past_two_to_the_31_weight_elements(device, lmax, ch, n_nodes, n_edges):
    """3.2 million edges x 11 paths x 64 channels = 2.25e9 weight elements (9 GB; its gradient as much), and 700 000
    edges x 106 paths x 32 channels at lmax = 6: every element offset past 2^31 must be formed in 64 bits.  No oracle at this size: the fused segment kernels (forward and all
    gradients) against the row-mode kernels followed by segment sums, which share no addressing code with them;
    1e-5 of the tensor's scale (the two paths add in different orders)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan
    from equitorch_amd.ops import kernels
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 50 GB of device memory")
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    d = (lmax + 1) ** 2
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uu").to(device)
    g = torch.Generator(device=device).manual_seed(1)
    src = torch.randint(0, n_nodes, (n_edges,), generator=g, device=device)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g, device=device)
    plan = EdgePlan(src, dst, n_nodes)
    x = torch.randn(n_nodes, d, ch, generator=g, device=device)
    sh = torch.randn(n_edges, d, generator=g, device=device)
    w = torch.randn(n_edges, mod.num_paths, ch, generator=g, device=device)
    ct = torch.randn(n_nodes, d, ch, generator=g, device=device)
    assert w.numel() > 2 ** 31
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    out = kernels.uvu_forward(cfg, dims, x, sh, w, seg=plan.fwd_index)
    gx, gy, gw = kernels.uvu_backward(cfg, dims, x, sh, w, ct, (True, True, True), seg=plan.bwd_index)
    msg = kernels.uvu_forward(cfg, dims, x, sh, w, gather=plan.src)
    out2 = kernels.segment_sum(msg.view(1, n_edges, -1), None, plan.perm_dst, plan.ptr_dst, n_nodes).view(n_nodes, d, ch)
    del msg
    gxe, gy2, gw2 = kernels.uvu_backward(cfg, dims, x, sh, w, ct, (True, True, True), gather=plan.dst,
                                         x_gather=plan.src)
    gx2 = kernels.segment_sum(gxe.view(1, n_edges, -1), None, plan.perm_src, plan.ptr_src, n_nodes).view(n_nodes, d, ch)
    del gxe
    for name, a, b in (("out", out, out2), ("grad_x", gx, gx2), ("grad_sh", gy, gy2), ("grad_w", gw, gw2)):
        scale = max(1.0, b.abs().max().item())
        assert (a - b).abs().max().item() <= 1e-5 * scale, name
    del out, out2, gx, gx2, gy, gy2, gw, gw2, w, sh
    torch.cuda.empty_cache()


def test_fully_connected_bf16_past_two_to_the_31_elements(device):
    """1.2 million samples x 16 x 128 bf16 = 2.46e9 elements per operand: rows at both ends of the batch (the last ones
    lie past 2^31 elements) must come out bit-equal to the same rows computed as a small batch of their own (a row's
    result depends on nothing else), for the output and the gradients of both per-sample operands; the weight
    gradient, a sum over all samples, must be the sum over the two halves of the batch (rel 1e-2, bf16)."""
    from equitorch_amd.nn import SO3Linear
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 40 GB of device memory")
    irreps, ch, n = "0e+1o+2e+3o", 128, 1_200_000
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator(device=device).manual_seed(2)
    x = torch.randn(n, 16, ch, generator=g, device=device).bfloat16().requires_grad_(True)
    y = torch.randn(n, 16, generator=g, device=device).bfloat16().requires_grad_(True)
    w = (torch.randn(mod.num_paths, ch, ch, generator=g, device=device) / 40).bfloat16().requires_grad_(True)
    ct = torch.randn(n, 16, ch, generator=g, device=device).bfloat16()
    assert x.numel() > 2 ** 31
    out = mod(x, y, w)
    gx, gy, gw = torch.autograd.grad(out, (x, y, w), ct)
    idx = torch.cat([torch.arange(0, 64, device=device), torch.arange(n - 1100, n - 1000, device=device),
                     torch.arange(n - 64, n, device=device)])
    xs, ys = (t.detach()[idx].clone().requires_grad_(True) for t in (x, y))
    gxs, gys, _ = torch.autograd.grad(mod(xs, ys, w), (xs, ys, w), ct[idx])
    assert torch.equal(out[idx], mod(xs, ys, w)), "out"
    assert torch.equal(gx[idx], gxs), "grad_x"
    assert torch.equal(gy[idx], gys), "grad_sh"
    del out, gx, gy
    half = n // 2
    parts = []
    for lo, hi in ((0, half), (half, n)):
        xh, yh = x.detach()[lo:hi], y.detach()[lo:hi]
        (gwh,) = torch.autograd.grad(mod(xh, yh, w), (w,), ct[lo:hi])
        parts.append(gwh.float())
    ref = parts[0] + parts[1]
    assert (gw.float() - ref).abs().max().item() <= 1e-2 * ref.abs().max().item(), "grad_w"
    del x, y, ct
    torch.cuda.empty_cache()
