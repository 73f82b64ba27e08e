"""GPU parity of the channel-wise tensor product (compiled-in and table-driven kernels) against the dense
float64 oracle, on seeded inputs.  Tolerance: rel/abs 1e-5 for fp32, 1e-12 for fp64 (see helpers.assert_close)."""
import pytest
import torch

from helpers import assert_close, tp_inputs
from oracle import ref_ops

pytestmark = pytest.mark.gpu

SH = {1: "0e+1o", 2: "0e+1o+2e", 3: "0e+1o+2e+3o"}


def _module(irreps_in1, irreps_in2, irreps_out, **kw):
    from equitorch_amd.nn import SO3Linear
    return SO3Linear(irreps_in1, irreps_in2, irreps_out, internal_weights=False, feature_mode="uu", **kw)


def _run(mod, x, sh, w, ct, device):
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
    out = mod(xd, shd, wd)
    (out * ct.to(device)).sum().backward()
    torch.cuda.synchronize()
    return out, xd.grad, shd.grad, wd.grad


@pytest.mark.parametrize("lmax", [1, 2, 3])
@pytest.mark.parametrize("channels", [64, 16, 20, 7, 128])
@pytest.mark.parametrize("shared_w", [False, True])
def test_u1u_compiled_fp32(device, lmax, channels, shared_w):
    from equitorch_amd.ops import kernels
    irreps = SH[lmax]
    mod = _module(irreps, irreps, irreps).to(device)
    assert kernels.uvu_config_of(mod.tp_info_forward) >= 0, "table should be compiled in"
    n, d = 300, (lmax + 1) ** 2
    x, sh, w = tp_inputs(n, d, lmax, mod.num_paths, channels, shared_w, seed=lmax * 100 + channels)
    ct = torch.randn(n, d, channels, generator=torch.Generator().manual_seed(7))
    got = _run(mod, x, sh, w, ct, device)
    T = ref_ops.dense_coupling(irreps, irreps, irreps)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"lmax={lmax} C={channels} shared={shared_w} {name}")


@pytest.mark.parametrize("shared_w", [False, True])
def test_u1u_compiled_fp64(device, shared_w):
    irreps = SH[2]
    mod = _module(irreps, irreps, irreps).to(device)
    x, sh, w = tp_inputs(100, 9, 2, 11, 10, shared_w, seed=3, dtype=torch.float64)
    ct = torch.randn(100, 9, 10, generator=torch.Generator().manual_seed(7), dtype=torch.float64)
    got = _run(mod, x, sh, w, ct, device)
    # fp32 table coefficients, so compare against a dense oracle built from the same rounded table
    T = ref_ops.dense_coupling(irreps, irreps, irreps).float().double()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-12, f"fp64 shared={shared_w} {name}")


@pytest.mark.parametrize("shared_w", [False, True])
@pytest.mark.parametrize("channels", [33, 64])
def test_u1u_table_driven(device, shared_w, channels):
    """Irreps with no compiled-in table go through the LDS-table kernel."""
    from equitorch_amd.ops import kernels
    i1, i2, io = "0e+1o+2e", "0e+1o", "1o+2e+1e"
    mod = _module(i1, i2, io).to(device)
    assert kernels.uvu_config_of(mod.tp_info_forward) < 0
    n = 257
    x, sh, w = tp_inputs(n, 9, 1, mod.num_paths, channels, shared_w, seed=11)
    ct = torch.randn(n, mod.irreps_out.dim, channels, generator=torch.Generator().manual_seed(7))
    got = _run(mod, x, sh, w, ct, device)
    T = ref_ops.dense_coupling(io, i1, i2)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"table-driven C={channels} shared={shared_w} {name}")


@pytest.mark.parametrize("shared_w", [False, True])
def test_edge_fused_small(device, shared_w):
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    irreps = SH[2]
    mod = _module(irreps, irreps, irreps).to(device)
    gen = torch.Generator().manual_seed(5)
    n_nodes, n_edges, ch = 97, 1500, 64
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes - 3, (n_edges,), generator=gen)  # last nodes receive nothing
    x, sh, w = tp_inputs(n_edges, 9, 2, 11, ch, shared_w, seed=6)
    x = x[:n_nodes].contiguous()
    ct = torch.randn(n_nodes, 9, ch, generator=gen)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
    out = edge_tensor_product_uu(xd, shd, wd, plan, mod.tp_info_forward)
    (out * ct.to(device)).sum().backward()
    T = ref_ops.dense_coupling(irreps, irreps, irreps)

    def ref_fn(T, x, sh, w):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, xd.grad, shd.grad, wd.grad),
                          (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"edge fused shared={shared_w} {name}")


@pytest.mark.parametrize("pos_per_wave,ch", [(4, 32), (8, 32), (32, 32), (60, 32), (8, 7), (12, 18), (8, 64)])
@pytest.mark.parametrize("hub", [False, True])
def test_edge_fused_range_modes(device, pos_per_wave, ch, hub):
    """Ranges cut by position (partial rows + fix-up kernel) must give the same rows as segment-aligned ranges,
    including with a hub node whose segment spans many wavefronts and with empty segments.  7 and 18 channels: rows
    whose length is no multiple of four, which the fix-up kernel adds element by element."""
    from equitorch_amd.nn.functional import EdgePlan
    from equitorch_amd.ops import kernels
    irreps = SH[2]
    mod = _module(irreps, irreps, irreps).to(device)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    gen = torch.Generator().manual_seed(9)
    n_nodes, n_edges = 61, 900
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    if hub:
        dst[100:600] = 17
        src[300:700] = 5
    x, sh, w = tp_inputs(n_edges, 9, 2, 11, ch, False, seed=10)
    x = x[:n_nodes].contiguous()
    ct = torch.randn(n_nodes, 9, ch, generator=gen)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd, ctd = (t.to(device) for t in (x, sh, w, ct))
    T = ref_ops.dense_coupling(irreps, irreps, irreps)

    def ref_fn(T, x, sh, w):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, sh, w), ct)
    out = kernels.uvu_forward(cfg, dims, xd, shd, wd, seg=plan.fwd_index, pos_per_wave=pos_per_wave)
    gx, gy, gw = kernels.uvu_backward(cfg, dims, xd, shd, wd, ctd, (True, True, True), seg=plan.bwd_index,
                                      pos_per_wave=pos_per_wave)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"ppw={pos_per_wave} C={ch} hub={hub} {name}")
    if not hub:
        assert plan.fwd_index.wave_seg is not None
    out_a = kernels.uvu_forward(cfg, dims, xd, shd, wd, seg=plan.fwd_index)
    assert_close(out_a, ref_out, 1e-5, "aligned out")


SH6 = "0e+1o+2e+3o+4e+5o+6e"


@pytest.mark.parametrize("lmax,channels", [(6, 32), (6, 20), (6, 64), (4, 48), (5, 32)])
def test_u1u_large_table_fp32(device, lmax, channels):
    """lmax = 4..6 (lmax = 6: 106 paths, 6460 coefficients) on the large-table kernels: forward and all gradients,
    per-row weights, against the dense float64 oracle."""
    from equitorch_amd.ops import kernels
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    d = (lmax + 1) ** 2
    mod = _module(irreps, irreps, irreps).to(device)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    assert cfg >= 0 and kernels.uvu_dims(cfg)[:4] == (d, d, d, mod.num_paths)
    if lmax == 6:
        assert kernels.uvu_dims(cfg) == (49, 49, 49, 106, 6460)
    n = 77
    x, sh, w = tp_inputs(n, d, lmax, mod.num_paths, channels, False, seed=100 * lmax + channels)
    ct = torch.randn(n, d, channels, generator=torch.Generator().manual_seed(7))
    assert kernels.uvu_launchable(cfg, x.to(device), sh.to(device), w.to(device))
    got = _run(mod, x, sh, w, ct, device)
    T = ref_ops.dense_coupling(irreps, irreps, irreps)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"lmax={lmax} C={channels} {name}")


@pytest.mark.parametrize("lmax,n,ch", [(6, 40, 16), (4, 700, 32), (2, 300, 64), (2, 5000, 64), (1, 9000, 32)])
def test_u1u_block_wise_shared_weight(device, lmax, n, ch):
    """Shared weight on the block-wise kernels: its gradient is written per row and summed in two fixed-order
    passes (700 rows: three first-pass chunks; 5000 and 9000 rows: more wavefronts than the register-resident
    kernels' grid-stride launch would use)."""
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    d = (lmax + 1) ** 2
    mod = _module(irreps, irreps, irreps).to(device)
    x, sh, w = tp_inputs(n, d, lmax, mod.num_paths, ch, True, seed=66 + lmax)
    ct = torch.randn(n, d, ch, generator=torch.Generator().manual_seed(7))
    got = _run(mod, x, sh, w, ct, device)
    T = ref_ops.dense_coupling(irreps, irreps, irreps)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"lmax={lmax} shared {name}")


@pytest.mark.parametrize("lmax,n,ch", [(4, 700, 32), (2, 5000, 64)])
def test_shared_weight_backward_in_row_parts(device, monkeypatch, lmax, n, ch):
    """The same gradients when the rows are taken in parts because the per-row weight-gradient workspace would pass
    its limit (set to 1 MB here: several parts with an uneven tail), against the dense oracle and against the single
    launch."""
    from equitorch_amd.ops import kernels
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    d = (lmax + 1) ** 2
    mod = _module(irreps, irreps, irreps).to(device)
    x, sh, w = tp_inputs(n, d, lmax, mod.num_paths, ch, True, seed=166 + lmax)
    ct = torch.randn(n, d, ch, generator=torch.Generator().manual_seed(8))
    whole = _run(mod, x, sh, w, ct, device)
    calls = []
    real = kernels._lib.lib.cgtp_uvu_bwd
    monkeypatch.setattr(kernels, "_GW_WORKSPACE_BYTES", 1 << 20)
    monkeypatch.setattr(kernels._lib.lib, "cgtp_uvu_bwd", lambda a, s: (calls.append(1), real(a, s))[1])
    parts = _run(mod, x, sh, w, ct, device)
    assert len(calls) > 1, "the backward was not split"
    T = ref_ops.dense_coupling(irreps, irreps, irreps)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    gw32 = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct, dtype=torch.float32)[1][2]
    for name, g, h, r in zip(("out", "grad_x", "grad_sh", "grad_w"), parts, whole, (ref_out, *ref_grads)):
        # the shared weight's gradient sums over all rows: norm-wise, and within three times the fp32 contraction's own loss
        assert_close(g, r, 1e-5, f"lmax={lmax} rows in parts {name}", norm="max" if name == "grad_w" else "element",
                     fp32_ref=gw32 if name == "grad_w" else None)
        if name != "grad_w":            # per-row results do not depend on the split
            assert torch.equal(g, h), name


@pytest.mark.parametrize("ch", [32, 20, 64])
def test_edge_large_table(device, ch):
    """Edge message passing at lmax = 6 (BASELINE configs[4] shapes, small graph) through the public path: the
    block-wise kernels in segment mode (gather, product and segment sum in one launch) against the dense oracle."""
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    mod = _module(SH6, SH6, SH6).to(device)
    gen = torch.Generator().manual_seed(15)
    n_nodes, n_edges = 41, 333
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes - 2, (n_edges,), generator=gen)
    x, sh, w = tp_inputs(n_edges, 49, 6, mod.num_paths, ch, False, seed=16)
    x = x[:n_nodes].contiguous()
    ct = torch.randn(n_nodes, 49, ch, generator=gen)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    assert kernels.uvu_launchable(cfg, xd.detach(), shd.detach(), wd.detach(), segments=True), "fused path expected"
    out = edge_tensor_product_uu(xd, shd, wd, plan, mod.tp_info_forward)
    (out * ct.to(device)).sum().backward()
    T = ref_ops.dense_coupling(SH6, SH6, SH6)

    def ref_fn(T, x, sh, w):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, xd.grad, shd.grad, wd.grad),
                          (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"edge lmax=6 C={ch} {name}")


@pytest.mark.parametrize("lmax,ch,per", [(4, 32, 1), (4, 16, 3), (4, 32, 7), (6, 32, 64), (4, 8, 5), (4, 32, 5000)])
def test_edge_large_table_ranges(device, lmax, ch, per):
    """The same kernels with ranges of `per` sorted positions: a hub node whose segment spans many ranges, nodes
    without edges, a last range that is not full, and one range that holds everything."""
    from equitorch_amd.nn.functional import EdgePlan
    from equitorch_amd.ops import kernels
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    mod = _module(irreps, irreps, irreps).to(device)
    d = (lmax + 1) ** 2
    gen = torch.Generator().manual_seed(100 + per)
    n_nodes, n_edges = 37, 301
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes - 3, (n_edges,), generator=gen)
    dst[::3] = 5                                           # hub: a third of all edges end at node 5
    src[1::4] = 11                                         # and a quarter start at node 11
    x, sh, w = tp_inputs(n_edges, d, lmax, mod.num_paths, ch, False, seed=17)
    x = x[:n_nodes].contiguous()
    ct = torch.randn(n_nodes, d, ch, generator=gen)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    xd, shd, wd, ctd = (t.to(device) for t in (x, sh, w, ct))
    out = kernels.uvu_forward(cfg, dims, xd, shd, wd, seg=plan.fwd_index, pos_per_wave=per)
    gx, gy, gw = kernels.uvu_backward(cfg, dims, xd, shd, wd, ctd, (True, True, True), seg=plan.bwd_index,
                                      pos_per_wave=per)
    T = ref_ops.dense_coupling(irreps, irreps, irreps)

    def ref_fn(T, x, sh, w):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"edge lmax={lmax} C={ch} per={per} {name}")
    # only some gradients requested
    gx2, gy2, gw2 = kernels.uvu_backward(cfg, dims, xd, shd, wd, ctd, (True, False, False), seg=plan.bwd_index,
                                         pos_per_wave=per)
    assert gy2 is None and gw2 is None and torch.equal(gx2, gx)
    gx3, gy3, gw3 = kernels.uvu_backward(cfg, dims, xd, shd, wd, ctd, (False, True, True), seg=plan.bwd_index,
                                         pos_per_wave=per)
    assert gx3 is None and torch.equal(gy3, gy) and torch.equal(gw3, gw)


@pytest.mark.parametrize("lmax,n,ch", [(3, 130, 128), (2, 257, 200), (2, 33, 65)])
@pytest.mark.parametrize("shared_w", [False, True])
def test_u1u_block_wise_wide_rows(device, lmax, n, ch, shared_w):
    """More than 64 channels, fp32: forward and backward run one channel chunk per wavefront; grad_sh is summed over
    the chunks' partial sums in a fixed order."""
    irreps = SH[lmax]
    d = (lmax + 1) ** 2
    mod = _module(irreps, irreps, irreps).to(device)
    x, sh, w = tp_inputs(n, d, lmax, mod.num_paths, ch, shared_w, seed=90 + lmax)
    ct = torch.randn(n, d, ch, generator=torch.Generator().manual_seed(8))
    got = _run(mod, x, sh, w, ct, device)
    T = ref_ops.dense_coupling(irreps, irreps, irreps)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"lmax={lmax} C={ch} shared={shared_w} {name}")


@pytest.mark.parametrize("lmax,channels", [(2, 64), (2, 20), (3, 48), (2, 96)])
@pytest.mark.parametrize("shared_w", [False, True])
def test_uuu_on_the_block_wise_kernels(device, lmax, channels, shared_w):
    """TensorProduct('uuu') with a compiled table: both operands channelled, fp32, forward and all gradients against
    the dense oracle; a second-order gradient goes through the table-driven contraction and must agree too."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.nn import TensorProduct
    from equitorch_amd.ops import kernels
    irr = SH[lmax]
    d = (lmax + 1) ** 2
    mod = TensorProduct(irr, irr, irr, channels, channels, channels, feature_mode="uuu", internal_weights=False).to(device)
    assert kernels.uvu_config_of(mod.tp_info_forward) >= 0
    g = torch.Generator().manual_seed(31 + lmax)
    n = 77
    x = torch.randn(n, d, channels, generator=g)
    y = torch.randn(n, d, channels, generator=g)
    w = torch.randn(*(() if shared_w else (n,)), mod.num_paths, channels, generator=g)
    ct = torch.randn(n, d, channels, generator=g)
    T = ref_ops.dense_coupling(irr, irr, irr)
    xr, yr, wr = (t.double().requires_grad_(True) for t in (x, y, w))
    ref = torch.einsum(f"pmab,nau,nbu,{'' if shared_w else 'n'}pu->nmu", T, xr, yr, wr)
    rg = torch.autograd.grad(ref, (xr, yr, wr), ct.double(), create_graph=True)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = F.tensor_product_uuu(xd, yd, wd, mod.tp_info_forward)
    assert kernels.uvu_launchable(kernels.uvu_config_of(mod.tp_info_forward), xd.detach(), yd.detach(), wd.detach())
    got = torch.autograd.grad(out, (xd, yd, wd), ct.to(device), create_graph=True)
    assert_close(out, ref, 1e-5, "uuu out")
    for name, a, b in zip(("grad_x", "grad_y", "grad_w"), got, rg):
        assert_close(a, b, 1e-5, f"uuu lmax={lmax} shared={shared_w} {name}")
    # first-order gradients without create_graph take the compiled backward kernel
    plain = torch.autograd.grad(F.tensor_product_uuu(xd, yd, wd, mod.tp_info_forward), (xd, yd, wd), ct.to(device))
    for name, a, b in zip(("grad_x", "grad_y", "grad_w"), plain, rg):
        assert_close(a, b, 1e-5, f"uuu compiled backward {name}")
    # second order: d/dx of <grad_y, ct2>
    ct2 = torch.randn(n, d, channels, generator=g)
    (hx,) = torch.autograd.grad((got[1] * ct2.to(device)).sum(), xd)
    (rhx,) = torch.autograd.grad((rg[1] * ct2.double()).sum(), xr)
    assert_close(hx, rhx, 1e-5, "uuu second order")


@pytest.mark.parametrize("hub", [False, True])
def test_edge_large_table_hub_and_shared_weight(device, hub):
    """lmax = 4, C = 48 on the block-wise kernels, with and without a hub node: per-edge weights take the fused segment
    mode, a shared weight the gathered row-mode launches plus segment sums; both against the dense oracle."""
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    irr = "0e+1o+2e+3o+4e"
    mod = _module(irr, irr, irr).to(device)
    gen = torch.Generator().manual_seed(21)
    n_nodes, n_edges, ch = 37, 700, 48
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes - 2, (n_edges,), generator=gen)
    if hub:
        dst[50:450] = 11
        src[200:600] = 3
    T = ref_ops.dense_coupling(irr, irr, irr)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    for shared in (False, True):
        x, sh, w = tp_inputs(n_edges, 25, 4, mod.num_paths, ch, shared, seed=22)
        x = x[:n_nodes].contiguous()
        ct = torch.randn(n_nodes, 25, ch, generator=gen)
        xd, shd, wd = (t.to(device).requires_grad_(True) for t in (x, sh, w))
        out = edge_tensor_product_uu(xd, shd, wd, plan, mod.tp_info_forward)
        (out * ct.to(device)).sum().backward()

        def ref_fn(T, x, sh, w):
            return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w), dst, n_nodes)
        ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, sh, w), ct)
        for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, xd.grad, shd.grad, wd.grad),
                              (ref_out, *ref_grads)):
            assert_close(g, r, 1e-5, f"lmax=4 hub={hub} shared={shared} {name}")


def _subset_paths(irreps, drop):
    from oracle import ref_tables
    full = ref_tables.fully_connected_paths(*(ref_tables.parse(irreps),) * 3)
    return [p for n, p in enumerate(full) if n not in drop]


@pytest.mark.parametrize("kw", [{"path_norm": False}, {"path": "subset"}, {"path": "subset", "path_norm": False}])
@pytest.mark.parametrize("shared_w", [False, True])
def test_u1u_options_that_rescale_or_drop_paths_stay_on_the_compiled_kernels(device, kw, shared_w):
    """``path_norm=False`` and an explicit ``path=`` subset (``SO3Linear`` arguments of the reference,
    ``equitorch/nn/linears.py:85-95``) give tables that differ from the compiled one by a factor per weight path and
    by missing paths: they must select the same compiled kernels, in row mode and in the fused edge mode, and agree
    with the dense oracle built with the same options."""
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    irreps = SH[2]
    kw = dict(kw)
    if kw.get("path") == "subset":
        kw["path"] = _subset_paths(irreps, (2, 5, 6))
    mod = _module(irreps, irreps, irreps, **kw).to(device)
    base = _module(irreps, irreps, irreps).to(device)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    assert cfg >= 0 and int(cfg) == int(kernels.uvu_config_of(base.tp_info_forward))
    assert cfg.path_scale is not None
    n, ch = 300, 64
    x, sh, w = tp_inputs(n, 9, 2, mod.num_paths, ch, shared_w, seed=77)
    ct = torch.randn(n, 9, ch, generator=torch.Generator().manual_seed(7))
    got = _run(mod, x, sh, w, ct, device)
    T = ref_ops.dense_coupling(irreps, irreps, irreps, path=kw.get("path"), path_norm=kw.get("path_norm", True))
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, sh, w), ct)
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), got, (ref_out, *ref_grads)):
        assert_close(g, r, 1e-5, f"{sorted(kw)} shared={shared_w} {name}")
    # fused edge mode
    gen = torch.Generator().manual_seed(5)
    n_nodes = 40
    src = torch.randint(0, n_nodes, (n,), generator=gen)
    dst = torch.randint(0, n_nodes, (n,), generator=gen)
    xn, ctn = x[:n_nodes].contiguous(), ct[:n_nodes].contiguous()
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd = (t.to(device).requires_grad_(True) for t in (xn, sh, w))
    out = edge_tensor_product_uu(xd, shd, wd, plan, mod.tp_info_forward)
    (out * ctn.to(device)).sum().backward()

    def ref_fn(T, x, sh, w, dtype=torch.float64):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w, dtype=dtype), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (xn, sh, w), ctn)
    gw32 = ref_ops.dense_grads(ref_fn, T, (xn, sh, w), ctn, dtype=torch.float32)[1][2] if shared_w else None
    for name, g, r in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, xd.grad, shd.grad, wd.grad),
                          (ref_out, *ref_grads)):
        # a shared weight's gradient sums over all edges: norm-wise, and within three times the fp32 contraction's own loss
        long_sum = shared_w and name == "grad_w"
        assert_close(g, r, 1e-5, f"edge {sorted(kw)} shared={shared_w} {name}",
                     norm="max" if long_sum else "element", fp32_ref=gw32 if long_sum else None)


def test_u1u_so3_lmax4_reference_test_irreps(device):
    """``0e+1e+2e+3e+4e`` for all three operands — the irreps of the reference's own comparison test
    (``test/test_tp/test_tensor_product_channel_e3nn.py:639-646``) — runs on a compiled table, with and without
    ``path_norm``."""
    from equitorch_amd.ops import kernels
    irreps = "0e+1e+2e+3e+4e"
    for path_norm in (True, False):
        mod = _module(irreps, irreps, irreps, path_norm=path_norm).to(device)
        assert kernels.uvu_config_of(mod.tp_info_forward) >= 0
        n, ch = 256, 16
        g = torch.Generator().manual_seed(3)
        x = torch.randn(n, 25, ch, generator=g)
        y = torch.randn(n, 25, generator=g)
        w = torch.randn(n, mod.num_paths, ch, generator=g)
        ct = torch.randn(n, 25, ch, generator=g)
        assert kernels.uvu_launchable(kernels.uvu_config_of(mod.tp_info_forward), x.to(device), y.to(device), w.to(device))
        got = _run(mod, x, y, w, ct, device)
        T = ref_ops.dense_coupling(irreps, irreps, irreps, path_norm=path_norm)
        ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, y, w), ct)
        for name, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), got, (ref_out, *ref_grads)):
            # up to 61 paths x hundreds of coefficients per element, inputs not normalised: norm-wise for the sums
            assert_close(a, b, 1e-5, f"so3 lmax=4 path_norm={path_norm} {name}",
                         norm="element" if name == "grad_w" else "max")


@pytest.mark.parametrize("hub", [False, True])
def test_edge_fused_ranges_balanced_by_steps(device, hub):
    """Ranges cut after equal numbers of steps (``cgtp_uvu_args.wave_pos``; cuts inside segments, partial rows and
    the fix-up kernel) give the rows of segment-aligned ranges, forward and backward, also with a hub node whose
    segment spans many wavefronts and with empty segments."""
    from equitorch_amd.nn.functional import EdgePlan
    from equitorch_amd.ops import kernels
    irreps = SH[2]
    mod = _module(irreps, irreps, irreps).to(device)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    dims = kernels.uvu_dims(cfg)
    gen = torch.Generator().manual_seed(19)
    n_nodes, n_edges, ch = 83, 2100, 64
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes - 2, (n_edges,), generator=gen)
    if hub:
        dst[100:900] = 17
        src[300:1200] = 5
    x, sh, w = tp_inputs(n_edges, 9, 2, 11, ch, False, seed=20)
    x = x[:n_nodes].contiguous()
    ct = torch.randn(n_nodes, 9, ch, generator=gen)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, shd, wd, ctd = (t.to(device) for t in (x, sh, w, ct))
    results = {}
    for mode in ("aligned", "balanced"):
        kernels._RANGE_MODE = mode
        try:
            out = kernels.uvu_forward(cfg, dims, xd, shd, wd, seg=plan.fwd_index)
            grads = kernels.uvu_backward(cfg, dims, xd, shd, wd, ctd, (True, True, True), seg=plan.bwd_index)
        finally:
            kernels._RANGE_MODE = "auto"
        results[mode] = (out, *grads)
    wave_pos = plan.bwd_index.balanced_positions(4)
    assert wave_pos[0] == 0 and wave_pos[-1] == n_edges and bool((wave_pos[1:] > wave_pos[:-1]).all())
    for name, a, b in zip(("out", "grad_x", "grad_sh", "grad_w"), results["balanced"], results["aligned"]):
        # per-edge results are the same numbers; node rows cut by a range boundary are summed in another order
        assert_close(a, b, 1e-5, f"balanced vs aligned hub={hub} {name}")
