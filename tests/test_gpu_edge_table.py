"""Edge message passing for irreps WITHOUT a compiled table: gather, channel-wise product and segment sum still run
as one launch, on the table-driven segment kernels (``cgtp_uvu_tab_fwd`` / ``cgtp_uvu_tab_bwd``: the table is data,
read through the scalar cache; per-edge operands and segment sums live in LDS).  The reference runs such irreps on
its table-driven kernels at the same speed as any other (``equitorch/ops/batched_sparse_dense_op.py:63-152``).
Forward and all gradients against the dense float64 oracle; the kernel route is asserted."""
import pytest
import torch

from helpers import assert_close, stable_seed
from oracle import ref_ops

pytestmark = pytest.mark.gpu

# (irreps_out, irreps_in1, irreps_in2): none of them has a compiled table
TABLES = [
    ("1o+2e+1e", "0e+1o+2e", "0e+1o"),
    ("0e+1o+2e+3o", "1o+2e+3o", "0e+1o+2e"),
    ("2x0e+1o+1e", "0e+2x1o", "0e+1o+1e"),
]


def _graph(n_nodes, n_edges, gen, hub=False):
    src = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=gen)
    if hub:                       # one node collects a third of the edges, one node has none
        dst[torch.rand(n_edges, generator=gen) < 0.33] = 3
        dst[dst == 5] = 6
        src[src == 9] = 10
    return src, dst


def _run_case(device, irreps, channels, n_nodes, n_edges, hub, shared_w, seed, monkeypatch):
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    io, i1, i2 = irreps
    mod = SO3Linear(i1, i2, io, channels, channels, internal_weights=False, feature_mode="uu").to(device)
    assert int(kernels.uvu_config_of(mod.tp_info_forward)) < 0, "pick irreps without a compiled table for this test"
    d1, d2, do = Irreps(i1).dim, Irreps(i2).dim, Irreps(io).dim
    gen = torch.Generator().manual_seed(seed)
    src, dst = _graph(n_nodes, n_edges, gen, hub)
    x = torch.randn(n_nodes, d1, channels, generator=gen)
    y = torch.randn(n_edges, d2, generator=gen)
    w = torch.randn(*(() if shared_w else (n_edges,)), mod.num_paths, channels, generator=gen)
    ct = torch.randn(n_nodes, do, channels, generator=gen)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, yd = x.to(device).requires_grad_(True), y.to(device).requires_grad_(True)
    wd = w.to(device).requires_grad_(not shared_w)
    out = edge_tensor_product_uu(xd, yd, wd, plan, mod.tp_info_forward)
    assert seen and "table-driven fused" in seen[-1], seen
    grads = torch.autograd.grad(out, (xd, yd) + ((wd,) if not shared_w else ()), ct.to(device))
    T = ref_ops.dense_coupling(io, i1, i2).float().double()        # the tables hold fp32 coefficients

    def ref_fn(T, x, y, w, dtype=torch.float64):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), y, w, dtype=dtype), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, y, w), ct)
    what = f"{io} <- {i1} x {i2} C={channels} hub={hub} shared_w={shared_w}"
    assert_close(out, ref_out, 1e-5, what + " out")
    for name, a, b in zip(("grad_x", "grad_y", "grad_w"), grads, ref_grads):
        assert_close(a, b, 1e-5, what + " " + name)


@pytest.mark.parametrize("irreps", TABLES)
@pytest.mark.parametrize("channels,hub", [(64, False), (64, True), (20, False), (7, True), (128, False)])
def test_edge_product_without_a_compiled_table(device, monkeypatch, irreps, channels, hub):
    """64 channels: four per lane, four edges per wavefront; 20: five lanes of four (groups of eight lanes, three
    idle); 7: one channel per lane; 128: one edge per wavefront half.  ``hub``: a node with a third of all edges (its
    segment spans many ranges: partial rows and the fix-up pass), a node without edges (a zero row)."""
    _run_case(device, irreps, channels, 60, 1500, hub, False, stable_seed("edge table", irreps, channels, hub),
              monkeypatch)


def test_shared_weight_forward_and_operand_gradients(device, monkeypatch):
    """A shared weight that needs no gradient stays on the fused kernels (its gradient, a sum over all edges, is not
    formed there: a weight that requires one takes the separate launches)."""
    _run_case(device, TABLES[0], 32, 50, 900, True, True, 11, monkeypatch)


def test_ranges_of_every_length(device, monkeypatch):
    """Few edges (ranges of the minimum length, most wavefront slots past the end of the list) and many (ranges of
    several dozen positions)."""
    _run_case(device, TABLES[0], 64, 10, 37, False, False, 5, monkeypatch)
    _run_case(device, TABLES[1], 32, 2000, 70000, False, False, 6, monkeypatch)


def test_speed_next_to_the_other_routes(device, monkeypatch):
    """E = 65536, N = 4096, C = 64, forward + backward.  The fused table-driven launch must beat the separate launches
    it replaces (index_select, table-driven product, segment sum), and its time per coefficient stays within six times
    that of the compiled lmax = 2 table on the same graph (measured: 4.3 times; interpreting a table costs about four
    vector instructions where generated code has one — irreps that matter are compiled in, see
    ``equitorch_amd/csrc/register.py``)."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    n_nodes, n_edges, ch = 4096, 65536, 64
    gen = torch.Generator().manual_seed(0)
    src, dst = _graph(n_nodes, n_edges, gen)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    fused_table = kernels.uvu_table_of
    ms, nnz = {}, {}
    for name, (io, i1, i2), table_of in (("table", TABLES[1], fused_table), ("separate", TABLES[1], lambda *a: None),
                                         ("compiled", ("0e+1o+2e",) * 3, fused_table)):
        monkeypatch.setattr(kernels, "uvu_table_of", table_of)
        mod = SO3Linear(i1, i2, io, ch, ch, internal_weights=False, feature_mode="uu").to(device)
        nnz[name] = kernels.coo_of(mod.tp_info_forward).coef.shape[0]
        x = torch.randn(n_nodes, Irreps(i1).dim, ch, device=device, requires_grad=True)
        y = torch.randn(n_edges, Irreps(i2).dim, device=device, requires_grad=True)
        w = torch.randn(n_edges, mod.num_paths, ch, device=device, requires_grad=True)
        ct = torch.randn(n_nodes, Irreps(io).dim, ch, device=device)

        def step():
            out = edge_tensor_product_uu(x, y, w, plan, mod.tp_info_forward)
            torch.autograd.grad(out, (x, y, w), ct)
        for _ in range(3):
            step()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for _ in range(10):
            step()
        b.record()
        torch.cuda.synchronize()
        ms[name] = a.elapsed_time(b) / 10
        print(f"{name}: {nnz[name]} coefficients, {ms[name]:.3f} ms per forward + backward")
    assert ms["table"] < ms["separate"], ms
    assert ms["table"] / nnz["table"] <= 6.0 * ms["compiled"] / nnz["compiled"], (ms, nnz)


@pytest.mark.parametrize("irreps,channels", [(TABLES[0], 64), (TABLES[2], 20), (("0e+2e+4e",) * 3, 32)])
def test_plain_batch_without_a_compiled_table(device, monkeypatch, irreps, channels):
    """``SO3Linear('uu')`` on a batch for irreps without a compiled table: the segment kernels with every row a node of
    one edge; forward, all gradients and a gradient of the gradient (which goes to the differentiable contraction)."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.ops import kernels
    io, i1, i2 = irreps
    mod = SO3Linear(i1, i2, io, channels, channels, internal_weights=False, feature_mode="uu").to(device)
    assert int(kernels.uvu_config_of(mod.tp_info_forward)) < 0
    n = 777
    gen = torch.Generator().manual_seed(stable_seed("row table", irreps, channels))
    x, y = torch.randn(n, Irreps(i1).dim, channels, generator=gen), torch.randn(n, Irreps(i2).dim, generator=gen)
    w, ct = torch.randn(n, mod.num_paths, channels, generator=gen), torch.randn(n, Irreps(io).dim, channels, generator=gen)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = mod(xd, yd, wd)
    assert "segment kernels on the batch" in seen[-1], seen
    grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device), retain_graph=True)
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, y, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads)):
        assert_close(a, b, 1e-5, f"{io} C={channels} batch {name}")
    gx, = torch.autograd.grad(out, xd, ct.to(device), create_graph=True)
    gg = torch.autograd.grad(gx.square().sum(), (yd, wd))
    xr, yr, wr = (t.double().requires_grad_(True) for t in (x, y, w))
    rgx, = torch.autograd.grad(ref_ops.dense_u1u(T, xr, yr, wr), xr, ct.double(), create_graph=True)
    rgg = torch.autograd.grad(rgx.square().sum(), (yr, wr))
    for name, a, b in zip(("d/dy", "d/dw"), gg, rgg):
        assert_close(a, b, 1e-5, f"{io} batch second order {name}", norm="max")
