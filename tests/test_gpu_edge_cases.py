"""Degenerate inputs through the public modules: an empty batch, a single row, a graph without edges, and modules
converted to bfloat16 (their coefficient tables are then bfloat16 tensors too, as after ``module.to(dtype)`` in the
reference).  An empty batch yields empty outputs and zero parameter gradients without a launch; reduced precision
is computed in float32 and rounded once, so it agrees with the float32 module to bfloat16 rounding."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_ops

pytestmark = pytest.mark.gpu

IRR, C = "0e+1o+2e", 32


def _modules(device):
    from equitorch_amd import nn as enn
    from equitorch_amd.nn.functional import sincos

    def angles(n, dt):
        return tuple(sincos(torch.linspace(-2.0, 2.5, n, device=device).to(dt) * (k + 1), 2) for k in range(3))

    return {
        "LayerRMSNorm": (lambda: enn.LayerRMSNorm(IRR, C), lambda n, dt: ()),
        "Gate": (lambda: enn.Gate(IRR, activation=None), lambda n, dt: (torch.randn(n, 3, C, device=device, dtype=dt),)),
        "SquaredNorm": (lambda: enn.SquaredNorm(IRR), lambda n, dt: ()),
        "Norm": (lambda: enn.Norm(IRR), lambda n, dt: ()),
        "TensorDot": (lambda: enn.TensorDot(IRR, "uu"),
                      lambda n, dt: (torch.randn(n, 9, C, device=device, dtype=dt),)),
        "IrrepsLinear": (lambda: enn.IrrepsLinear(IRR, IRR, C, C), lambda n, dt: ()),
        "IrrepWiseLinear": (lambda: enn.IrrepWiseLinear(IRR, C, C), lambda n, dt: ()),
        "SO2Linear_uu": (lambda: enn.SO2Linear(IRR, IRR, C, C, feature_mode="uu"), lambda n, dt: ()),
        "SO2Linear_uv": (lambda: enn.SO2Linear(IRR, IRR, C, C, feature_mode="uv"), lambda n, dt: ()),
        "SparseWignerRotation": (lambda: enn.SparseWignerRotation(IRR), angles),
        "SO3Linear_uu": (lambda: enn.SO3Linear(IRR, IRR, IRR, C, C, feature_mode="uu"),
                         lambda n, dt: (torch.randn(n, 9, device=device, dtype=dt),)),
        "SO3Linear_uv": (lambda: enn.SO3Linear(IRR, IRR, IRR, C, C, feature_mode="uv"),
                         lambda n, dt: (torch.randn(n, 9, device=device, dtype=dt),)),
        "TensorProduct_uuu": (lambda: enn.TensorProduct(IRR, IRR, IRR, C, C, C, feature_mode="uuu"),
                              lambda n, dt: (torch.randn(n, 9, C, device=device, dtype=dt),)),
    }


NAMES = ["LayerRMSNorm", "Gate", "SquaredNorm", "Norm", "TensorDot", "IrrepsLinear", "IrrepWiseLinear", "SO2Linear_uu",
         "SO2Linear_uv", "SparseWignerRotation", "SO3Linear_uu", "SO3Linear_uv", "TensorProduct_uuu"]


def _run(mod, x, extra):
    out = mod(x, *extra)
    params = list(mod.parameters())
    grads = torch.autograd.grad(out.float().sum(), [x] + params, allow_unused=True)
    return out, grads[0], grads[1:]


@pytest.mark.parametrize("name", NAMES)
def test_empty_batch_and_single_row(device, name):
    torch.manual_seed(0)
    make, extra = _modules(device)[name]
    mod = make().to(device)
    x = torch.randn(0, 9, C, device=device, requires_grad=True)
    out, gx, gparams = _run(mod, x, extra(0, torch.float32))
    assert out.shape[0] == 0 and gx.shape == x.shape
    for p, g in zip(mod.parameters(), gparams):
        assert g is None or (g.shape == p.shape and not g.any()), "a sum over no rows must be zero"
    # one row against the same row inside a batch of five
    xs = torch.randn(5, 9, C, device=device, requires_grad=True)
    ex = extra(5, torch.float32)
    full, _, _ = _run(mod, xs, ex)
    one, _, _ = _run(mod, xs[2:3].detach().requires_grad_(True), tuple(e[2:3] for e in ex))
    assert_close(one, full[2:3], tol=1e-6, what=f"{name}: row alone vs in a batch")


@pytest.mark.parametrize("name", NAMES)
def test_module_converted_to_bfloat16(device, name):
    torch.manual_seed(1)
    make, extra = _modules(device)[name]
    ref = make().to(device)
    low = make().to(device)
    low.load_state_dict(ref.state_dict())
    low = low.to(torch.bfloat16)
    n = 70
    x = torch.randn(n, 9, C, device=device)
    torch.manual_seed(2)
    ex = extra(n, torch.float32)
    exl = tuple(e.to(torch.bfloat16) for e in ex)
    xl = x.to(torch.bfloat16).requires_grad_(True)
    out, gx, _ = _run(low, xl, exl)
    assert out.dtype == torch.bfloat16 and gx.dtype == torch.bfloat16
    # the float32 module on the same (rounded) inputs and parameters
    for p, q in zip(ref.parameters(), low.parameters()):
        p.data.copy_(q.data.float())
    xr = xl.detach().float().requires_grad_(True)
    want, gwant, _ = _run(ref, xr, tuple(e.float() for e in exl))
    assert_close(out.float(), want, tol=3e-2, what=f"{name} bf16 output", norm="max")
    assert_close(gx.float(), gwant, tol=3e-2, what=f"{name} bf16 grad_x", norm="max")


@pytest.mark.parametrize("n_nodes,n_edges", [(10, 0), (0, 0), (10, 1)])
@pytest.mark.parametrize("vectors", [False, True])
def test_graph_without_edges(device, n_nodes, n_edges, vectors):
    from equitorch_amd import nn as enn
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_vectors
    torch.manual_seed(3)
    tp = enn.SO3Linear(IRR, IRR, IRR, C, C, internal_weights=False, feature_mode="uu").to(device)
    src = torch.randint(0, max(n_nodes, 1), (n_edges,), device=device)
    dst = torch.randint(0, max(n_nodes, 1), (n_edges,), device=device)
    plan = EdgePlan(src, dst, n_nodes)
    x = torch.randn(n_nodes, 9, C, device=device, requires_grad=True)
    w = torch.randn(n_edges, tp.num_paths, C, device=device, requires_grad=True)
    if vectors:
        y = torch.randn(n_edges, 3, device=device, requires_grad=True)
        out = edge_tensor_product_uu_vectors(x, y, w, plan, tp.tp_info_forward)
    else:
        y = torch.randn(n_edges, 9, device=device, requires_grad=True)
        out = edge_tensor_product_uu(x, y, w, plan, tp.tp_info_forward)
    gx, gy, gw = torch.autograd.grad(out.sum(), [x, y, w])
    assert out.shape == (n_nodes, 9, C) and gx.shape == x.shape and gy.shape == y.shape and gw.shape == w.shape
    touched = torch.zeros(n_nodes, dtype=torch.bool, device=device)
    touched[dst] = True
    assert not out[~touched].any(), "nodes without incoming edges receive zero"
    if n_edges == 0:
        assert not gx.any()


def test_converted_module_runs_on_the_compiled_kernels(device):
    """``SO3Linear(..., 'uv').to(torch.bfloat16)`` carries bfloat16 tables; they still select the matrix-core
    kernels, and the result agrees with the float32 module on the same rounded operands."""
    from equitorch_amd import nn as enn
    from equitorch_amd.nn.functional import _uvw_mfma
    from equitorch_amd.ops import kernels
    torch.manual_seed(4)
    irr, c, n = "0e+1o+2e+3o", 64, 300
    ref = enn.SO3Linear(irr, irr, irr, c, c, feature_mode="uv").to(device)
    low = enn.SO3Linear(irr, irr, irr, c, c, feature_mode="uv").to(device)
    low.load_state_dict(ref.state_dict())
    low = low.to(torch.bfloat16)
    assert low.tp_info_forward.info_Mij_fwd.scale.dtype == torch.bfloat16
    assert kernels.uv_config_of(low.tp_info_forward) == kernels.uv_config_of(ref.tp_info_forward) >= 0
    x = torch.randn(n, 16, c, device=device).bfloat16().requires_grad_(True)
    y = torch.randn(n, 16, device=device).bfloat16().requires_grad_(True)
    assert _uvw_mfma.try_forward(x, y, low.weight, low.tp_info_forward) is not None
    out = low(x, y)
    ct = torch.randn_like(out)
    grads = torch.autograd.grad(out, [x, y, low.weight], ct)
    with torch.no_grad():
        ref.weight.copy_(low.weight.float())
    xr, yr = x.detach().float().requires_grad_(True), y.detach().float().requires_grad_(True)
    want = ref(xr, yr)
    gwant = torch.autograd.grad(want, [xr, yr, ref.weight], ct.float())
    # bf16 results: rel 1e-2 of the tensor's magnitude (twice that: both operands of the comparison are rounded)
    assert_close(out.float(), want, tol=2e-2, what="bf16 module output", norm="max")
    for name, a, b in zip(("grad_x", "grad_y", "grad_w"), grads, gwant):
        assert_close(a.float(), b, tol=2e-2, what=name, norm="max")
    # the channel-wise product of a float16 module finds its compiled table as well
    half = enn.SO3Linear("0e+1o+2e", "0e+1o+2e", "0e+1o+2e", c, c, feature_mode="uu").to(device).half()
    assert kernels.uvu_config_of(half.tp_info_forward) >= 0


def test_baseline_configurations_take_their_kernels(device, monkeypatch):
    """The five benchmark configurations, at small sizes, must reach the kernels written for them: the fused segment
    kernels for the edge products (lmax = 2 and lmax = 6), the compiled channel-wise kernel for the row product with a
    shared weight, the bf16 matrix-core kernel for the fully connected product."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils._sh import spherical_harmonics
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append((op, tier)))
    g = torch.Generator().manual_seed(3)

    def irreps(lmax):
        return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))

    def unit(n):
        v = torch.randn(n, 3, generator=g)
        return v / v.norm(dim=1, keepdim=True)
    # configs 1-2 (lmax = 2, C = 64) and 4 (lmax = 6, C = 32): per-edge weights on a graph
    for lmax, ch in ((2, 64), (6, 32)):
        irr, d = irreps(lmax), (lmax + 1) ** 2
        mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu").to(device)
        n_nodes, n_edges = 50, 400
        plan = EdgePlan(torch.randint(0, n_nodes, (n_edges,), generator=g).to(device),
                        torch.randint(0, n_nodes, (n_edges,), generator=g).to(device), n_nodes)
        x = torch.randn(n_nodes, d, ch, generator=g).to(device).requires_grad_(True)
        sh = spherical_harmonics(unit(n_edges), lmax).to(device)
        w = torch.randn(n_edges, mod.num_paths, ch, generator=g).to(device)
        edge_tensor_product_uu(x, sh, w, plan, mod.tp_info_forward).sum().backward()
        assert seen[-1] == ("edge_tensor_product_uu", "fused gather / product / segment sum"), (lmax, seen)
    # config 0: B = 1024, C = 16, shared weight
    irr = irreps(2)
    mod = SO3Linear(irr, irr, irr, 16, 16, internal_weights=False, feature_mode="uu").to(device)
    x = torch.randn(1024, 9, 16, generator=g).to(device)
    mod(x, spherical_harmonics(unit(1024), 2).to(device), torch.randn(mod.num_paths, 16, generator=g).to(device))
    assert seen[-1] == ("tensor_product_u1u", "compiled table"), seen
    # config 3: bf16, 128 -> 128 channels, lmax = 3, shared weight
    irr = irreps(3)
    mod = SO3Linear(irr, irr, irr, 128, 128, internal_weights=False, feature_mode="uv").to(device)
    x = torch.randn(256, 16, 128, generator=g).to(device).bfloat16()
    y = spherical_harmonics(unit(256), 3).to(device).bfloat16()
    w = (torch.randn(mod.num_paths, 128, 128, generator=g) / 40).to(device).bfloat16()
    mod(x, y, w)
    assert seen[-1] == ("tensor_product_u1v", "matrix-core kernel (compiled table)"), seen


@pytest.mark.parametrize("irreps", [("2e+0e", "0e", "0e"), ("0e+1o+2e", "0e+1e+2e", "1o"), ("0e+1o+2e", "0e+1e+2e", "0e")])
def test_output_irreps_that_no_path_reaches_follow_the_reference_tables(device, irreps):
    """The reference numbers the rows of its second-stage table ``info_M_fwd`` by their rank among the output rows
    that some path reaches (``equitorch/utils/_structs.py:228-231``: the batch index of ``extract_batch_segments``, not
    the row it stands for), and every product Function takes its output rows from that table
    (``nn/functional/linears.py:24-25, :262-263``, ``tensor_products.py:17-18, :100-101``).  When an output irrep that
    no path reaches precedes one that is reached — ``0e x 0e -> 2e+0e`` — the reference therefore writes the result
    into the first rows of the output and leaves the last ones zero.  The tables of this package are the reference's
    bit for bit, so the kernels do the same: the product here must equal the reference's algorithm on the reference's
    tables (the CPU oracle), which differs from the dense contraction with the Clebsch-Gordan tensor in exactly the
    rows that moved."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from oracle import ref_tables
    io, i1, i2 = irreps
    c, n = 8, 33
    fwd = ref_ops.tables_to_torch(ref_tables.tp_infos(io, i1, i2)[0], torch.float64)
    g = torch.Generator().manual_seed(5)
    d1, d2, do = Irreps(i1).dim, Irreps(i2).dim, Irreps(io).dim
    x = torch.randn(n, d1, c, generator=g, dtype=torch.float64)
    y = torch.randn(n, d2, generator=g, dtype=torch.float64)
    for mode, oracle in (("uu", ref_ops.cpu_u1u_forward), ("uv", ref_ops.cpu_u1v_forward)):
        mod = SO3Linear(i1, i2, io, c, c, internal_weights=False, feature_mode=mode).to(device)
        w = torch.randn(*((mod.num_paths, c) if mode == "uu" else (mod.num_paths, c, c)), generator=g, dtype=torch.float64)
        out = mod(x.float().to(device), y.float().to(device), w.float().to(device))
        ref, _ = oracle(x, y, w, fwd)
        assert out.shape == (n, do, c)
        assert_close(out, ref, 1e-5, f"{mode} {i1} x {i2} -> {io}: the reference's algorithm on its tables", norm="max")
        T = ref_ops.dense_coupling(io, i1, i2, **({"channel_scale": c ** -0.5} if mode == "uv" else {})).double()
        dense = (ref_ops.dense_u1u if mode == "uu" else ref_ops.dense_u1v)(T, x, y, w)
        assert float((dense - ref).abs().max()) > 0.1, "the dense contraction places these rows elsewhere"


@pytest.mark.parametrize("irreps,kw", [(("0e+1o+2e", "0e+1o+2e", "0e+1o+2e+3o"), {}),
                                       (("0e+1o+2e", "0e+1o+2e", "0e+1o+2e"), {"path_norm": False}),
                                       (("0e+1o+2e", "0e+1o+2e", "0e+1o+2e"), {})])
def test_float64_on_a_table_that_matches_a_compiled_one_up_to_rounding(device, monkeypatch, irreps, kw):
    """The reference's tables hold the fp32 product of coupling and normalisation.  A table that is a compiled one
    times a factor per path (a subset of its paths, another normalisation) matches it entry by entry only to an fp32
    rounding: good enough for fp32 operands, 1e-8 off for float64 ones.  float64 operands take the compiled kernels
    for bit-exact matches only and the table-driven kernels otherwise — 1e-11 against the dense oracle built from the
    module's own fp32 coefficients either way, on a batch and over an edge list."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    from equitorch_amd.ops import kernels
    i1, i2, io = irreps
    ch, n_nodes, n_edges = 8, 40, 333
    mod = SO3Linear(i1, i2, io, ch, ch, internal_weights=False, feature_mode="uu", **kw).to(device)
    cfg = kernels.uvu_config_of(mod.tp_info_forward)
    assert int(cfg) >= 0
    if io != i1:
        assert not cfg.exact        # a subset of the paths of a larger compiled table, renormalised
    elif not kw:
        assert cfg.exact and cfg.path_scale is None
    T = ref_ops.dense_coupling(io, i1, i2, **kw).float().double()
    g = torch.Generator().manual_seed(len(io) + len(kw))
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    src, dst = torch.randint(0, n_nodes, (n_edges,), generator=g), torch.randint(0, n_nodes, (n_edges,), generator=g)
    x, sh, w = rd(n_nodes, Irreps(i1).dim, ch), rd(n_edges, Irreps(i2).dim), rd(n_edges, mod.num_paths, ch)
    ct = rd(n_nodes, Irreps(io).dim, ch)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    dev = [t.to(device).requires_grad_(True) for t in (x, sh, w)]
    out = edge_tensor_product_uu(*dev, plan, mod.tp_info_forward)
    assert ("fused gather / product / segment sum" == seen[0]) == cfg.exact, seen
    grads = torch.autograd.grad(out, dev, ct.to(device))
    ref_fn = lambda T, x, sh, w: ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), sh, w), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, (x, sh, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, *grads), (ref_out, *ref_grads)):
        assert_close(a, b, 1e-11, f"{io} {kw} edge list {name}", norm="max")
    xe = x.index_select(0, src)
    dev = [t.to(device).requires_grad_(True) for t in (xe, sh, w)]
    cte = rd(n_edges, Irreps(io).dim, ch)
    out = mod(*dev)
    grads = torch.autograd.grad(out, dev, cte.to(device))
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (xe, sh, w), cte)
    for name, a, b in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, *grads), (ref_out, *ref_grads)):
        assert_close(a, b, 1e-11, f"{io} {kw} batch {name}", norm="max")


def test_empty_batch_with_a_weight_per_sample(device):
    """No samples and a weight with a sample axis: the weight has no elements, which the reference's per-sample rule
    (``weight.numel() > weight_numel`` then ``view(-1, ...)``, ``equitorch/nn/linears.py:163-168``) cannot tell from a
    malformed shared weight.  Taken as zero sets of weights here: empty result, empty gradients of the right shapes."""
    from equitorch_amd import nn as enn
    irr = "0e+1o+2e"
    mods = [
        (enn.IrrepsLinear(irr, irr, 8, 12, internal_weights=False), lambda m: [(0, 9, 8), (0, m.num_paths, 8, 12)], (0, 9, 12)),
        (enn.IrrepWiseLinear(irr, 8, 12, internal_weights=False), lambda m: [(0, 9, 8), (0, 3, 8, 12)], (0, 9, 12)),
        (enn.SO2Linear(irr, irr, 8, 12, internal_weights=False, feature_mode="uv"),
         lambda m: [(0, 9, 8), (0, m.num_weights, 8, 12)], (0, 9, 12)),
        (enn.SO2Linear(irr, irr, 8, 8, internal_weights=False, feature_mode="uu"),
         lambda m: [(0, 9, 8), (0, m.num_weights, 8)], (0, 9, 8)),
        (enn.SO3Linear(irr, irr, irr, 8, 8, internal_weights=False, feature_mode="uu"),
         lambda m: [(0, 9, 8), (0, 9), (0, m.num_paths, 8)], (0, 9, 8)),
        (enn.SO3Linear(irr, irr, irr, 8, 12, internal_weights=False, feature_mode="uv"),
         lambda m: [(0, 9, 8), (0, 9), (0, m.num_paths, 8, 12)], (0, 9, 12)),
        (enn.TensorProduct(irr, irr, irr, 4, 4, 8, internal_weights=False, feature_mode="uvw"),
         lambda m: [(0, 9, 4), (0, 9, 4), (0, m.num_paths, 4, 4, 8)], (0, 9, 8)),
    ]
    for mod, shapes, out_shape in mods:
        mod = mod.to(device)
        ops = [torch.zeros(*s, device=device, requires_grad=True) for s in shapes(mod)]
        out = mod(*ops)
        assert tuple(out.shape) == out_shape, (type(mod).__name__, out.shape)
        grads = torch.autograd.grad(out, ops, torch.zeros_like(out), allow_unused=True)
        for t, g in zip(ops, grads):
            assert g is None or g.shape == t.shape
