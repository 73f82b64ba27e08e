"""GPU parity of the table-driven operator family and of the uv / uvw tensor products against the oracle.

The operator sweep follows the reference's own test procedure (test/test_op/test_sparse_structs.py:668-733):
Irreps((1,3)) tables, N=135, every shared / accumulated flag combination, forward and gradients, here against
the oracle's restatement of the reference CPU ops (and dense einsum for the matrix members)."""
import itertools

import pytest
import torch

from helpers import assert_close, fp32_twin, stable_seed
from oracle import ref_ops, ref_tables

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tables13():
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr = Irreps((1, 3))
    mine = tp_infos(irr, irr, irr)[0]
    ref = ref_ops.tables_to_torch(ref_tables.tp_infos((1, 3), (1, 3), (1, 3))[0], torch.float64)
    return mine, ref


def _dense_from_info(info, size1, size2):
    """(out, size1, size2) float64 coupling of one sparse product table."""
    n = info["scale"].shape[0]
    i1 = info["index1"] if info["index1"] is not None else torch.arange(n)
    i2 = info["index2"] if info["index2"] is not None else torch.arange(n)
    seg = info["seg_out"]
    out_idx = torch.repeat_interleave(torch.arange(seg.shape[0] - 1), seg[1:] - seg[:-1])
    T = torch.zeros(seg.shape[0] - 1, size1, size2, dtype=torch.float64)
    T.index_put_((out_idx, i1, i2), info["scale"].double(), accumulate=True)
    return T


EW = {  # name: (oracle fn, axes1, axes2)
    "mul": (ref_ops.cpu_mul, "u", "u"), "inner": (ref_ops.cpu_inner, "u", "u"),
    "vecsca": (ref_ops.cpu_vecsca, "u", ""), "scavec": (ref_ops.cpu_scavec, "", "u"),
}


@pytest.mark.parametrize("op", sorted(EW))
@pytest.mark.parametrize("shared1,shared2,acc", [s for s in itertools.product([False, True], repeat=3)
                                                 if not (s[0] and s[1] and s[2])])
@pytest.mark.parametrize("channels", [97, 35])
def test_elementwise_ops_sweep(device, tables13, op, shared1, shared2, acc, channels):
    import equitorch_amd.nn.functional as F
    mine, ref = tables13
    oracle, ax1, ax2 = EW[op]
    info_m, info_r = mine.info_Mij_fwd.to(device), ref["info_Mij_fwd"]
    g = torch.Generator().manual_seed(stable_seed(op, shared1, shared2, acc, channels))
    n, d = 135, 15

    def mk(axes, shared):
        shape = (() if shared else (n,)) + (d,) + ((channels,) if axes else ())
        return torch.randn(*shape, generator=g, dtype=torch.float64)
    x, y = mk(ax1, shared1), mk(ax2, shared2)
    fn = getattr(F, f"sparse_{op}")
    xd, yd = (t.float().to(device).requires_grad_(True) for t in (x, y))
    out = fn(xd, yd, info_m, out_accumulated=acc)
    xr, yr = (t.float().double().requires_grad_(True) for t in (x, y))
    ref_out = oracle(xr, yr, info_r, out_accumulated=acc)
    assert_close(out, ref_out, 1e-5, f"{op} forward")
    ct = torch.randn(ref_out.shape, generator=g, dtype=torch.float64)
    gx, gy = torch.autograd.grad(out, (xd, yd), ct.float().to(device))
    rgx, rgy = torch.autograd.grad(ref_out, (xr, yr), ct.float().double())
    assert_close(gx, rgx, 1e-5, f"{op} grad1")
    assert_close(gy, rgy, 1e-5, f"{op} grad2")


@pytest.mark.parametrize("table", ["info_Mij_fwd", "info_M_fwd"])
@pytest.mark.parametrize("n,channels,dtype", [(1025, 97, torch.float32), (1500, 260, torch.float32),
                                              (3000, 97, torch.float32), (1500, 130, torch.float64),
                                              (2000, 64, torch.float32)])
def test_row_sums_beyond_1024_rows(device, tables13, table, n, channels, dtype):
    """Sums over the batch (``out_accumulated``, gradient of a shared operand) with more rows than the row-by-row
    kernel has wavefronts (1024): shares of the rows are then uneven and the last wavefronts own none.  Heavy
    (``info_Mij_fwd``) and light (``info_M_fwd``: one coefficient per row) tables, channel counts that take the
    staged, the 16-byte and the one-channel-per-lane kernels, fp32 and fp64; against the CPU restatement."""
    import equitorch_amd.nn.functional as F
    mine, ref = tables13
    info_m, info_r = getattr(mine, table).to(device), dict(ref[table])
    if info_r["scale"] is not None:
        info_r["scale"] = info_r["scale"].float().double()      # the tables hold fp32 coefficients
    nnz = info_r["scale"].shape[0] if info_r["scale"] is not None else info_r["seg_out"][-1].item()
    size = lambda idx: nnz if idx is None else int(idx.max()) + 1
    d1, d2 = size(info_r["index1"]), size(info_r["index2"])
    g = torch.Generator().manual_seed(n + channels)
    x = torch.randn(n, d1, channels, generator=g, dtype=torch.float64).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    for op, oracle, y in (("mul", ref_ops.cpu_mul, torch.randn(n, d2, channels, generator=g, dtype=torch.float64)),
                          ("inner", ref_ops.cpu_inner, torch.randn(n, d2, channels, generator=g, dtype=torch.float64)),
                          ("vecsca", ref_ops.cpu_vecsca, torch.randn(n, d2, generator=g, dtype=torch.float64))):
        y = y.to(dtype)
        out = getattr(F, f"sparse_{op}")(x.to(device), y.to(device), info_m, out_accumulated=True)
        # sums of n products of N(0,1) numbers: magnitude sqrt(n) * coefficients; compared norm-wise, and against what
        # the same CPU function loses in fp32
        r32 = fp32_twin(oracle, x, y, info_r, out_accumulated=True) if dtype == torch.float32 else None
        assert_close(out, oracle(x.double(), y.double(), info_r, out_accumulated=True), tol, f"{op} row sum",
                     norm="max", fp32_ref=r32)
    # gradient of a shared second operand (the sum over rows happens in the backward launch)
    w = torch.randn(d2, channels, generator=g, dtype=torch.float64).to(dtype)
    wd = w.to(device).requires_grad_(True)
    ct = torch.randn(n, info_r["seg_out"].shape[0] - 1, channels, generator=g, dtype=torch.float64).to(dtype)
    (gw,) = torch.autograd.grad(F.sparse_mul(x.to(device), wd, info_m), (wd,), ct.to(device))
    def shared_grad(dt):
        wr = w.detach().to(dt).clone().requires_grad_(True)
        info = {k: (v.to(dt) if isinstance(v, torch.Tensor) and v.is_floating_point() else v) for k, v in info_r.items()}
        return torch.autograd.grad(ref_ops.cpu_mul(x.to(dt), wr, info), (wr,), ct.to(dt))[0]
    assert_close(gw, shared_grad(torch.float64), tol, "shared-operand gradient", norm="max",
                 fp32_ref=shared_grad(torch.float32) if dtype == torch.float32 else None)


MAT = {  # name: (axes1, axes2, out axes, einsum)
    "outer": ("u", "w", "uw", "mab,{a}au,{b}bw->{o}muw"),
    "vecmat": ("u", "uw", "w", "mab,{a}au,{b}buw->{o}mw"),
    "mat_t_vec": ("uw", "u", "w", "mab,{a}auw,{b}bu->{o}mw"),
}


@pytest.mark.parametrize("op", sorted(MAT))
@pytest.mark.parametrize("shared1,shared2,acc", [(False, False, False), (False, True, False), (True, False, False),
                                                 (False, False, True), (False, True, True)])
def test_matrix_ops_sweep(device, tables13, op, shared1, shared2, acc):
    import equitorch_amd.nn.functional as F
    mine, ref = tables13
    ax1, ax2, axo, eq = MAT[op]
    info_m = mine.info_Mij_fwd.to(device)
    T = _dense_from_info(ref["info_Mij_fwd"], 15, 15)
    g = torch.Generator().manual_seed(stable_seed(op, shared1, shared2, acc))
    n, d, U, W = 37, 15, 21, 13
    ext = {"u": U, "w": W}

    def mk(axes, shared):
        return torch.randn(*((() if shared else (n,)) + (d,) + tuple(ext[a] for a in axes)), generator=g,
                           dtype=torch.float64)
    x, y = mk(ax1, shared1), mk(ax2, shared2)
    xd, yd = (t.float().to(device).requires_grad_(True) for t in (x, y))
    out = getattr(F, f"sparse_{op}")(xd, yd, info_m, out_accumulated=acc)
    eq = eq.format(a="" if shared1 else "n", b="" if shared2 else "n", o="" if (shared1 and shared2) else "n")

    def dense(dt):      # the dense contraction in float64 (the arbiter) and in float32 (what fp32 arithmetic loses)
        xr, yr = (t.float().detach().to(dt).clone().requires_grad_(True) for t in (x, y))
        o = torch.einsum(eq, T.to(dt), xr, yr)
        return (o.sum(0) if acc else o), xr, yr
    ref_out, xr, yr = dense(torch.float64)
    out32, x32, y32 = dense(torch.float32)
    # results summed over the batch (accumulated output, gradient of a shared operand) and over up to 21 channels
    # and ~40 coefficients per element: norm-wise; per-row results element-wise
    assert_close(out, ref_out, 1e-5, f"{op} forward", norm="max" if acc else "element", fp32_ref=out32)
    ct = torch.randn(ref_out.shape, generator=g, dtype=torch.float64)
    gx, gy = torch.autograd.grad(out, (xd, yd), ct.float().to(device))
    rgx, rgy = torch.autograd.grad(ref_out, (xr, yr), ct.float().double())
    gx32, gy32 = torch.autograd.grad(out32, (x32, y32), ct.float())
    assert_close(gx, rgx, 1e-5, f"{op} grad1", norm="max" if shared1 else "element", fp32_ref=gx32)
    assert_close(gy, rgy, 1e-5, f"{op} grad2", norm="max" if shared2 else "element", fp32_ref=gy32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("op", ["vecmat", "mat_t_vec"])
def test_shared_matrix_ops_on_the_matrix_core_kernels(device, monkeypatch, op, dtype):
    """``sparse_vecmat`` / ``sparse_mat_t_vec`` with a shared matrix operand and channel counts that are multiples of
    4 run on the table-driven matrix-core kernels, and so do their gradients (vector operand: the same kernel with
    the matrix transposed; matrix operand: the outer product summed over the rows); the route is asserted, results
    against the dense contraction in float64.  The table is a random one (11 output rows, 9 vector rows, 6
    matrices, 60 entries, one output row without entries)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.ops import kernels
    from equitorch_amd.structs import SparseProductInfo
    ax1, ax2, axo, eq = MAT[op]
    g = torch.Generator().manual_seed(stable_seed(op, str(dtype)))
    n, n_out, ext = 203, 11, {"u": 24, "w": 16}
    size = {"vecmat": (9, 6), "mat_t_vec": (6, 9)}[op]
    nnz = 60
    out_idx = torch.sort(torch.randint(0, n_out - 1, (nnz,), generator=g)).values     # row 10 stays empty
    seg = torch.searchsorted(out_idx, torch.arange(n_out + 1))
    i1, i2 = (torch.randint(0, sz, (nnz,), generator=g) for sz in size)
    scale = torch.randn(nnz, generator=g)
    info = SparseProductInfo(scale, i1, i2, seg, None, None, n_out).to(device)
    T = torch.zeros(n_out, *size, dtype=torch.float64)
    T.index_put_((out_idx, i1, i2), scale.double(), accumulate=True)
    shared = {"vecmat": (False, True), "mat_t_vec": (True, False)}[op]

    def mk(axes, sh, d):
        return torch.randn(*((() if sh else (n,)) + (d,) + tuple(ext[a] for a in axes)), generator=g,
                           dtype=torch.float64)
    x, y = mk(ax1, shared[0], size[0]), mk(ax2, shared[1], size[1])
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op_, tier, detail="": seen.append(tier))
    xd, yd = (t.to(dtype).to(device).requires_grad_(True) for t in (x, y))
    out = getattr(F, f"sparse_{op}")(xd, yd, info)
    eq = eq.format(a="" if shared[0] else "n", b="" if shared[1] else "n", o="n")
    ct = None

    def dense(dt):      # (out, grad1, grad2) of the dense contraction carried out in ``dt``
        nonlocal ct
        xr, yr = (t.to(dtype).detach().to(dt).clone().requires_grad_(True) for t in (x, y))
        o = torch.einsum(eq, T.to(dt), xr, yr)
        if ct is None:
            ct = torch.randn(o.shape, generator=g, dtype=torch.float64).to(dtype)
        return (o, *torch.autograd.grad(o, (xr, yr), ct.to(dt)))
    ref_out, rgx, rgy = dense(torch.float64)
    r32 = dense(torch.float32) if dtype == torch.float32 else (None, None, None)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    # sums over 16 or 24 channels and several entries per element: norm-wise in fp32, and against fp32 arithmetic
    assert_close(out, ref_out, tol, f"{op} forward", norm="max", fp32_ref=r32[0])
    assert out[:, n_out - 1].abs().max().item() == 0.0
    gx, gy = torch.autograd.grad(out, (xd, yd), ct.to(device))
    assert_close(gx, rgx, tol, f"{op} grad1", norm="max", fp32_ref=r32[1])
    assert_close(gy, rgy, tol, f"{op} grad2", norm="max", fp32_ref=r32[2])
    assert sum("shared matrix" in t for t in seen) == 2, seen          # forward and the vector operand's gradient
    assert sum("summed over rows" in t for t in seen) == 1, seen       # the matrix operand's gradient


@pytest.mark.parametrize("case", range(16))
def test_matrix_core_route_random_shapes(device, case):
    """The same route on seeded random tables and extents: batches below and across the 16-sample blocks (1 .. 700
    rows), channel counts from 4 that are no multiples of 16, weight paths and output rows without entries, repeated
    (row, row, path) entries, fp32 and fp64; forward and both gradients against the dense contraction in float64."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.structs import SparseProductInfo
    g = torch.Generator().manual_seed(stable_seed("matrix core route", case))
    ri = lambda lo, hi: int(torch.randint(lo, hi + 1, (1,), generator=g))
    dtype = torch.float64 if case % 4 == 3 else torch.float32
    n = [1, 15, 16, 17, 33, 100, 257, 700][case % 8]
    n_out, d_vec, n_mat = ri(1, 12), ri(1, 10), ri(1, 7)
    cu, cw = 4 * ri(1, 10), 4 * ri(1, 10)
    nnz = ri(1, 50)
    out_idx = torch.sort(torch.randint(0, n_out, (nnz,), generator=g)).values
    seg = torch.searchsorted(out_idx, torch.arange(n_out + 1))
    i1 = torch.randint(0, d_vec, (nnz,), generator=g)
    i2 = torch.randint(0, n_mat, (nnz,), generator=g)
    scale = torch.randn(nnz, generator=g)
    info = SparseProductInfo(scale, i1, i2, seg, None, None, n_out).to(device)
    T = torch.zeros(n_out, d_vec, n_mat, dtype=torch.float64)
    T.index_put_((out_idx, i1, i2), scale.double(), accumulate=True)
    x = torch.randn(n, d_vec, cu, generator=g, dtype=torch.float64).to(dtype)
    m = torch.randn(n_mat, cu, cw, generator=g, dtype=torch.float64).to(dtype)
    xd, md = (t.to(device).requires_grad_(True) for t in (x, m))
    out = F.sparse_vecmat(xd, md, info)
    ct = torch.randn(n, n_out, cw, generator=g, dtype=torch.float64).to(dtype)

    def dense(dt):      # (out, grad vector, grad matrix) of the dense contraction carried out in ``dt``
        xr, mr = (t.detach().to(dt).clone().requires_grad_(True) for t in (x, m))
        o = torch.einsum("mab,nau,buw->nmw", T.to(dt), xr, mr)
        return (o, *torch.autograd.grad(o, (xr, mr), ct.to(dt)))
    ref_out, rgx, rgm = dense(torch.float64)
    r32 = dense(torch.float32) if dtype == torch.float32 else (None, None, None)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    what = f"case {case}: n={n} out={n_out} rows={d_vec} paths={n_mat} {cu}->{cw} nnz={nnz} {dtype}"
    # sums over up to 40 channels and several entries per element, and over the batch for the matrix: norm-wise, and
    # against what the same contraction loses in fp32
    assert_close(out, ref_out, tol, what + " forward", norm="max", fp32_ref=r32[0])
    gx, gm = torch.autograd.grad(out, (xd, md), ct.to(device))
    assert_close(gx, rgx, tol, what + " grad vector", norm="max", fp32_ref=r32[1])
    assert_close(gm, rgm, tol, what + " grad matrix", norm="max", fp32_ref=r32[2])


@pytest.mark.parametrize("scaled,indexed,segmented", [(True, True, True), (False, True, True), (True, False, True),
                                                      (True, True, False), (False, False, False)])
def test_indexed_scale_segment(device, scaled, indexed, segmented):
    from equitorch_amd.ops import indexed_scale_segment
    g = torch.Generator().manual_seed(3)
    n, in_size, c, n_out = 3, 50, 37, 11
    x = torch.randn(n, in_size, c, generator=g)
    if segmented:
        counts = torch.randint(0, 9, (n_out,), generator=g)
        seg = torch.cat([torch.zeros(1, dtype=torch.int64), torch.cumsum(counts, 0)])
        t = int(seg[-1])
    else:
        seg, t = None, n_out
    index = torch.randint(0, in_size, (t,), generator=g) if indexed else None
    scale = torch.randn(t, generator=g) if scaled else None
    if not indexed:
        x = x[:, :t].contiguous()
    dev = lambda v: None if v is None else v.to(device)
    out = indexed_scale_segment(x.to(device), dev(scale), dev(index), dev(seg), out_size=n_out)
    ref = ref_ops.cpu_scale_segment(x.double(), None if scale is None else scale.double(), index, seg)
    assert_close(out, ref, 1e-5, "indexed_scale_segment")


@pytest.mark.parametrize("mode", ["u1v", "1vu", "vu1", "uvw", "uuu", "1uu", "uu1"])
@pytest.mark.parametrize("shared_w", [True, False])
def test_tensor_product_family_vs_dense(device, mode, shared_w):
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = "0e+1o+2e", "0e+1o+2e", "0e+1o"
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2)
    p = T.shape[0]
    g = torch.Generator().manual_seed(stable_seed(mode, shared_w))
    n, u, v, w = 29, 12, 5, 9
    shapes = {  # mode: (x channels, y channels, weight channels, einsum)
        "u1v": ((u,), (), (u, w), "pmab,nau,nb,{W}puw->nmw"), "1vu": ((), (u,), (u, w), "pmab,na,nbu,{W}puw->nmw"),
        "vu1": ((u,), (w,), (u, w), "pmab,nau,nbw,{W}puw->nm"), "uvw": ((u,), (v,), (u, v, w), "pmab,nau,nbv,{W}puvw->nmw"),
        "uuu": ((u,), (u,), (u,), "pmab,nau,nbu,{W}pu->nmu"), "1uu": ((), (u,), (u,), "pmab,na,nbu,{W}pu->nmu"),
        "uu1": ((u,), (u,), (u,), "pmab,nau,nbu,{W}pu->nm"),
    }
    cx, cy, cw, eq = shapes[mode]
    x = torch.randn(n, 9, *cx, generator=g, dtype=torch.float64)
    y = torch.randn(n, 4, *cy, generator=g, dtype=torch.float64)
    wt = torch.randn(*(() if shared_w else (n,)), p, *cw, generator=g, dtype=torch.float64)
    xd, yd, wd = (t.float().to(device).requires_grad_(True) for t in (x, y, wt))
    out = getattr(F, f"tensor_product_{mode}")(xd, yd, wd, *infos)
    xr, yr, wr = (t.float().double().requires_grad_(True) for t in (x, y, wt))
    oracle = {"u1v": ref_ops.dense_u1v, "uvw": ref_ops.dense_uvw, "uuu": ref_ops.dense_uuu}.get(mode)
    # the three members the oracle names directly (pinned on the CPU in tests/test_oracle_uv.py); the role-rotated
    # siblings are the same contraction with the channel axes on other operands
    ref_out = (oracle(T, xr, yr, wr) if oracle else
               torch.einsum(eq.format(W="" if shared_w else "n"), T, xr, yr, wr))
    assert_close(out, ref_out, 1e-5, f"{mode} forward")
    ct = torch.randn(ref_out.shape, generator=g, dtype=torch.float64)
    grads = torch.autograd.grad(out, (xd, yd, wd), ct.float().to(device))
    refs = torch.autograd.grad(ref_out, (xr, yr, wr), ct.float().double())
    for name, a, b in zip(("grad1", "grad2", "grad_w"), grads, refs):
        assert_close(a, b, 1e-5, f"{mode} {name}")


def test_modules_uv_uvw_and_gradgradcheck(device):
    """Module API for the fully connected modes, and second-order correctness (the reference checks gradcheck and
    gradgradcheck in float64 on 0e+1e+2e x 0e+1e+2e -> 0e+1e+2e+3e, test/test_tp/test_grad_tp.py:57-103)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.nn import SO3Linear, TensorProduct
    io, i1, i2 = "0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e"
    g = torch.Generator().manual_seed(1)
    n = 6
    for mode, ch in (("uu", (3, 3)), ("uv", (3, 4))):
        mod = SO3Linear(i1, i2, io, ch[0], ch[1], feature_mode=mode).to(device).double()
        x = torch.randn(n, 9, ch[0], generator=g, dtype=torch.float64).to(device).requires_grad_(True)
        y = torch.randn(n, 9, generator=g, dtype=torch.float64).to(device).requires_grad_(True)
        assert mod(x, y).shape == (n, 16, ch[1])
        op = getattr(F, "so3_linear_" + mode)
        fn = lambda x, y, w: op(x, y, w, mod.tp_info_forward)
        w = mod.weight.detach().clone().requires_grad_(True)
        assert torch.autograd.gradcheck(fn, (x, y, w), eps=1e-6, atol=1e-5, rtol=1e-5, nondet_tol=1e-9)
        assert torch.autograd.gradgradcheck(fn, (x, y, w), eps=1e-6, atol=1e-5, rtol=1e-5, nondet_tol=1e-9)
    for mode, ch in (("uuu", (3, 3, 3)), ("uvw", (3, 2, 4))):
        mod = TensorProduct(i1, i2, io, *ch, feature_mode=mode).to(device).double()
        x = torch.randn(n, 9, ch[0], generator=g, dtype=torch.float64).to(device).requires_grad_(True)
        y = torch.randn(n, 9, ch[1], generator=g, dtype=torch.float64).to(device).requires_grad_(True)
        assert mod(x, y).shape == (n, 16, ch[2])
        tp = getattr(F, "tensor_product_" + mode)
        w = mod.weight.detach().clone().requires_grad_(True)
        fn = lambda x, y, w: tp(x, y, w, mod.tp_info_forward)
        assert torch.autograd.gradcheck(fn, (x, y, w), eps=1e-6, atol=1e-5, rtol=1e-5, nondet_tol=1e-9)
        assert torch.autograd.gradgradcheck(fn, (x, y, w), eps=1e-6, atol=1e-5, rtol=1e-5, nondet_tol=1e-9)


@pytest.mark.parametrize("lmax,cin,cout,n", [(1, 32, 32, 70), (2, 64, 128, 100), (3, 128, 128, 257), (3, 128, 64, 33),
                                             (3, 128, 128, 1100), (2, 32, 64, 700)])
def test_uv_mfma_bf16(device, lmax, cin, cout, n):
    """bf16 matrix-core path of SO3Linear('uv'): forward and all gradients against the dense float64 oracle
    evaluated on the bf16-rounded inputs; tolerance rel 1e-2 of the tensor's largest magnitude (bf16 output)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import _uvw_mfma
    from equitorch_amd.utils._sh import spherical_harmonics
    from helpers import unit_vectors
    irreps = "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))
    mod = SO3Linear(irreps, irreps, irreps, cin, cout, internal_weights=False, feature_mode="uv").to(device)
    assert _uvw_mfma.uv_config_of(mod.tp_info_forward) >= 0
    d = (lmax + 1) ** 2
    g = torch.Generator().manual_seed(lmax * 1000 + cin + cout)
    x = torch.randn(n, d, cin, generator=g).bfloat16()
    y = spherical_harmonics(unit_vectors(n, g), lmax).bfloat16()
    w = (torch.randn(mod.num_paths, cin, cout, generator=g) / (cin * mod.num_paths) ** 0.5).bfloat16()
    ct = torch.randn(n, d, cout, generator=g).bfloat16()
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = mod(xd, yd, wd)
    assert out.dtype == torch.bfloat16
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    T = ref_ops.dense_coupling(irreps, irreps, irreps).float().double()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads)):
        a, b = a.detach().double().cpu(), b.double()
        err = float((a - b).abs().max())
        assert err <= 1e-2 * float(b.abs().max()), f"lmax={lmax} {name}: max abs err {err:.3e} vs scale {float(b.abs().max()):.3e}"


@pytest.mark.parametrize("kw", [{"path_norm": False}, {"channel_norm": True},
                                {"channel_norm": True, "path_norm": False}])
def test_uv_mfma_bf16_normalisation_options(device, kw):
    """``channel_norm=True`` (the reference's channel-normalised comparison test) and ``path_norm=False`` only
    rescale the coefficients of a path: the bf16 matrix-core kernels must still be selected (the factors are folded
    into the packed weights and into the weight gradient), and agree with the dense oracle built with those options."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import _uvw_mfma
    from equitorch_amd.utils._sh import spherical_harmonics
    from helpers import unit_vectors
    lmax, cin, cout, n = 3, 64, 128, 300
    irreps = "0e+1o+2e+3o"
    mod = SO3Linear(irreps, irreps, irreps, cin, cout, internal_weights=False, feature_mode="uv", **kw).to(device)
    cfg = _uvw_mfma.uv_config_of(mod.tp_info_forward)
    assert cfg >= 0 and cfg.path_scale is not None
    g = torch.Generator().manual_seed(21)
    x = torch.randn(n, 16, cin, generator=g).bfloat16()
    y = spherical_harmonics(unit_vectors(n, g), lmax).bfloat16()
    w = (torch.randn(mod.num_paths, cin, cout, generator=g) / mod.num_paths ** 0.5).bfloat16()
    ct = torch.randn(n, 16, cout, generator=g).bfloat16()
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    assert _uvw_mfma.try_forward(xd.detach(), yd.detach(), wd.detach(), mod.tp_info_forward) is not None
    out = mod(xd, yd, wd)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    T = ref_ops.dense_coupling(irreps, irreps, irreps, path_norm=kw.get("path_norm", True),
                               channel_norm=kw.get("channel_norm", False), channel_scale=cin ** -0.5).float().double()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_sh", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads)):
        a, b = a.detach().double().cpu(), b.double()
        err = float((a - b).abs().max())
        assert err <= 1e-2 * float(b.abs().max()), f"{kw} {name}: max abs err {err:.3e} vs {float(b.abs().max()):.3e}"


def test_uv_mfma_full_size_properties(device):
    """BASELINE configs[3] shapes (B = 32768, lmax = 3, C = 128, bf16).  The dense oracle is run on a strided
    subset of the rows for out / grad_x / grad_sh (each row depends on its own sample only); the weight gradient
    sums over the batch, so it is checked through additivity over two halves of the batch (bf16 rounding of the
    three results bounds the difference) and against the oracle's sum over the subset when the other rows'
    output gradients are zero."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.utils._sh import spherical_harmonics
    from helpers import unit_vectors
    lmax, ch, n = 3, 128, 32768
    irreps = "0e+1o+2e+3o"
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(n, 16, ch, generator=g).bfloat16()
    y = spherical_harmonics(unit_vectors(n, g), lmax).bfloat16()
    w = (torch.randn(mod.num_paths, ch, ch, generator=g) / (ch * mod.num_paths) ** 0.5).bfloat16()
    ct = torch.randn(n, 16, ch, generator=g).bfloat16()
    sub = torch.arange(5, n, 257)                      # 128 rows spread over all chunks
    mask = torch.zeros(n, 1, 1, dtype=torch.bfloat16)
    mask[sub] = 1
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = mod(xd, yd, wd)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    T = ref_ops.dense_coupling(irreps, irreps, irreps).float().double()
    ref_out, (rgx, rgy, rgw_sub) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub])
    for name, a, b in (("out", out[sub.to(device)], ref_out), ("grad_x", gx[sub.to(device)], rgx),
                       ("grad_sh", gy[sub.to(device)], rgy)):
        a, b = a.detach().double().cpu(), b.double()
        assert float((a - b).abs().max()) <= 1e-2 * float(b.abs().max()), name
    # weight gradient restricted to the subset (all other output gradients zero) against the oracle
    out = mod(xd, yd, wd)
    (gw_sub,) = torch.autograd.grad(out, (wd,), (ct * mask).to(device))
    a, b = gw_sub.double().cpu(), rgw_sub.double()
    assert float((a - b).abs().max()) <= 1e-2 * float(b.abs().max())
    # additivity over the batch
    half = n // 2
    parts = []
    for lo, hi in ((0, half), (half, n)):
        xs, ys = xd[lo:hi].detach(), yd[lo:hi].detach()
        ws = wd.detach().requires_grad_(True)
        (gp,) = torch.autograd.grad(mod(xs, ys, ws), (ws,), ct[lo:hi].to(device))
        parts.append(gp.double())
    scale = float(gw.double().abs().max())
    assert float((gw.double() - parts[0] - parts[1]).abs().max()) <= 2e-2 * scale


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("channels", [(8, 16, 4), (32, 32, 8), (6, 20, 5)])
def test_uvw_on_the_two_operand_kernels(device, dtype, channels):
    """``tensor_product_uvw`` on enough rows for the outer-product and contraction kernels of the two-axis family
    (16-byte lanes along the contiguous axis; (6, 20, .): 5 lanes per row do not divide the workgroup, the general
    kernel runs): forward and all three gradients against the dense einsum, shared weight."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = "0e+1o+2e", "0e+1o+2e", "0e+1o"
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()      # the tables hold fp32 coefficients
    p = T.shape[0]
    g = torch.Generator().manual_seed(7)
    n = 301
    u, v, w = channels
    x = torch.randn(n, 9, u, generator=g, dtype=torch.float64).to(dtype).double()
    y = torch.randn(n, 4, v, generator=g, dtype=torch.float64).to(dtype).double()
    wt = (torch.randn(p, u, v, w, generator=g, dtype=torch.float64) / (u * v) ** 0.5).to(dtype).double()
    xd, yd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, y, wt))
    out = F.tensor_product_uvw(xd, yd, wd, *infos)
    xr, yr, wr = (t.clone().requires_grad_(True) for t in (x, y, wt))
    ref_out = torch.einsum("pmab,nau,nbv,puvw->nmw", T, xr, yr, wr)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    assert_close(out, ref_out, tol, "uvw forward")
    ct = torch.randn(ref_out.shape, generator=g, dtype=torch.float64).to(dtype).double()
    grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device, dtype))
    refs = torch.autograd.grad(ref_out, (xr, yr, wr), ct)
    for name, a, b in zip(("grad1", "grad2", "grad_w"), grads, refs):
        assert_close(a, b, tol * 10, f"uvw {name}")
