"""Fully connected products with a weight per sample (``cgtp_psw_fwd`` / ``cgtp_psw_bwd``: one streaming launch each way,
no library GEMM, no intermediate in memory) against the dense float64 oracle: u1v, 1vu, uvw and the channel mixing
between irreps, forward and all first-order gradients.  The reference takes a weight with a batch axis through its
table-driven kernels like a shared one (``equitorch/nn/tensor_products.py:152-155``,
``equitorch/nn/functional/linears.py:254-412``).  While the product and its backward run, ``torch.matmul`` / ``bmm``
/ ``baddbmm`` raise."""
import pytest
import torch

from helpers import assert_close, fp32_twin, stable_seed
from oracle import ref_ops

pytestmark = pytest.mark.gpu


def _sh(lmax):
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


@pytest.fixture
def no_library_gemm():
    """Context manager: inside it ``torch.matmul`` / ``bmm`` / ``baddbmm`` / ``einsum`` raise."""
    import contextlib

    @contextlib.contextmanager
    def guard():
        def refuse(*a, **k):
            raise AssertionError("a library GEMM was called")
        names = ("matmul", "bmm", "baddbmm", "einsum")
        saved = {name: getattr(torch, name) for name in names}
        for name in names:
            setattr(torch, name, refuse)
        try:
            yield
        finally:
            for name, fn in saved.items():
                setattr(torch, name, fn)
    return guard


def _tiers(monkeypatch):
    from equitorch_amd.ops import kernels
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    return seen


U1V = [  # irreps (out, in1, in2), C_in, C_out, N, dtype
    ((_sh(2),) * 3, 32, 32, 300, torch.float32),          # 8 lanes a row, one sample a wavefront, 8 row slices
    ((_sh(2),) * 3, 16, 16, 20000, torch.float32),        # several samples a wavefront
    ((_sh(3),) * 3, 64, 64, 70, torch.float32),           # blocks of 7 rows
    ((_sh(2),) * 3, 5, 20, 129, torch.float32),           # 5 lanes of 4 channels, C_in below a chunk
    ((_sh(2),) * 3, 33, 7, 1000, torch.float32),          # one channel a lane, chunks of 32 + 1
    ((_sh(1),) * 3, 100, 128, 77, torch.float32),         # 32 lanes a row, chunks of 64 + 36
    ((_sh(1),) * 3, 8, 256, 40, torch.float32),           # a row over the whole wavefront
    (("1o+2e+1e", "0e+1o+2e", "0e+1o"), 24, 40, 200, torch.float32),
    (("2x0e+1o+1e", "0e+2x1o", "0e+1o+1e"), 12, 12, 64, torch.float32),
    (("0e+4e", "2e+3o", "2e+3o"), 8, 16, 50, torch.float32),      # a block of 9 rows: the 16-row pass
    ((_sh(2),) * 3, 32, 32, 300, torch.float64),
    ((_sh(3), _sh(2), _sh(3)), 20, 6, 45, torch.float64),
]


@pytest.mark.parametrize("irreps,cin,cout,n,dtype", U1V)
def test_u1v_per_sample_weight(device, monkeypatch, no_library_gemm, irreps, cin, cout, n, dtype):
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = irreps
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    g = torch.Generator().manual_seed(stable_seed("psw u1v", irreps, cin, cout, n))
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    x, y, w = rd(n, T.shape[2], cin), rd(n, T.shape[3]), rd(n, T.shape[0], cin, cout) / cin ** 0.5
    ct = rd(n, T.shape[1], cout)
    seen = _tiers(monkeypatch)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    with no_library_gemm():
        out = F.tensor_product_u1v(xd, yd, wd, *infos)
        grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    assert seen and "per-sample weight streaming" in seen[-1], seen
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    twin = (None,) * 4
    if dtype == torch.float32:
        o32, g32 = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct, dtype=torch.float32)
        twin = (o32, *g32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), twin):
        assert_close(a, b, tol, f"u1v per-sample {io} {cin}->{cout} N={n} {dtype} {name}", norm="max", fp32_ref=b32)


@pytest.mark.parametrize("irreps,cin,cout,n", [((_sh(2),) * 3, 32, 32, 300), (("1o+2e+1e", "0e+1o", "0e+1o+2e"), 10, 24, 99)])
def test_1vu_per_sample_weight(device, monkeypatch, no_library_gemm, irreps, cin, cout, n):
    """The channels on the second operand: the same kernels with the operands' places exchanged."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = irreps
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    g = torch.Generator().manual_seed(stable_seed("psw 1vu", irreps, cin, cout, n))
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).float()
    x, y, w = rd(n, T.shape[2]), rd(n, T.shape[3], cin), rd(n, T.shape[0], cin, cout) / cin ** 0.5
    ct = rd(n, T.shape[1], cout)
    seen = _tiers(monkeypatch)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    with no_library_gemm():
        out = F.tensor_product_1vu(xd, yd, wd, *infos)
        grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    assert seen and "per-sample weight streaming" in seen[-1], seen

    def dense_1vu(T, x, y, w, dtype=torch.float64):
        return ref_ops.dense_u1v(T.transpose(2, 3), y, x, w, dtype=dtype)
    ref_out, ref_grads = ref_ops.dense_grads(dense_1vu, T, (x, y, w), ct)
    o32, g32 = ref_ops.dense_grads(dense_1vu, T, (x, y, w), ct, dtype=torch.float32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), (o32, *g32)):
        assert_close(a, b, 1e-5, f"1vu per-sample {io} {cin}->{cout} {name}", norm="max", fp32_ref=b32)


UVW = [  # irreps, U, V, C_out, N, dtype
    ((_sh(2), _sh(2), "0e+1o"), 16, 8, 12, 301, torch.float32),      # chunks of 8 u
    ((_sh(1),) * 3, 4, 64, 32, 90, torch.float32),                   # chunks of one u
    ((_sh(2),) * 3, 6, 3, 5, 2000, torch.float32),                   # chunks of 21 u > U, one channel a lane
    ((_sh(1),) * 3, 3, 100, 16, 33, torch.float32),                  # V beyond the lanes of a sample
    ((_sh(2), _sh(2), "0e+1o"), 8, 8, 8, 64, torch.float64),
]


@pytest.mark.parametrize("irreps,u,v,cout,n,dtype", UVW)
def test_uvw_per_sample_weight(device, monkeypatch, no_library_gemm, irreps, u, v, cout, n, dtype):
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = irreps
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    g = torch.Generator().manual_seed(stable_seed("psw uvw", irreps, u, v, cout, n))
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    x, y, w = rd(n, T.shape[2], u), rd(n, T.shape[3], v), rd(n, T.shape[0], u, v, cout) / (u * v) ** 0.5
    ct = rd(n, T.shape[1], cout)
    seen = _tiers(monkeypatch)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    with no_library_gemm():
        out = F.tensor_product_uvw(xd, yd, wd, *infos)
        grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    assert seen and "per-sample weight streaming" in seen[-1], seen
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_uvw, T, (x, y, w), ct)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    twin = (None,) * 4
    if dtype == torch.float32:
        o32, g32 = ref_ops.dense_grads(ref_ops.dense_uvw, T, (x, y, w), ct, dtype=torch.float32)
        twin = (o32, *g32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), twin):
        assert_close(a, b, tol, f"uvw per-sample {io} {u}x{v}->{cout} N={n} {dtype} {name}", norm="max", fp32_ref=b32)


def test_only_some_gradients(device, no_library_gemm):
    """Operands that need no gradient: the backward forms only what is asked for."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr = _sh(2)
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator().manual_seed(3)
    n, cin, cout = 150, 16, 24
    x, y, w, ct = (torch.randn(*s, generator=g) for s in ((n, 9, cin), (n, 9), (n, T.shape[0], cin, cout), (n, 9, cout)))
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for need in ((True, False, False), (False, True, False), (False, False, True), (True, True, False)):
        leaves = [t.to(device).requires_grad_(r) for t, r in zip((x, y, w), need)]
        with no_library_gemm():
            out = F.tensor_product_u1v(*leaves, *infos)
            grads = torch.autograd.grad(out, [t for t, r in zip(leaves, need) if r], ct.to(device))
        for a, b in zip(grads, [b for b, r in zip(ref_grads, need) if r]):
            assert_close(a, b, 1e-5, f"u1v per-sample, gradients {need}", norm="max")


def test_second_order_goes_through_the_differentiable_route(device):
    """A gradient of the gradient: the backward re-expresses the product through differentiable pieces."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr = _sh(1)
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator().manual_seed(5)
    n, cin, cout = 20, 8, 8
    x, y, w, ct = (torch.randn(*s, generator=g, dtype=torch.float64)
                   for s in ((n, 4, cin), (n, 4), (n, T.shape[0], cin, cout), (n, 4, cout)))

    def second(fn, x, y, w, ct):
        x, y, w = (t.clone().requires_grad_(True) for t in (x, y, w))
        gx, = torch.autograd.grad(fn(x, y, w), x, ct, create_graph=True)
        return torch.autograd.grad(gx.square().sum(), (y, w))
    got = second(lambda a, b, c: F.tensor_product_u1v(a, b, c, *infos), *(t.to(device) for t in (x, y, w, ct)))
    ref = second(lambda a, b, c: ref_ops.dense_u1v(T, a, b, c), x, y, w, ct)
    for name, a, b in zip(("d/dy", "d/dw"), got, ref):
        assert_close(a, b, 1e-11, f"u1v per-sample second order {name}", norm="max")


@pytest.mark.parametrize("io,ii,dtype", [("0e+1o+2e", "0e+1o+1o+2e+0e", torch.float32),
                                         ("2x0e+1o+3x2e", "0e+2x1o+2e+3e", torch.float32),
                                         ("0e+1o", "0e+1e+2e", torch.float64)])
def test_channel_mixing_per_sample_weight(device, monkeypatch, no_library_gemm, io, ii, dtype):
    """``IrrepsLinear`` with a weight per sample: the same kernels with the scalar 1 as second operand (several input
    irreps feeding one output irrep share its rows; an output irrep without a source stays zero)."""
    from equitorch_amd.nn import IrrepsLinear
    from oracle import ref_tables
    n, cin, cout = 210, 24, 40
    mod = IrrepsLinear(ii, io, cin, cout, internal_weights=False).to(device)
    info = ref_tables.irreps_linear_infos(io, ii)[0]
    info["scale_MM0"] = torch.tensor(info["scale_MM0"]).double().tolist()    # the tables hold fp32 values
    g = torch.Generator().manual_seed(8)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
    x, w, ct = rd(n, mod.irreps_in_dim, cin), rd(n, mod.num_paths, cin, cout), rd(n, mod.irreps_out_dim, cout)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irreps_linear(xr, wr, info)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    seen = _tiers(monkeypatch)
    xd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, w))
    with no_library_gemm():
        out = mod(xd, wd)
        gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device, dtype))
    assert seen and "per-sample weight streaming" in seen[-1], seen
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert_close(a, b, tol, f"IrrepsLinear per-sample {io}<-{ii} {dtype} {name}")


def test_irrep_wise_per_sample_weight(device, monkeypatch, no_library_gemm):
    from equitorch_amd.nn import IrrepWiseLinear
    from oracle import ref_tables
    irr, cin, cout, n = "0e+1o+2e+1o", 16, 8, 333
    mod = IrrepWiseLinear(irr, cin, cout, internal_weights=False).to(device)
    info = ref_tables.irreps_info(irr)
    g = torch.Generator().manual_seed(2)
    x, w, ct = (torch.randn(*s, generator=g, dtype=torch.float64) for s in ((n, 12, cin), (n, 4, cin, cout), (n, 12, cout)))
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irrep_wise_linear(xr, wr, info)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    seen = _tiers(monkeypatch)
    xd, wd = (t.to(device).requires_grad_(True) for t in (x, w))
    with no_library_gemm():
        out = mod(xd, wd)
        gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device))
    assert seen and "per-sample weight streaming" in seen[-1], seen
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert_close(a, b, 1e-12, f"IrrepWiseLinear per-sample {name}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_so2_linear_uv_per_sample_weight(device, monkeypatch, no_library_gemm, dtype):
    """``SO2Linear('uv')`` with a weight per sample: a weight couples the rows +m and -m of an output irrep, so the
    blocks of the walk are whole output irreps with most (path, row) pairs empty."""
    from equitorch_amd.nn import SO2Linear
    from oracle import ref_tables
    irr_in, irr_out, n, cin, cout = "0e+1o+2e+3o", "0e+1o+2e", 130, 8, 12
    info = ref_tables.so2_linear_infos(irr_out, irr_in)[0]
    info["scale"] = None if info.get("scale") is None else torch.tensor(info["scale"]).double().tolist()
    mod = SO2Linear(irr_in, irr_out, cin, cout, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator().manual_seed(12)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
    x, w, ct = rd(n, 16, cin), rd(n, mod.num_weights, cin, cout), rd(n, 9, cout)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_so2_linear(xr, wr, info, per_sample=True)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    seen = _tiers(monkeypatch)
    xd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, w))
    with no_library_gemm():
        out = mod(xd, wd)
        gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device, dtype))
    assert seen and "per-sample weight streaming" in seen[-1], seen
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert_close(a, b, tol, f"SO2Linear uv per-sample {dtype} {name}")


@pytest.mark.parametrize("c1,c2,n,dtype", [(16, 8, 301, torch.float32), (5, 70, 64, torch.float32), (8, 8, 50, torch.float64)])
def test_vu1_per_sample_weight(device, monkeypatch, no_library_gemm, c1, c2, n, dtype):
    """``out[n,M] = sum c x[n,a,u] W[n,p,u,w] y[n,b,w]``: the uvw product with a single output channel — a weight row is
    one element, the lanes of a sample run over the rows."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = _sh(2), _sh(2), "0e+1o"
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    g = torch.Generator().manual_seed(stable_seed("psw vu1", c1, c2, n))
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    x, y, w, ct = rd(n, 9, c1), rd(n, 4, c2), rd(n, T.shape[0], c1, c2) / (c1 * c2) ** 0.5, rd(n, 9)

    def dense_vu1(T, x, y, w, dtype=torch.float64):
        return ref_ops.dense_uvw(T, x, y, w.unsqueeze(-1), dtype=dtype).squeeze(-1)
    seen = _tiers(monkeypatch)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    with no_library_gemm():
        out = F.tensor_product_vu1(xd, yd, wd, *infos)
        grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    assert seen and "per-sample weight streaming" in seen[-1], seen
    ref_out, ref_grads = ref_ops.dense_grads(dense_vu1, T, (x, y, w), ct)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    twin = (None,) * 4
    if dtype == torch.float32:
        o32, g32 = ref_ops.dense_grads(dense_vu1, T, (x, y, w), ct, dtype=torch.float32)
        twin = (o32, *g32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), twin):
        assert_close(a, b, tol, f"vu1 per-sample {c1}x{c2} N={n} {dtype} {name}", norm="max", fp32_ref=b32)


@pytest.mark.parametrize("n", [1, 2, 63, 4097])
def test_sample_counts_at_the_edges_of_a_wavefront(device, monkeypatch, no_library_gemm, n):
    """One sample, fewer samples than a wavefront takes, and a count that leaves the last wavefront partly empty
    (16 -> 8 channels: 16 samples a wavefront at 4097)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr = _sh(2)
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator().manual_seed(n)
    x, y, w, ct = (torch.randn(*s, generator=g) for s in ((n, 9, 16), (n, 9), (n, T.shape[0], 16, 8), (n, 9, 8)))
    seen = _tiers(monkeypatch)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    with no_library_gemm():
        out = F.tensor_product_u1v(xd, yd, wd, *infos)
        grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    assert "per-sample weight streaming" in seen[-1], seen
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads)):
        assert_close(a, b, 1e-5, f"u1v per-sample N={n} {name}", norm="max")


def test_no_samples_and_operands_the_kernels_do_not_take(device, monkeypatch):
    """An empty batch, a weight view that is not contiguous, and more output channels than a wavefront covers: the
    product still returns the right result (an empty tensor; a copy; the library route)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr = _sh(1)
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    p = T.shape[0]
    out = F.tensor_product_u1v(torch.zeros(0, 4, 8, device=device), torch.zeros(0, 4, device=device),
                               torch.zeros(0, p, 8, 8, device=device), *infos)
    assert out.shape == (0, 4, 8)
    g = torch.Generator().manual_seed(0)
    n = 33
    x, y = torch.randn(n, 4, 8, generator=g), torch.randn(n, 4, generator=g)
    w_t = torch.randn(n, p, 12, 8, generator=g)                    # the product sees its transpose: a strided view
    seen = _tiers(monkeypatch)
    out = F.tensor_product_u1v(x.to(device), y.to(device), w_t.to(device).transpose(2, 3), *infos)
    assert "per-sample weight streaming" in seen[-1], seen
    assert_close(out, ref_ops.dense_u1v(T, x, y, w_t.transpose(2, 3)), 1e-5, "u1v per-sample, strided weight", norm="max")
    w_wide = torch.randn(n, p, 8, 260, generator=g)                # 260 channels: beyond 64 lanes of four
    out = F.tensor_product_u1v(x.to(device), y.to(device), w_wide.to(device), *infos)
    assert "per-sample weight streaming" not in seen[-1], seen
    assert_close(out, ref_ops.dense_u1v(T, x, y, w_wide), 1e-5, "u1v per-sample, 260 output channels", norm="max")


def test_weights_beyond_the_last_level_cache(device, monkeypatch, no_library_gemm):
    """1.08 GB of per-sample weights (N = 24 000, 32 -> 32 channels): the launcher then keeps four rows of W per lane
    in flight in the backward.  Samples are independent, so a strided subset of them is compared with the dense
    oracle evaluated on exactly those samples (output, and every gradient including the subset's rows of grad_W)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr, n, ch = _sh(2), 24000, 32
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator(device=device).manual_seed(1)
    x = torch.randn(n, 9, ch, device=device, generator=g).requires_grad_(True)
    y = torch.randn(n, 9, device=device, generator=g).requires_grad_(True)
    w = (torch.randn(n, T.shape[0], ch, ch, device=device, generator=g) / ch ** 0.5).requires_grad_(True)
    ct = torch.randn(n, 9, ch, device=device, generator=g)
    assert w.numel() * 4 > 256 << 20
    seen = _tiers(monkeypatch)
    with no_library_gemm():
        out = F.tensor_product_u1v(x, y, w, *infos)
        grads = torch.autograd.grad(out, (x, y, w), ct)
    assert "per-sample weight streaming" in seen[-1], seen
    rows = torch.arange(5, n, 371, device=device)
    sub = lambda t: t.detach()[rows].cpu()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (sub(x), sub(y), sub(w)), sub(ct))
    o32, g32 = ref_ops.dense_grads(ref_ops.dense_u1v, T, (sub(x), sub(y), sub(w)), sub(ct), dtype=torch.float32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), (o32, *g32)):
        assert_close(sub(a), b, 1e-5, f"u1v per-sample, 1.08 GB of weights, {name}", norm="max", fp32_ref=b32)


def test_gradcheck_and_gradgradcheck_with_a_weight_per_sample(device):
    """The reference checks ``gradcheck`` and ``gradgradcheck`` of all four modes with shared and with per-sample
    weights in float64 (``test/test_tp/test_grad_tp.py:57-103``, ``0e+1e+2e x 0e+1e+2e -> 0e+1e+2e+3e``); here for
    the weight per sample: first order on the streaming kernels (uv, uvw) and the compiled / table-driven kernels
    (uu, uuu), second order through the differentiable route behind them."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = "0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e"
    info = tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[0].to(device)
    from equitorch_amd.ops import kernels
    p = kernels.coo_of(info).P
    g = torch.Generator().manual_seed(2)
    n = 5
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(device).requires_grad_(True)
    cases = (("u1u", F.tensor_product_u1u, rd(n, 9, 3), rd(n, 9), rd(n, p, 3)),
             ("u1v", F.tensor_product_u1v, rd(n, 9, 3), rd(n, 9), rd(n, p, 3, 4)),
             ("uuu", F.tensor_product_uuu, rd(n, 9, 3), rd(n, 9, 3), rd(n, p, 3)),
             ("uvw", F.tensor_product_uvw, rd(n, 9, 3), rd(n, 9, 2), rd(n, p, 3, 2, 4)))
    for name, op, x, y, w in cases:
        fn = lambda x, y, w: op(x, y, w, info)
        assert fn(x, y, w).shape[:2] == (n, 16), name
        assert torch.autograd.gradcheck(fn, (x, y, w), eps=1e-6, atol=1e-5, rtol=1e-5, nondet_tol=1e-9), name
        assert torch.autograd.gradgradcheck(fn, (x, y, w), eps=1e-6, atol=1e-5, rtol=1e-5, nondet_tol=1e-9), name


def test_weight_tensor_past_two_to_the_31_elements(device, monkeypatch, no_library_gemm):
    """N = 70 000 samples, 64 -> 64 channels, lmax = 2: the per-sample weight has 3.15e9 elements (12.6 GB), so every
    offset into it and into its gradient past sample 47 662 exceeds 32 bits.  Samples from the far end, and a strided
    subset, against the dense oracle on exactly those samples."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    irr, n, ch = _sh(2), 70000, 64
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator(device=device).manual_seed(2)
    x = torch.randn(n, 9, ch, device=device, generator=g).requires_grad_(True)
    y = torch.randn(n, 9, device=device, generator=g).requires_grad_(True)
    w = torch.randn(n, T.shape[0], ch, ch, device=device, generator=g).mul_(ch ** -0.5).requires_grad_(True)
    ct = torch.randn(n, 9, ch, device=device, generator=g)
    assert w.numel() > 2 ** 31
    seen = _tiers(monkeypatch)
    with no_library_gemm():
        out = F.tensor_product_u1v(x, y, w, *infos)
        gx, gy, gw = torch.autograd.grad(out, (x, y, w), ct)
    assert "per-sample weight streaming" in seen[-1], seen
    rows = torch.cat([torch.arange(3, n, 5000, device=device), torch.arange(n - 8, n, device=device)])
    sub = lambda t: t.detach()[rows].cpu()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (sub(x), sub(y), sub(w)), sub(ct))
    o32, g32 = ref_ops.dense_grads(ref_ops.dense_u1v, T, (sub(x), sub(y), sub(w)), sub(ct), dtype=torch.float32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads), (o32, *g32)):
        assert_close(sub(a), b, 1e-5, f"u1v per-sample, 3.15e9 weights, {name}", norm="max", fp32_ref=b32)
    del w, gw
    torch.cuda.empty_cache()
