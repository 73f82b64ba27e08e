"""GPU parity of the fully connected products in fp32 on the table-driven matrix-core kernels (``cgtp_uvt_*``):
``SO3Linear('uv')`` / ``tensor_product_u1v`` and ``TensorProduct('uvw')`` / ``tensor_product_uvw`` with a shared
weight, forward and all first-order gradients, against the dense float64 oracle (pinned on the CPU in
tests/test_oracle_uv.py).  Results are sums over C_in (x C_2) channels and all paths of an output irrep of products
of N(0,1) numbers: compared norm-wise (1e-5 of the tensor's largest magnitude)."""
import pytest
import torch

from helpers import assert_close, unit_vectors
from oracle import ref_ops

pytestmark = pytest.mark.gpu


def _sh(lmax):
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


U1V_CASES = [  # irreps (out, in1, in2), C_in, C_out, N, module options
    ((_sh(1),) * 3, 32, 32, 70, {}),
    ((_sh(2),) * 3, 64, 128, 257, {}),
    ((_sh(3),) * 3, 128, 128, 300, {}),
    ((_sh(3),) * 3, 128, 64, 33, {"path_norm": False}),
    ((_sh(2),) * 3, 20, 12, 1100, {}),                          # C_in padded to 32, C_out below one block of 16
    ((_sh(2),) * 3, 32, 36, 515, {"channel_norm": True}),       # C_out = 2 blocks + 4
    (("1o+2e+1e", "0e+1o+2e", "0e+1o"), 48, 40, 200, {}),       # irreps without a compiled table
    (("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e"), 16, 16, 64, {}),
    (("0e", _sh(2), _sh(2)), 32, 64, 17000, {}),                # one output row: wavefronts spent on sample blocks
    (("0e+1o", _sh(1), _sh(1)), 16, 256, 530, {}),              # output channels over two workgroups
    ((_sh(2),) * 3, 8, 8, 515, {}),                             # a fragment ring of two blocks, half of it padding
    ((_sh(3), _sh(2), _sh(3)), 16, 40, 333, {}),                # ... one block of k, output channels 2 blocks + 8
    ((_sh(2),) * 3, 96, 80, 300, {}),                           # six blocks of k: a ring of two past 64 channels
    ((_sh(1), _sh(2), _sh(1)), 160, 96, 130, {}),               # ten blocks
    ((_sh(2),) * 3, 112, 48, 77, {}),                           # seven blocks: padded to eight, a ring of four
]


@pytest.mark.parametrize("irreps,cin,cout,n", [((_sh(2),) * 3, 64, 32, 300), ((_sh(2), _sh(3), _sh(2)), 32, 48, 70),
                                              (("1o+2e+1e", "0e+1o+2e", "0e+1o"), 20, 12, 515)])
def test_u1v_fp64_native(device, irreps, cin, cout, n):
    """The same kernels in double precision (v_mfma_f64_16x16x4_f64): forward and all gradients to 1e-11 of the
    tensor's largest magnitude (sums over C_in x paths products)."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import _uv_native
    io, i1, i2 = irreps
    mod = SO3Linear(i1, i2, io, cin, cout, internal_weights=False, feature_mode="uv").to(device)
    d1, d2, do = Irreps(i1).dim, Irreps(i2).dim, Irreps(io).dim
    g = torch.Generator().manual_seed(cin + cout + n)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x, y, w, ct = rd(n, d1, cin), rd(n, d2), rd(mod.num_paths, cin, cout) / cin ** 0.5, rd(n, do, cout)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    assert _uv_native.u1v_supported(xd, yd, wd, mod.tp_info_forward)
    out = mod(xd, yd, wd)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    T = ref_ops.dense_coupling(io, i1, i2, channel_scale=cin ** -0.5).float().double()   # tables hold fp32 coefficients
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads)):
        assert_close(a, b, 1e-11, f"u1v fp64 {io} C={cin}->{cout} N={n} {name}", norm="max")


def test_uvw_fp64_native(device):
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn.functional import _uv_native
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = _sh(2), _sh(2), "0e+1o"
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    u, v, wc, n = 16, 8, 12, 301
    g = torch.Generator().manual_seed(4)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    x, y, w, ct = rd(n, 9, u), rd(n, 4, v), rd(T.shape[0], u, v, wc) / (u * v) ** 0.5, rd(n, 9, wc)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    assert _uv_native.uvw_supported(xd, yd, wd, infos[0])
    out = F.tensor_product_uvw(xd, yd, wd, *infos)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_uvw, T, (x, y, w), ct)
    for name, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads)):
        assert_close(a, b, 1e-11, f"uvw fp64 {name}", norm="max")


@pytest.mark.parametrize("irreps,cin,cout,n,kw", U1V_CASES)
def test_u1v_fp32_native(device, irreps, cin, cout, n, kw):
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import _uv_native
    io, i1, i2 = irreps
    mod = SO3Linear(i1, i2, io, cin, cout, internal_weights=False, feature_mode="uv", **kw).to(device)
    d1, d2, do = Irreps(i1).dim, Irreps(i2).dim, Irreps(io).dim
    g = torch.Generator().manual_seed(cin * 1000 + cout + n)
    x = torch.randn(n, d1, cin, generator=g)
    y = torch.randn(n, d2, generator=g)
    w = torch.randn(mod.num_paths, cin, cout, generator=g) / cin ** 0.5
    ct = torch.randn(n, do, cout, generator=g)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    assert _uv_native.u1v_supported(xd, yd, wd, mod.tp_info_forward)
    out = mod(xd, yd, wd)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    T = ref_ops.dense_coupling(io, i1, i2, path_norm=kw.get("path_norm", True),
                               channel_norm=kw.get("channel_norm", False), channel_scale=cin ** -0.5).float().double()
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    out32, grads32 = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct, dtype=torch.float32)
    for name, a, b, r in zip(("out", "grad_x", "grad_y", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads),
                             (out32, *grads32)):
        # sums over C_in x paths products (the weight's over the batch too): norm-wise, and within three times what the
        # same contraction loses in fp32 arithmetic
        assert_close(a, b, 1e-5, f"u1v {io} C={cin}->{cout} N={n} {name}", norm="max", fp32_ref=r)


UVW_CASES = [  # irreps, (U, V, W), N
    ((_sh(2), _sh(2), "0e+1o"), (8, 16, 4), 301),
    ((_sh(2), _sh(2), "0e+1o"), (32, 32, 8), 301),
    ((_sh(2),) * 3, (32, 32, 32), 129),
    ((_sh(2),) * 3, (16, 4, 64), 1000),
    ((_sh(1), _sh(2), _sh(1)), (32, 8, 20), 700),      # weight gradient in 256 x 32 blocks, 20 of the 32 columns used
    ((_sh(1), _sh(2), _sh(1)), (32, 16, 48), 515),     # 256 x 64 blocks
    (("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e"), (16, 16, 16), 256),   # the reference's comparison-test shape
    ((_sh(2), _sh(2), _sh(1)), (4, 8, 16), 515),       # 32 contracted channel pairs: a fragment ring of two blocks
    ((_sh(1), _sh(1), _sh(2)), (4, 4, 8), 130),        # 16 pairs: half of that ring is padding
]


@pytest.mark.parametrize("irreps,channels,n", UVW_CASES)
def test_uvw_fp32_native(device, irreps, channels, n):
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn.functional import _uv_native
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = irreps
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    u, v, wc = channels
    g = torch.Generator().manual_seed(u * 100 + v * 10 + wc)
    x = torch.randn(n, Irreps(i1).dim, u, generator=g)
    y = torch.randn(n, Irreps(i2).dim, v, generator=g)
    w = torch.randn(T.shape[0], u, v, wc, generator=g) / (u * v) ** 0.5
    ct = torch.randn(n, Irreps(io).dim, wc, generator=g)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    assert _uv_native.uvw_supported(xd, yd, wd, infos[0])
    out = F.tensor_product_uvw(xd, yd, wd, *infos)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_uvw, T, (x, y, w), ct)
    out32, grads32 = ref_ops.dense_grads(ref_ops.dense_uvw, T, (x, y, w), ct, dtype=torch.float32)
    for name, a, b, r in zip(("out", "grad_x", "grad_y", "grad_w"), (out, gx, gy, gw), (ref_out, *ref_grads),
                             (out32, *grads32)):
        assert_close(a, b, 1e-5, f"uvw {channels} N={n} {name}", norm="max", fp32_ref=r)


def test_u1v_fp32_native_full_size(device):
    """The shapes of BASELINE configs[3] in fp32 (B = 32768, lmax = 3, C = 128): rows of a strided subset against
    the oracle (each output row depends on its own sample only)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.utils._sh import spherical_harmonics
    irr, ch, n = _sh(3), 128, 32768
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(n, 16, ch, generator=g)
    y = spherical_harmonics(unit_vectors(n, g), 3)
    w = torch.randn(mod.num_paths, ch, ch, generator=g) / (ch * mod.num_paths) ** 0.5
    ct = torch.randn(n, 16, ch, generator=g)
    sub = torch.arange(5, n, 257)
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = mod(xd, yd, wd)
    (gx,) = torch.autograd.grad(out, (xd,), ct.to(device))
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    ref_out, (rgx, _, _) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub])
    out32, (gx32, _, _) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub], dtype=torch.float32)
    assert_close(out[sub.to(device)], ref_out, 1e-5, "full size out", norm="max", fp32_ref=out32)
    assert_close(gx[sub.to(device)], rgx, 1e-5, "full size grad_x", norm="max", fp32_ref=gx32)


@pytest.mark.parametrize("irr1,lmax,cin,cout,n", [
    (None, 2, 128, 128, 16384 + 21), (None, 1, 128, 96, 32768), (None, 1, 112, 128, 16384 + 16), (None, 4, 32, 32, 16384 + 5),
    ("4e", 4, 128, 64, 16384 + 3),          # segments of more than eight terms: the part of a segment read from the tables
])
def test_u1v_fp32_large_batches_in_workgroups_of_32_samples(device, irr1, lmax, cin, cout, n):
    """From 16384 samples on, where the rows of 32 samples fit the LDS, the gradient of the second operand and (with
    a fragment ring of four and 64 or more output channels) the forward and the gradient of the first operand take
    workgroups of 32 samples, a weight fragment multiplied with two sets of 16; below that, and in every other test
    of this file, 16.  Rows of a strided subset, the last samples of a ragged batch among them, against the oracle
    (each row of the results depends on its own sample only)."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.utils._sh import spherical_harmonics
    irr = _sh(lmax)
    irr1 = irr1 or irr
    mod = SO3Linear(irr1, irr, irr1, cin, cout, internal_weights=False, feature_mode="uv").to(device)
    d = mod.irreps_in1_dim
    g = torch.Generator().manual_seed(11 + lmax)
    x = torch.randn(n, d, cin, generator=g)
    y = spherical_harmonics(unit_vectors(n, g), lmax)
    w = torch.randn(mod.num_paths, cin, cout, generator=g) / (cin * mod.num_paths) ** 0.5
    ct = torch.randn(n, d, cout, generator=g)
    sub = torch.cat([torch.arange(3, n, 509), torch.arange(n - 40, n)])
    xd, yd, wd = (t.to(device) for t in (x, y, w))
    xd.requires_grad_(True), yd.requires_grad_(True)
    out = mod(xd, yd, wd)
    gx, gy = torch.autograd.grad(out, (xd, yd), ct.to(device))
    T = ref_ops.dense_coupling(irr1, irr1, irr).float().double()
    ref_out, (rgx, rgy, _) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub])
    out32, (gx32, gy32, _) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub], dtype=torch.float32)
    on = sub.to(device)
    tag = f"{irr1} lmax {lmax} {cin}->{cout} N={n}"
    assert_close(out[on], ref_out, 1e-5, tag + " out", norm="max", fp32_ref=out32)
    assert_close(gx[on], rgx, 1e-5, tag + " grad_x", norm="max", fp32_ref=gx32)
    assert_close(gy[on], rgy, 1e-5, tag + " grad_y", norm="max", fp32_ref=gy32)


def test_u1v_fp32_full_size_properties(device):
    """The configs[3] shape in fp32 (B = 32768, lmax = 3, 128 -> 128) on the table-driven kernels.  out / grad_x /
    grad_y of a strided subset of the rows against the dense oracle (a row depends on its own sample only); the weight
    gradient, a sum over the batch, against the oracle's sum over the subset when every other output gradient is zero,
    and through additivity over two halves of the batch."""
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import _uv_native
    lmax, ch, n = 3, 128, 32768
    irreps = _sh(lmax)
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator().manual_seed(17)
    x = torch.randn(n, 16, ch, generator=g)
    y = torch.randn(n, 16, generator=g)
    w = torch.randn(mod.num_paths, ch, ch, generator=g) / (ch * mod.num_paths) ** 0.5
    ct = torch.randn(n, 16, ch, generator=g)
    sub = torch.arange(3, n, 331)                      # 99 rows spread over all workgroups
    mask = torch.zeros(n, 1, 1)
    mask[sub] = 1
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    assert _uv_native.u1v_supported(xd, yd, wd, mod.tp_info_forward)
    out = mod(xd, yd, wd)
    gx, gy, gw = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    T = ref_ops.dense_coupling(irreps, irreps, irreps).float().double()
    ref_out, (rgx, rgy, rgw_sub) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub])
    out32, (gx32, gy32, gw32) = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x[sub], y[sub], w), ct[sub],
                                                    dtype=torch.float32)
    sd = sub.to(device)
    for name, a, b, r in (("out", out[sd], ref_out, out32), ("grad_x", gx[sd], rgx, gx32),
                          ("grad_y", gy[sd], rgy, gy32)):
        # sums over 128 channels x paths: norm-wise, and within three times the fp32 contraction's own loss
        assert_close(a, b, 1e-5, f"u1v fp32 full size {name} rows", norm="max", fp32_ref=r)
    (gw_sub,) = torch.autograd.grad(mod(xd, yd, wd), (wd,), (ct * mask).to(device))
    assert_close(gw_sub, rgw_sub, 1e-5, "u1v fp32 full size grad_w of the subset", norm="max", fp32_ref=gw32)
    half = n // 2
    parts = []
    for lo, hi in ((0, half), (half, n)):
        ws = wd.detach().requires_grad_(True)
        (gp,) = torch.autograd.grad(mod(xd[lo:hi].detach(), yd[lo:hi].detach(), ws), (ws,), ct[lo:hi].to(device))
        parts.append(gp.double())
    # a sum of 32768 x 16 products per element, in chunks: rounding of the three results bounds the difference
    assert_close(gw.double(), parts[0] + parts[1], 1e-5, "u1v fp32 full size grad_w additivity", norm="max")


def test_fp32_fully_connected_past_two_to_the_31_elements(device):
    """1.1 million samples x 16 x 128 fp32 = 2.25e9 elements per operand on the table-driven matrix-core kernels: rows
    at both ends of the batch against the same rows as a batch of their own (1e-5), the weight gradient against the
    sum over the two halves of the batch (1e-4 norm-wise: sums of a million terms in different groupings)."""
    from equitorch_amd.nn import SO3Linear
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 50 GB of device memory")
    n, ch, irreps = 1_100_000, 128, "0e+1o+2e+3o"
    mod = SO3Linear(irreps, irreps, irreps, ch, ch, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator(device=device).manual_seed(5)
    x = torch.randn(n, 16, ch, generator=g, device=device).requires_grad_(True)
    y = torch.randn(n, 16, generator=g, device=device).requires_grad_(True)
    w = (torch.randn(mod.num_paths, ch, ch, generator=g, device=device) / 40).requires_grad_(True)
    ct = torch.randn(n, 16, ch, generator=g, device=device)
    assert x.numel() > 2 ** 31
    out = mod(x, y, w)
    gx, gy, gw = torch.autograd.grad(out, (x, y, w), ct)
    idx = torch.cat([torch.arange(0, 64, device=device), torch.arange(n - 64, n, device=device)])
    xs, ys = (t.detach()[idx].clone().requires_grad_(True) for t in (x, y))
    outs = mod(xs, ys, w)
    gxs, gys, _ = torch.autograd.grad(outs, (xs, ys, w), ct[idx])
    for name, a, b in (("out", out[idx], outs), ("grad_x", gx[idx], gxs), ("grad_sh", gy[idx], gys)):
        assert (a - b).abs().max().item() <= 1e-5 * max(1.0, b.abs().max().item()), name
    del out, gx, gy
    half = n // 2
    parts = [torch.autograd.grad(mod(x.detach()[lo:hi], y.detach()[lo:hi], w), (w,), ct[lo:hi])[0]
             for lo, hi in ((0, half), (half, n))]
    ref = parts[0] + parts[1]
    assert (gw - ref).abs().max().item() <= 1e-4 * ref.abs().max().item(), "grad_w"
    del x, y, ct
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("per_sample", [False, True])
def test_16_bit_operands_without_a_compiled_table(device, monkeypatch, dtype, per_sample):
    """bf16 / fp16 operands on irreps whose table has no compiled matrix-core kernels (the reference's own comparison
    irreps ``0e+1e+2e+3e``): the table-driven kernels in fp32 arithmetic on widened copies, the result rounded once —
    no ``(N, segments, C)`` intermediate and no library GEMM.  Against the float64 oracle on the rounded inputs."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    irr, n, cin, cout = "0e+1e+2e+3e", 300, 32, 48
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator().manual_seed(3)
    rd = lambda *s: torch.randn(*s, generator=g).to(dtype)
    x, y = rd(n, 16, cin), rd(n, 16)
    w = (torch.randn(*((n,) if per_sample else ()), T.shape[0], cin, cout, generator=g) / (cin * T.shape[0]) ** 0.5).to(dtype)
    ct = rd(n, 16, cout)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = F.tensor_product_u1v(xd, yd, wd, *infos)
    assert out.dtype == dtype
    assert "widened" in seen[0] and ("streaming" in seen[-1] if per_sample else "matrix-core" in seen[-1]), seen
    grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x.double(), y.double(), w.double()), ct.double())
    for name, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads)):
        assert a.dtype == dtype
        assert_close(a.float(), b, 1e-2, f"u1v {dtype} widened per_sample={per_sample} {name}", norm="max")


def test_all_even_table_at_128_channels(device, monkeypatch):
    """``0e+1e+2e+3e`` (34 paths, 611 coefficients) at 128 -> 128 channels, fp32 and bf16: the 16 staged samples and the
    walk tables of every kernel of the step fit the LDS (the host's estimate for the gradient of the second operand
    used to count an item per coefficient and sent this shape to the library route)."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    irr, n, ch = "0e+1e+2e+3e", 1000, 128
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator().manual_seed(9)
    x, y, ct = (torch.randn(*s, generator=g) for s in ((n, 16, ch), (n, 16), (n, 16, ch)))
    w = torch.randn(T.shape[0], ch, ch, generator=g) / (ch * T.shape[0]) ** 0.5
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        seen = []
        monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
        xd, yd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, y, w))
        out = F.tensor_product_u1v(xd, yd, wd, *infos)
        assert "fp32 matrix-core kernel (table-driven)" in seen[-1], seen
        grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device, dtype))
        twins = (None,) * 4
        if dtype == torch.bfloat16:      # the oracle on the rounded inputs
            r = lambda t: t.to(dtype).double()
            ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (r(x), r(y), r(w)), r(ct))
        else:                            # the same contraction in fp32 arithmetic bounds what a norm-wise comparison allows
            o32, g32 = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct, dtype=torch.float32)
            twins = (o32, *g32)
        for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), twins):
            assert_close(a.float(), b, tol, f"u1v {irr} 128 -> 128 {dtype} {name}", norm="max", fp32_ref=b32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_channel_counts_that_are_not_multiples_of_four(device, monkeypatch, dtype):
    """10 -> 7 channels (u1v) and 5 x 6 -> 9 (uvw) with a shared weight: zero channels are appended up to multiples of
    4 and the same kernels run; forward and all gradients against the dense oracle."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    irr, n = _sh(2), 211
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    T = ref_ops.dense_coupling(irr, irr, irr).float().double()
    g = torch.Generator().manual_seed(10)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    cases = (("u1v", F.tensor_product_u1v, ref_ops.dense_u1v, (rd(n, 9, 10), rd(n, 9), rd(T.shape[0], 10, 7) / 3), rd(n, 9, 7)),
             ("uvw", F.tensor_product_uvw, ref_ops.dense_uvw, (rd(n, 9, 5), rd(n, 9, 6), rd(T.shape[0], 5, 6, 9) / 5), rd(n, 9, 9)))
    for name, fn, ref_fn, ops, ct in cases:
        seen = []
        monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
        leaves = [t.to(device).requires_grad_(True) for t in ops]
        out = fn(*leaves, *infos)
        assert "padded" in seen[0] and "matrix-core" in seen[-1], seen
        assert out.shape == ct.shape and out.is_contiguous()
        grads = torch.autograd.grad(out, leaves, ct.to(device))
        ref_out, ref_grads = ref_ops.dense_grads(ref_fn, T, ops, ct)
        for what, a, b in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads)):
            assert a.shape == b.shape
            assert_close(a, b, tol, f"{name} {dtype} odd channel counts {what}", norm="max")


@pytest.mark.parametrize("irreps,c1,c2,n,dtype", [((_sh(2),) * 3, 32, 48, 300, torch.float32),
                                                   (("1o+2e+1e", "0e+1o+2e", "0e+1o"), 16, 64, 515, torch.float32),
                                                   ((_sh(3), _sh(2), _sh(3)), 20, 12, 70, torch.float64)])
def test_vu1_native(device, monkeypatch, irreps, c1, c2, n, dtype):
    """``out[n,M] = sum c <y[n,b,:], x[n,a,:] @ W[p]>`` with a shared weight on the table-driven matrix-core kernels
    (the kernel of the second operand's gradient of u1v, run on the table with output and second-operand rows
    exchanged), forward and all gradients against the dense oracle."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = irreps
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    g = torch.Generator().manual_seed(c1 + c2 + n)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    x, y, w = rd(n, T.shape[2], c1), rd(n, T.shape[3], c2), rd(T.shape[0], c1, c2) / (c1 * c2) ** 0.5
    ct = rd(n, T.shape[1])

    def dense_vu1(T, x, y, w, dtype=torch.float64):
        return ref_ops.dense_uvw(T, x, y, w.unsqueeze(-1), dtype=dtype).squeeze(-1)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = F.tensor_product_vu1(xd, yd, wd, *infos)
    assert "matrix-core" in seen[-1], seen
    grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device))
    ref_out, ref_grads = ref_ops.dense_grads(dense_vu1, T, (x, y, w), ct)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    twin = (None,) * 4
    if dtype == torch.float32:
        o32, g32 = ref_ops.dense_grads(dense_vu1, T, (x, y, w), ct, dtype=torch.float32)
        twin = (o32, *g32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), twin):
        assert_close(a, b, tol, f"vu1 {io} {c1}x{c2} N={n} {dtype} {name}", norm="max", fp32_ref=b32)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_1vu_native(device, monkeypatch, dtype):
    """The channels on the second operand with a shared weight: the u1v kernels on the table with the operands' rows
    exchanged; forward, all gradients and a gradient of the gradient."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = "1o+2e+1e", "0e+1o", "0e+1o+2e"
    infos = [t.to(device) for t in tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[:3]]
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    n, cin, cout = 333, 24, 40
    g = torch.Generator().manual_seed(21)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype)
    x, y, w, ct = rd(n, T.shape[2]), rd(n, T.shape[3], cin), rd(T.shape[0], cin, cout) / cin ** 0.5, rd(n, T.shape[1], cout)

    def dense_1vu(T, x, y, w, dtype=torch.float64):
        return ref_ops.dense_u1v(T.transpose(2, 3), y, x, w, dtype=dtype)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
    out = F.tensor_product_1vu(xd, yd, wd, *infos)
    assert "matrix-core" in seen[-1], seen
    grads = torch.autograd.grad(out, (xd, yd, wd), ct.to(device), retain_graph=True)
    ref_out, ref_grads = ref_ops.dense_grads(dense_1vu, T, (x, y, w), ct)
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    twins = (None,) * 4
    if dtype == torch.float32:
        o32, g32 = ref_ops.dense_grads(dense_1vu, T, (x, y, w), ct, dtype=torch.float32)
        twins = (o32, *g32)
    for name, a, b, b32 in zip(("out", "grad_x", "grad_y", "grad_w"), (out, *grads), (ref_out, *ref_grads), twins):
        assert_close(a, b, tol, f"1vu {dtype} {name}", norm="max", fp32_ref=b32)
    if dtype == torch.float64:
        gy, = torch.autograd.grad(out, yd, ct.to(device), create_graph=True)
        gg = torch.autograd.grad(gy.square().sum(), (xd, wd))
        xr, yr, wr = (t.clone().requires_grad_(True) for t in (x, y, w))
        rgy, = torch.autograd.grad(dense_1vu(T, xr, yr, wr), yr, ct, create_graph=True)
        rgg = torch.autograd.grad(rgy.square().sum(), (xr, wr))
        for name, a, b in zip(("d/dx", "d/dw"), gg, rgg):
            assert_close(a, b, 1e-10, f"1vu second order {name}", norm="max")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_incoming_gradient_at_an_odd_offset_of_a_larger_buffer(device, dtype):
    """Autograd hands the backward whatever view the consumer produced: the gradient of a slice or of a ``cat`` is
    contiguous but starts at any element of a larger buffer.  The kernels want 16-byte boundaries; the Functions copy
    such a gradient first.  Same results as with an aligned gradient, for the u1v product, the uvw product and the
    channel mixing that runs on them."""
    import equitorch_amd.nn.functional as F
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import IrrepsLinear, SO3Linear
    from equitorch_amd.utils import tp_infos
    irr, n = _sh(2), 130
    g = torch.Generator().manual_seed(5)
    rd = lambda *s: torch.randn(*s, generator=g).to(device, dtype)
    uv = SO3Linear(irr, irr, irr, 8, 12, internal_weights=False, feature_mode="uv").to(device)
    lin = IrrepsLinear("1o+2e", "1o+2e", 4, 12, internal_weights=False).to(device)
    infos = [t.to(device) for t in tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[:3]]
    cases = [("u1v", lambda x, y, w: uv(x, y, w), (rd(n, 9, 8), rd(n, 9), rd(uv.num_paths, 8, 12))),
             ("uvw", lambda x, y, w: F.tensor_product_uvw(x, y, w, *infos), (rd(n, 9, 4), rd(n, 9, 4), rd(11, 4, 4, 8))),
             ("linear", lambda x, w: lin(x, w), (rd(n, 8, 4), rd(lin.num_paths, 4, 12)))]
    for name, fn, ops in cases:
        leaves = [t.clone().requires_grad_(True) for t in ops]
        out = fn(*leaves)
        ct = torch.randn(out.shape, generator=g).to(device, dtype)
        want = torch.autograd.grad(out, leaves, ct, retain_graph=True)
        for k in (1, 3):
            buf = torch.empty(ct.numel() + 3, dtype=dtype, device=device)
            buf[k:k + ct.numel()] = ct.reshape(-1)
            odd = buf[k:k + ct.numel()].view(ct.shape)
            assert odd.is_contiguous() and odd.data_ptr() % 16 != 0
            got = torch.autograd.grad(out, leaves, odd, retain_graph=True)
            for a, b in zip(got, want):
                assert torch.equal(a, b), f"{name}: gradient differs with the cotangent {k} elements off"
