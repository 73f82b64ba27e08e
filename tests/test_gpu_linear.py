"""GPU parity of IrrepsLinear / IrrepWiseLinear against the oracle's restatement of the reference forward and its
autograd gradients (first and second order)."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_ops, ref_tables

pytestmark = pytest.mark.gpu

CASES = [
    ("0e+1o+2e", "0e+1o+2e", {}),
    ("0e+1o+2e", "0e+1o+1o+2e+0e", {}),
    ("2x0e+1o+3x2e", "0e+2x1o+2e+3e", {}),
    ("0e+1o", "0e+1e+2e", {"path_norm": False}),          # 1o has no source: zero rows
    ("0e+1o+2e", "0e+1o+2e", {"channel_norm": True}),
]


def _grads(out, inputs, ct):
    return torch.autograd.grad(out, inputs, ct)


@pytest.mark.parametrize("io,ii,kw", CASES)
@pytest.mark.parametrize("shared", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_irreps_linear_matches_oracle(device, io, ii, kw, shared, dtype):
    from equitorch_amd.nn import IrrepsLinear
    n, cin, cout = 37, 24, 40
    mod = IrrepsLinear(ii, io, cin, cout, internal_weights=False, **kw).to(device)
    okw = dict(kw)
    if okw.get("channel_norm"):
        okw["channel_scale"] = cin            # what the reference's constructor passes (nn/linears.py:357-358)
    info = ref_tables.irreps_linear_infos(io, ii, **okw)[0]
    # the reference stores the scales with torch.tensor(list): fp32 values, also under fp64 inputs
    info["scale_MM0"] = torch.tensor(info["scale_MM0"]).double().tolist()
    g = torch.Generator().manual_seed(1)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
    x = rd(n, mod.irreps_in_dim, cin)
    w = rd(*(() if shared else (n,)), mod.num_paths, cin, cout)
    ct = rd(n, mod.irreps_out_dim, cout)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irreps_linear(xr, wr, info)
    rgx, rgw = _grads(ref, (xr, wr), ct)
    xd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, w))
    out = mod(xd, wd)
    gx, gw = _grads(out, (xd, wd), ct.to(device, dtype))
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    # the same CPU function on float32 tensors: what the reference's own fp32 arithmetic loses
    x32, w32 = x.float().requires_grad_(True), w.float().requires_grad_(True)
    ref32 = ref_ops.cpu_irreps_linear(x32, w32, info)
    r32 = (ref32, *_grads(ref32, (x32, w32), ct.float()))
    for (name, a, b), b32 in zip((("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)), r32):
        # channel_norm as the reference passes it (channel_scale = C_in) gives terms of order 10^2 that cancel:
        # that case is compared norm-wise in fp32, and held to three times the fp32 restatement's own error
        big = bool(kw.get("channel_norm")) and dtype == torch.float32
        assert_close(a, b, tol=tol, what=f"{io}<-{ii} shared={shared} {name}", norm="max" if big else "element",
                     fp32_ref=b32 if big else None)


@pytest.mark.parametrize("shared", [True, False])
def test_irrep_wise_linear_matches_oracle_and_leading_dims(device, shared):
    from equitorch_amd.nn import IrrepWiseLinear
    irr, cin, cout = "0e+1o+2e+1o", 16, 8
    mod = IrrepWiseLinear(irr, cin, cout, internal_weights=False, channel_norm=True).to(device)
    info = ref_tables.irreps_info(irr)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(3, 5, 12, cin, generator=g, dtype=torch.float64)
    w = torch.randn(*(() if shared else (15,)), 4, cin, cout, generator=g, dtype=torch.float64)
    ct = torch.randn(3, 5, 12, cout, generator=g, dtype=torch.float64)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irrep_wise_linear(xr.reshape(15, 12, cin), wr, info).reshape(3, 5, 12, cout) / cin ** 0.5
    rgx, rgw = _grads(ref, (xr, wr), ct)
    xd, wd = (t.to(device).requires_grad_(True) for t in (x, w))
    out = mod(xd, wd.reshape(-1) if shared else wd)       # a flat weight is viewed to (P, C_in, C_out)
    gx, gw = _grads(out, (xd, wd), ct.to(device))
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert_close(a, b, tol=1e-12, what=f"irrep-wise shared={shared} {name}")


def test_internal_weights_bf16_and_second_order(device):
    from equitorch_amd.nn import IrrepsLinear
    torch.manual_seed(0)
    mod = IrrepsLinear("0e+1o+2e", "0e+1o+2e", 32, 32).to(device)
    assert mod.weight.shape == (3, 32, 32) and float(mod.weight.detach().abs().max()) <= (3.0 / 32) ** 0.5
    x = torch.randn(64, 9, 32, device=device)
    ref = torch.cat([x[:, a:b] @ mod.weight[p] for p, (a, b) in enumerate([(0, 1), (1, 4), (4, 9)])], dim=1)
    assert_close(mod(x), ref, tol=1e-5, what="internal weights")
    out16 = mod.to(torch.bfloat16)(x.bfloat16())
    assert out16.dtype == torch.bfloat16
    assert float((out16.float() - ref).detach().abs().max()) <= 1e-2 * max(1.0, float(ref.detach().abs().max()))
    # second order: gradgradcheck of the two primitives in fp64 on a tiny case
    mod64 = IrrepsLinear("0e+1o+1o", "0e+1o", 3, 2, internal_weights=False).to(device)
    xs = torch.randn(4, 7, 3, device=device, dtype=torch.float64, requires_grad=True)
    for shape in ((3, 3, 2), (4, 3, 3, 2)):
        ws = torch.randn(*shape, device=device, dtype=torch.float64, requires_grad=True)
        assert torch.autograd.gradcheck(mod64, (xs, ws))
        assert torch.autograd.gradgradcheck(mod64, (xs, ws))
    with pytest.raises(Exception):
        mod64(torch.randn(4, 7, 3), torch.randn(3, 3, 2))     # CPU tensors are rejected


@pytest.mark.parametrize("irr,cin,cout,n", [("0e+1o+2e+3o", 128, 128, 1100), ("0e+1o+2e", 64, 32, 700)])
def test_bf16_shared_weight_runs_on_the_matrix_core_kernels(device, irr, cin, cout, n):
    """bf16 with a shared weight and a compiled-in table: the MFMA kernels of the fully connected product with the
    scalar 1 as second operand.  Output and both gradients within rel 1e-2 of the fp64 oracle."""
    from equitorch_amd.nn import IrrepsLinear
    from equitorch_amd.nn.functional import _irreps_gemm as G, _uvw_mfma
    mod = IrrepsLinear(irr, irr, cin, cout, internal_weights=False).to(device)
    plan = G.plan_of_linear_info(mod.forward_info)
    assert _uvw_mfma.uv_config_of(G._as_tensor_product(plan, mod.irreps_in_dim)) >= 0
    info = ref_tables.irreps_linear_infos(irr, irr)[0]
    g = torch.Generator().manual_seed(3)
    rd = lambda *s: torch.randn(*s, generator=g).bfloat16().double()
    x, w, ct = rd(n, mod.irreps_in_dim, cin), rd(mod.num_paths, cin, cout) / cin ** 0.5, rd(n, mod.irreps_out_dim, cout)
    w = w.bfloat16().double()
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irreps_linear(xr, wr, info)
    rgx, rgw = _grads(ref, (xr, wr), ct)
    xd, wd = (t.to(device, torch.bfloat16).requires_grad_(True) for t in (x, w))
    out = mod(xd, wd)
    gx, gw = _grads(out, (xd, wd), ct.to(device, torch.bfloat16))
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert a.dtype == torch.bfloat16
        assert_close(a.float(), b, tol=1e-2, what=f"bf16 {irr} {name}")


@pytest.mark.parametrize("cin,cout,n", [(64, 64, 20003), (48, 24, 1001), (16, 64, 70001), (64, 8, 31), (32, 32, 4099),
                                        (8, 24, 515)])
def test_weight_gradient_of_weights_up_to_64_by_64(device, cin, cout, n):
    """fp32 shared weights of at most 64 x 64: the weight gradient has a wavefront per (path, chunk of samples) that keeps
    the whole block in its registers (four channels a lane along an axis of up to 64 channels, two along one of up
    to 32: all four combinations).  Sample counts that leave a ragged last chunk (and a last group of fewer than
    four samples) and that make the chunks 32, 64 and 256 samples long; sums over up to 70 001 samples in fp32 are
    compared norm-wise, with the fp32 restatement beside them."""
    from equitorch_amd.nn import IrrepsLinear
    io, ii = "0e+1o+2e", "0e+1o+1o+2e"
    mod = IrrepsLinear(ii, io, cin, cout, internal_weights=False).to(device)
    info = ref_tables.irreps_linear_infos(io, ii)[0]
    info["scale_MM0"] = torch.tensor(info["scale_MM0"]).double().tolist()
    g = torch.Generator().manual_seed(n)
    rd = lambda *s: torch.randn(*s, generator=g).double()
    x, ct, w = rd(n, mod.irreps_in_dim, cin), rd(n, mod.irreps_out_dim, cout), rd(mod.num_paths, cin, cout)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irreps_linear(xr, wr, info)
    rgw, = _grads(ref, (wr,), ct)
    x32, w32 = x.float(), w.float().requires_grad_(True)
    r32, = _grads(ref_ops.cpu_irreps_linear(x32, w32, info), (w32,), ct.float())
    xd, wd = x.to(device, torch.float32), w.to(device, torch.float32).requires_grad_(True)
    gw, = _grads(mod(xd, wd), (wd,), ct.to(device, torch.float32))
    assert_close(gw, rgw, tol=1e-5, what=f"grad_w {cin}->{cout} n={n}", norm="max", fp32_ref=r32)


@pytest.mark.parametrize("dtype,cin,cout,shared", [(torch.float32, 10, 7, True), (torch.float64, 6, 9, True),
                                                    (torch.bfloat16, 24, 40, True), (torch.bfloat16, 10, 7, True),
                                                    (torch.float16, 16, 8, False)])
def test_operands_adapted_to_the_native_kernels(device, monkeypatch, dtype, cin, cout, shared):
    """Channel counts that are not multiples of 4 (zero channels appended) and 16-bit operands without a compiled
    matrix-core table (widened to fp32, the result rounded once) run on the table-driven / streaming kernels instead of
    the library GEMMs; against the oracle on the rounded inputs."""
    from equitorch_amd.nn import IrrepsLinear
    from equitorch_amd.ops import kernels
    io, ii, n = "0e+1o+2e", "0e+1o+1o+2e+0e", 130
    mod = IrrepsLinear(ii, io, cin, cout, internal_weights=False).to(device)
    info = ref_tables.irreps_linear_infos(io, ii)[0]
    info["scale_MM0"] = torch.tensor(info["scale_MM0"]).double().tolist()
    g = torch.Generator().manual_seed(4)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
    x, ct = rd(n, mod.irreps_in_dim, cin), rd(n, mod.irreps_out_dim, cout)
    w = rd(*(() if shared else (n,)), mod.num_paths, cin, cout) / cin ** 0.5
    w = w.to(dtype).double()
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_irreps_linear(xr, wr, info)
    rgx, rgw = _grads(ref, (xr, wr), ct)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    xd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, w))
    out = mod(xd, wd)
    assert seen and ("table-driven matrix-core" in seen[-1] or "streaming" in seen[-1]), seen
    assert out.dtype == dtype and out.shape == ref.shape and out.is_contiguous()
    gx, gw = _grads(out, (xd, wd), ct.to(device, dtype))
    tol = {torch.float32: 1e-5, torch.float64: 1e-12}.get(dtype, 1e-2)
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert a.dtype == dtype and a.shape == b.shape
        assert_close(a.double(), b, tol, f"IrrepsLinear {dtype} {cin}->{cout} shared={shared} {name}",
                     norm="element" if dtype in (torch.float32, torch.float64) else "max")
