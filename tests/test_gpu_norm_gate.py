"""GPU parity of Gate, the invariant norms and the RMS normalisation layers against the oracle (float64 torch
restatement of the reference's forwards; autograd of the oracle for the gradients)."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_ops, ref_tables

pytestmark = pytest.mark.gpu

IRR = "0e+1o+2e+1o"      # dim 12, 4 irreps


def _info():
    """The oracle's tables with 1/dim and dim^-1/2 rounded to fp32, which is how the reference stores them
    (``torch.tensor(list)``), also when the features are fp64."""
    info = ref_tables.irreps_info(IRR)
    for k in ("rdims", "rsqrt_dims"):
        info[k] = torch.tensor(info[k]).double().tolist()
    return info


def _data(n, c, dtype, seed=0, extra=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(n, 12 + extra, c, generator=g, dtype=torch.float64).to(dtype).double(), g


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("shared", [False, True])
def test_gate(device, dtype, shared):
    from equitorch_amd.nn import Gate
    info = _info()
    x, g = _data(33, 20, dtype)
    gate = torch.randn(*(() if shared else (33,)), 4, 20, generator=g, dtype=torch.float64).to(dtype).double()
    ct = torch.randn(33, 12, 20, generator=g, dtype=torch.float64).to(dtype).double()
    act = torch.nn.Sigmoid()
    xr, gr = x.clone().requires_grad_(True), gate.clone().requires_grad_(True)
    ref = ref_ops.cpu_gating(xr, act(gr), info)
    rg = torch.autograd.grad(ref, (xr, gr), ct)
    mod = Gate(IRR, activation=act).to(device)
    xd, gd = (t.to(device, dtype).requires_grad_(True) for t in (x, gate))
    out = mod(xd, gd)
    got = torch.autograd.grad(out, (xd, gd), ct.to(device, dtype))
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    for name, a, b in (("out", out, ref), ("grad_x", got[0], rg[0]), ("grad_gate", got[1], rg[1])):
        assert_close(a, b, tol=tol, what=f"gate shared={shared} {name}")
    if not shared:      # concatenated input and the global (not irrep-wise) gate
        cat = torch.cat([x, gate], dim=1).to(device, dtype)
        assert_close(mod(cat), ref, tol=tol, what="concatenated gates")
        glob = Gate(IRR, irrep_wise=False).to(device)
        assert_close(glob(xd, gd[:, :1]), x * gate[:, :1], tol=tol, what="global gate")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("scaled", [True, False])
def test_norms(device, dtype, scaled):
    from equitorch_amd.nn import MeanSquaredNorm, Norm, SquaredNorm
    info = _info()
    x, g = _data(41, 24, dtype, seed=1)
    x[3, 1:4] = 0.0                      # a zero block: the norm's gradient there is zero, not nan
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    cases = [("squared", SquaredNorm(IRR, scaled), ref_ops.cpu_squared_norm),
             ("norm", Norm(IRR, scaled), ref_ops.cpu_norm),
             ("channel mean", MeanSquaredNorm(IRR, scaled, dim=-1), ref_ops.cpu_channel_mean_squared_norm),
             ("batch mean", MeanSquaredNorm(IRR, scaled, dim=0), ref_ops.cpu_batch_mean_squared_norm)]
    for name, mod, ref_fn in cases:
        xr = x.clone().requires_grad_(True)
        ref = ref_fn(xr, info, scaled)
        ct = torch.randn(ref.shape, generator=g, dtype=torch.float64).to(dtype).double()
        (rgx,) = torch.autograd.grad(ref, xr, ct)
        rgx = torch.nan_to_num(rgx, nan=0.0)            # sqrt at the zero block: the reference defines 0
        xd = x.to(device, dtype).requires_grad_(True)
        out = mod.to(device)(xd)
        (gx,) = torch.autograd.grad(out, xd, ct.to(device, dtype))
        assert torch.isfinite(gx).all()
        assert_close(out, ref, tol=tol, what=f"{name} scaled={scaled}")
        assert_close(gx, rgx, tol=tol, what=f"{name} scaled={scaled} grad")


@pytest.mark.parametrize("affine", [True, False])
def test_rms_normalisation_layers(device, affine):
    from equitorch_amd.nn import BatchRMSNorm, LayerRMSNorm
    info = _info()
    x, g = _data(29, 16, torch.float64, seed=2)
    ct = torch.randn(29, 12, 16, generator=g, dtype=torch.float64)
    w = (1 + 0.3 * torch.randn(4, 16, generator=g, dtype=torch.float64)) if affine else None
    # layer norm
    mod = LayerRMSNorm(IRR, 16, affine=affine).to(device).double()
    if affine:
        mod.weight.data.copy_(w)
    xr = x.clone().requires_grad_(True)
    ref = ref_ops.cpu_layer_rms_norm(xr, info, w)
    (rgx,) = torch.autograd.grad(ref, xr, ct)
    xd = x.to(device).requires_grad_(True)
    out = mod(xd)
    (gx,) = torch.autograd.grad(out, xd, ct.to(device))
    assert_close(out, ref, tol=1e-12, what="layer rms")
    assert_close(gx, rgx, tol=1e-11, what="layer rms grad")
    # batch norm: training step (statistics of the batch, running average updated), then evaluation
    bn = BatchRMSNorm(IRR, 16, affine=affine, momentum=0.2).to(device).double()
    if affine:
        bn.weight.data.copy_(w)
    xr = x.clone().requires_grad_(True)
    ref, running = ref_ops.cpu_batch_rms_norm(xr, torch.ones(4, 16, dtype=torch.float64), info, w, training=True,
                                              momentum=0.2)
    (rgx,) = torch.autograd.grad(ref, xr, ct)
    xd = x.to(device).requires_grad_(True)
    out = bn(xd)
    (gx,) = torch.autograd.grad(out, xd, ct.to(device))
    assert_close(out, ref, tol=1e-12, what="batch rms (training)")
    assert_close(gx, rgx, tol=1e-11, what="batch rms grad")
    assert_close(bn.running_squared_norm, running, tol=1e-12, what="running statistic")
    bn.eval()
    ref_eval, _ = ref_ops.cpu_batch_rms_norm(x, running, info, w, training=False)
    assert_close(bn(x.to(device)), ref_eval, tol=1e-12, what="batch rms (evaluation)")
    with pytest.raises(ValueError):
        bn(x.to(device)[:, :5])


def test_irrep_wise_dropout(device):
    """Whole irrep blocks of a channel are dropped together and the survivors scaled by 1 / (1 - p); evaluation mode
    is the identity; the gradient is the mask itself."""
    from equitorch_amd.nn import Dropout
    torch.manual_seed(0)
    drop = Dropout(p=0.4, irreps=IRR).to(device)
    x = (1.0 + torch.rand(64, 12, 16, device=device)).requires_grad_(True)      # strictly positive entries
    y = drop(x)
    ratio = (y / x).detach()
    assert torch.all((ratio - 0).abs().lt(1e-6) | (ratio - 1 / 0.6).abs().lt(1e-5))
    seg = [0, 1, 4, 9, 12]
    for a, b in zip(seg[:-1], seg[1:]):
        block = ratio[:, a:b]
        assert float((block - block[:, :1]).abs().max()) < 1e-5                  # one decision per irrep and channel
    kept = float((ratio > 0).float().mean())
    assert 0.5 < kept < 0.7
    (g,) = torch.autograd.grad(y.sum(), x)
    assert_close(g, ratio, tol=1e-5, what="dropout gradient")
    drop.eval()
    assert drop(x) is x
    plain = Dropout(p=0.5, irrep_wise=False).to(device).train()
    z = plain(x.detach())
    per_channel = (z != 0).float().mean(dim=1)
    assert torch.all((per_channel == 0) | (per_channel == 1))                     # whole channels


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("scaled", [True, False])
def test_tensor_dot(device, dtype, scaled):
    """``TensorDot('uu')``: irrep-wise dot product and both gradients against the oracle; extra leading axes and a
    broadcast second operand; ``'uv'`` raises as in the reference."""
    from equitorch_amd.nn import TensorDot
    info = _info()
    x, g = _data(37, 24, dtype, seed=5)
    y = torch.randn(37, 12, 24, generator=g, dtype=torch.float64).to(dtype).double()
    ct = torch.randn(37, 4, 24, generator=g, dtype=torch.float64).to(dtype).double()
    xr, yr = x.clone().requires_grad_(True), y.clone().requires_grad_(True)
    ref = ref_ops.cpu_tensor_dot(xr, yr, info, scaled)
    rg = torch.autograd.grad(ref, (xr, yr), ct)
    mod = TensorDot(IRR, "uu", scaled=scaled).to(device)
    xd, yd = (t.to(device, dtype).requires_grad_(True) for t in (x, y))
    out = mod(xd, yd)
    got = torch.autograd.grad(out, (xd, yd), ct.to(device, dtype))
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    for name, a, b in (("out", out, ref), ("grad_1", got[0], rg[0]), ("grad_2", got[1], rg[1])):
        assert_close(a, b, tol=tol, what=f"tensor dot scaled={scaled} {name}")
    lead = mod(xd.detach().reshape(1, 37, 12, 24).expand(2, 37, 12, 24), yd.detach())
    assert lead.shape == (2, 37, 4, 24)
    assert_close(lead[1], ref, tol=tol, what="leading axes")
    with pytest.raises(NotImplementedError):
        TensorDot(IRR, "uv").to(device)(xd, yd)


def test_xyz_to_sincos_module(device):
    """``XYZToSinCos``: ``[1, sin(m a), cos(m a)]_m`` of the polar angles, against atan2 / acos in float64."""
    from equitorch_amd.nn import XYZToSinCos
    g = torch.Generator().manual_seed(6)
    v = torch.randn(50, 3, generator=g, dtype=torch.float64)
    u = v / v.norm(dim=-1, keepdim=True)
    theta, phi = torch.acos(u[:, 2].clamp(-1, 1)), torch.atan2(u[:, 1], u[:, 0])
    for normalised in (False, True):
        st, sp = XYZToSinCos(3, component_normalize=normalised)(v.to(device))
        scale = 2 ** 0.5 if normalised else 1.0
        for got, ang in ((st, theta), (sp, phi)):
            assert got.shape == (50, 7)
            ref = torch.stack([torch.ones_like(ang)] + [f(m * ang) * scale for m in (1, 2, 3)
                                                        for f in (torch.sin, torch.cos)], dim=-1)
            assert_close(got, ref, tol=1e-10, what=f"sincos normalised={normalised}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("channels", [64, 24, 10, 256])
@pytest.mark.parametrize("scaled", [True, False])
def test_layer_rms_fused_kernels(device, dtype, channels, scaled):
    """``cgtp_layer_rms_forward`` / ``cgtp_layer_rms_backward`` against the oracle: 16-byte lanes (64, 24, 256
    channels; 256 needs them in fp32 and is too wide in fp64, where the composed path takes over), one element per
    lane (10), irreps up to l = 6, rows not a multiple of the rows per wavefront, gradients of x and of the weight."""
    from equitorch_amd.nn.functional import layer_rms_norm
    from equitorch_amd.utils import irreps_info
    irr = "0e+1o+2e+6e+1o"
    info = ref_tables.irreps_info(irr)
    for k in ("rdims", "rsqrt_dims"):
        info[k] = torch.tensor(info[k]).double().tolist()
    d = 1 + 3 + 5 + 13 + 3
    g = torch.Generator().manual_seed(11)
    n = 131
    x = torch.randn(n, d, channels, generator=g, dtype=torch.float64).to(dtype).double()
    w = (1 + 0.3 * torch.randn(5, channels, generator=g, dtype=torch.float64)).to(dtype).double()
    ct = torch.randn(n, d, channels, generator=g, dtype=torch.float64).to(dtype).double()
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_layer_rms_norm(xr, info, wr, scaled=scaled, eps=1e-5)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    dev_info = irreps_info(irr).to(device)
    xd, wd = x.to(device, dtype).requires_grad_(True), w.to(device, dtype).requires_grad_(True)
    out = layer_rms_norm(xd, dev_info, wd, scaled=scaled, eps=1e-5)
    gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device, dtype))
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    assert_close(out, ref, tol=tol, what="out")
    assert_close(gx, rgx, tol=tol * 10, what="grad x")
    # the weight gradient sums 131 x dim terms of either sign: judged against the sum of their magnitudes
    assert_close(gw, rgw, tol=tol * 10, what="grad weight")
    # no weight, only the input's gradient
    out0 = layer_rms_norm(xd, dev_info, None, scaled=scaled, eps=1e-5)
    ref0 = ref_ops.cpu_layer_rms_norm(xr, info, None, scaled=scaled, eps=1e-5)
    assert_close(out0, ref0, tol=tol, what="out without weight")
    (g0,) = torch.autograd.grad(out0, xd, ct.to(device, dtype))
    (r0,) = torch.autograd.grad(ref0, xr, ct)
    assert_close(g0, r0, tol=tol * 10, what="grad x without weight")


def test_layer_rms_second_order_and_fallback(device):
    """Gradients of gradients go through the composed, differentiable path and agree with the oracle's; an irrep of
    degree 7 (15 components) is outside the fused kernel and runs composed."""
    from equitorch_amd.nn.functional import layer_rms_norm
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import irreps_info
    info = _info()
    x, g = _data(9, 8, torch.float64, seed=12)
    w = 1 + 0.3 * torch.randn(4, 8, generator=g, dtype=torch.float64)
    ct = torch.randn(9, 12, 8, generator=g, dtype=torch.float64)
    v = torch.randn(9, 12, 8, generator=g, dtype=torch.float64)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    (rg,) = torch.autograd.grad(ref_ops.cpu_layer_rms_norm(xr, info, wr), xr, ct, create_graph=True)
    rgg = torch.autograd.grad(rg, (xr, wr), v)
    dev_info = irreps_info(IRR).to(device)
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    (gd,) = torch.autograd.grad(layer_rms_norm(xd, dev_info, wd), xd, ct.to(device), create_graph=True)
    assert_close(gd, rg, tol=1e-10, what="first order under create_graph")
    gg = torch.autograd.grad(gd, (xd, wd), v.to(device))
    assert_close(gg[0], rgg[0], tol=1e-9, what="second order x")
    assert_close(gg[1], rgg[1], tol=1e-9, what="second order weight")
    big = irreps_info("0e+7o").to(device)
    assert not kernels.layer_rms_supported(big.irrep_seg, 8, torch.float64)
    xb = torch.randn(5, 16, 8, generator=g, dtype=torch.float64)
    ref = ref_ops.cpu_layer_rms_norm(xb, ref_tables.irreps_info("0e+7o"), None)
    assert_close(layer_rms_norm(xb.to(device), big, None), ref, tol=1e-6, what="composed path")


def test_rows_past_two_to_the_31_elements(device):
    """3.8 million rows x 9 x 64 fp32 = 2.19e9 elements: gate, layer norm and squared norm, forward and gradients.
    A row's result depends on its own row only, so rows from both ends of the batch (the last ones lie past 2^31
    elements) must be bit-equal to the same rows computed as a batch of their own."""
    from equitorch_amd.nn import Gate, LayerRMSNorm, SquaredNorm
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 50 GB of device memory")
    n, ch = 3_800_000, 64
    g = torch.Generator(device=device).manual_seed(3)
    x = torch.randn(n, 9, ch, generator=g, device=device).requires_grad_(True)
    assert x.numel() > 2 ** 31
    gate = torch.randn(n, 3, ch, generator=g, device=device).requires_grad_(True)
    ct = torch.randn(n, 9, ch, generator=g, device=device)
    idx = torch.cat([torch.arange(0, 50, device=device), torch.arange(n - 2000, n - 1950, device=device),
                     torch.arange(n - 50, n, device=device)])

    def check(name, fn, inputs, cot):
        out = fn(*inputs)
        grads = torch.autograd.grad(out, inputs, cot)
        small = [t.detach()[idx].clone().requires_grad_(True) for t in inputs]
        outs = fn(*small)
        gs = torch.autograd.grad(outs, small, cot[idx])
        assert torch.equal(out[idx], outs), name
        for a, b in zip(grads, gs):
            assert torch.equal(a[idx], b), name
    check("gate", Gate("0e+1o+2e").to(device), (x, gate), ct)
    check("layer rms norm", LayerRMSNorm("0e+1o+2e", ch).to(device), (x,), ct)
    check("squared norm", SquaredNorm("0e+1o+2e", True).to(device), (x,), torch.randn(n, 3, ch, generator=g, device=device))
    del x, gate, ct
    torch.cuda.empty_cache()


def test_node_layers_past_two_to_the_31_elements(device):
    """The same check (rows at both ends of 3.8 million rows x 9 x 64 fp32 bit-equal to the same rows as a batch of their
    own, forward and input gradient) for the fused Wigner rotation, the channel-wise SO(2) map, the irrep-wise linear
    layer and the batch norm in evaluation mode."""
    import math
    import equitorch_amd.nn as enn
    from equitorch_amd.nn.functional import sincos
    if torch.cuda.get_device_properties(0).total_memory < 80 * 2 ** 30:
        pytest.skip("needs about 50 GB of device memory")
    irr, n, ch = "0e+1o+2e", 3_800_000, 64
    g = torch.Generator(device=device).manual_seed(6)
    x = torch.randn(n, 9, ch, generator=g, device=device).requires_grad_(True)
    ct = torch.randn(n, 9, ch, generator=g, device=device)
    assert x.numel() > 2 ** 31
    idx = torch.cat([torch.arange(0, 50, device=device), torch.arange(n - 50, n, device=device)])

    def check(name, fn):
        out = fn(x, slice(None))
        (gx,) = torch.autograd.grad(out, x, ct)
        xs = x.detach()[idx].clone().requires_grad_(True)
        outs = fn(xs, idx)
        (gxs,) = torch.autograd.grad(outs, xs, ct[idx])
        assert torch.equal(out[idx], outs) and torch.equal(gx[idx], gxs), name
        del out, gx
        torch.cuda.empty_cache()
    sc = [sincos(torch.rand(n, generator=g, device=device) * 2 * math.pi, 2) for _ in range(3)]
    rot = enn.SparseWignerRotation(irr).to(device)
    check("rotation", lambda t, i: rot(t, *(s[i] for s in sc)))
    so2 = enn.SO2Linear(irr, irr, ch, ch, feature_mode="uu").to(device)
    check("so2 uu", lambda t, i: so2(t))
    lin = enn.IrrepsLinear(irr, irr, ch, ch).to(device)
    check("irreps linear", lambda t, i: lin(t))
    bn = enn.BatchRMSNorm(irr, ch).to(device).eval()
    check("batch rms norm (eval)", lambda t, i: bn(t))
    del x, ct
    torch.cuda.empty_cache()
