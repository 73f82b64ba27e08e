"""A whole message-passing layer assembled from the public modules — harmonics of the edge vectors, radial basis and
cutoff, per-edge weights from a small MLP, fused gather / tensor product / scatter, channel mixing, gate and layer
normalisation — forward and backward on the GPU against the same layer written with the oracle's functions in
float64.  Checks that the pieces compose (devices, dtypes, strides, autograd) the way a user of the reference
would combine them."""
import pytest
import torch

from helpers import assert_close
from oracle import ref_ops, ref_sh, ref_tables

pytestmark = pytest.mark.gpu

IRR = "0e+1o+2e"


class Layer(torch.nn.Module):
    def __init__(self, channels, num_basis, r_max):
        super().__init__()
        from equitorch_amd import nn as enn
        self.sh = enn.SphericalHarmonics(2, normalize_input=True)
        self.basis = enn.BesselBasis(r_max, num_basis, trainable=False)
        self.cutoff = enn.PolynomialCutoff(r_max)
        self.tp = enn.SO3Linear(IRR, IRR, IRR, channels, channels, internal_weights=False, feature_mode="uu")
        self.radial = torch.nn.Sequential(torch.nn.Linear(num_basis, 16), torch.nn.SiLU(),
                                          torch.nn.Linear(16, self.tp.num_paths * channels))
        self.mix = enn.IrrepsLinear(IRR, IRR, channels, channels)
        self.gate_lin = enn.IrrepsLinear(IRR, "0e+0e+0e", channels, channels)      # scalars -> one gate per irrep
        self.gate = enn.Gate(IRR, activation=torch.nn.Sigmoid())
        self.norm = enn.LayerRMSNorm(IRR, channels)
        self.channels = channels

    def forward(self, x, edge_vec, plan, fused_harmonics):
        from equitorch_amd.nn.functional import edge_tensor_product_uu, edge_tensor_product_uu_vectors
        r = edge_vec.norm(dim=-1)
        w = self.radial(self.basis(r) * self.cutoff(r)[:, None]).view(-1, self.tp.num_paths, self.channels)
        if fused_harmonics:
            msg = edge_tensor_product_uu_vectors(x, edge_vec, w, plan, self.tp.tp_info_forward)
        else:
            msg = edge_tensor_product_uu(x, self.sh(edge_vec), w, plan, self.tp.tp_info_forward)
        h = self.mix(msg)
        h = self.gate(h, self.gate_lin(h))
        return self.norm(h)


def _reference(layer, x, edge_vec, src, dst, n_nodes, mix_w, radial_w, dtype=torch.float64):
    """The same layer from the oracle's pieces and plain torch, in float64 (the arbiter) or in float32 (what plain
    fp32 arithmetic loses on this computation); the operands come in ``dtype``."""
    P, C = layer.tp.num_paths, layer.channels
    d = lambda t: t.detach().to(dtype).cpu()
    r = edge_vec.norm(dim=-1)
    n = torch.arange(1, layer.basis.num_basis + 1, dtype=dtype)
    basis = (2.0 / layer.basis.r_max) * torch.sin(n * torch.pi * r[:, None] / layer.basis.r_max) / r[:, None]
    u = (r / layer.cutoff.r_max).clamp(0, 1)
    p = layer.cutoff.p
    cut = 1 - (p + 1) * (p + 2) / 2 * u ** p + p * (p + 2) * u ** (p + 1) - p * (p + 1) / 2 * u ** (p + 2)
    lin0, lin1 = layer.radial[0], layer.radial[2]
    h = torch.nn.functional.silu((basis * cut[:, None]) @ d(lin0.weight).T + d(lin0.bias))
    w = (h @ radial_w.T + d(lin1.bias)).view(-1, P, C)
    sh = ref_sh.spherical_harmonics(ref_sh.normalize(edge_vec), 2)
    T = ref_ops.dense_coupling(IRR, IRR, IRR)
    msg = ref_ops.scatter_sum(ref_ops.dense_u1u(T, x[src], sh, w, dtype=dtype), dst, n_nodes)
    f32 = lambda info: {**info, "scale_MM0": torch.tensor(info["scale_MM0"]).double().tolist()}
    mixed = ref_ops.cpu_irreps_linear(msg, mix_w, f32(ref_tables.irreps_linear_infos(IRR, IRR)[0]))
    gates = ref_ops.cpu_irreps_linear(mixed, d(layer.gate_lin.weight),
                                      f32(ref_tables.irreps_linear_infos("0e+0e+0e", IRR)[0]))
    info = ref_tables.irreps_info(IRR)
    info["rdims"] = torch.tensor(info["rdims"]).double().tolist()
    gated = ref_ops.cpu_gating(mixed, torch.sigmoid(gates), info)
    return ref_ops.cpu_layer_rms_norm(gated, info, d(layer.norm.weight))


@pytest.mark.parametrize("fused_harmonics", [False, True])
def test_message_passing_layer(device, fused_harmonics):
    from equitorch_amd.nn.functional import EdgePlan
    torch.manual_seed(0)
    n_nodes, n_edges, channels = 40, 500, 64
    layer = Layer(channels, num_basis=8, r_max=3.0).to(device)
    g = torch.Generator().manual_seed(1)
    src = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g)
    x = torch.randn(n_nodes, 9, channels, generator=g)
    vec = torch.randn(n_edges, 3, generator=g)
    vec = vec / vec.norm(dim=-1, keepdim=True) * (0.5 + 2.0 * torch.rand(n_edges, 1, generator=g))
    ct = torch.randn(n_nodes, 9, channels, generator=g)
    plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
    xd, vd = x.to(device).requires_grad_(True), vec.to(device).requires_grad_(True)
    out = layer(xd, vd, plan, fused_harmonics)
    params = [layer.mix.weight, layer.radial[2].weight]
    grads = torch.autograd.grad(out, [xd, vd] + params, ct.to(device))
    xr, vr = x.double().requires_grad_(True), vec.double().requires_grad_(True)
    mix_w, radial_w = (p.detach().double().cpu().requires_grad_(True) for p in params)
    ref = _reference(layer, xr, vr, src, dst, n_nodes, mix_w, radial_w)
    ref_grads = torch.autograd.grad(ref, [xr, vr, mix_w, radial_w], ct.double())
    # the same reference in float32 arithmetic: the norm-wise comparisons are also held to three times its error
    x32, v32 = x.clone().requires_grad_(True), vec.clone().requires_grad_(True)
    mix32, radial32 = (p.detach().float().cpu().requires_grad_(True) for p in params)
    ref32 = _reference(layer, x32, v32, src, dst, n_nodes, mix32, radial32, dtype=torch.float32)
    ref32_grads = torch.autograd.grad(ref32, [x32, v32, mix32, radial32], ct)
    assert_close(out, ref, tol=1e-5, what="layer output")
    for name, a, b, b32 in zip(("grad_x", "grad_edge_vec", "grad_mix_weight", "grad_radial_weight"), grads, ref_grads,
                               ref32_grads):
        # the parameter gradients sum over all nodes / edges, grad_edge_vec over every channel and coefficient of
        # the layer behind it: norm-wise; grad_x element-wise
        big = name != "grad_x"
        assert_close(a, b, tol=1e-5, what=name, norm="max" if big else "element", fp32_ref=b32 if big else None)
