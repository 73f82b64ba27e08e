"""The library under HIP graph capture: every entry point launches on the caller's stream, allocates through the
caller's allocator only and never synchronises, so a whole forward + backward can be recorded once with
``torch.cuda.graph`` and replayed.  Each test replays the graph several times with new inputs, with eager work and
synchronisations of the program between the replays, and checks every replay against the eager result of the same
inputs (the kernels are deterministic, so the two agree to rounding of the library GEMMs around them)."""
import pytest
import torch

from helpers import assert_close
from test_gpu_layer import IRR, Layer

pytestmark = pytest.mark.gpu


def _capture(step, warmup=3):
    """Warm up on a side stream of default priority (tables, plans and workspaces are built there), then record."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(warmup):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        results = step()
    return graph, results


def _check_replays(graph, recorded, statics, fresh_inputs, eager, n_replays=4, tol=1e-6):
    for trial in range(n_replays):
        new = fresh_inputs(trial)
        for s, n in zip(statics, new):
            s.detach().copy_(n)
        graph.replay()
        torch.cuda.synchronize()
        got = [r.clone() for r in recorded]
        expect = eager(*[n.clone().requires_grad_(s.requires_grad) for s, n in zip(statics, new)])
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, expect)):
            assert_close(a, b, tol=tol, what=f"replay {trial}, result {i}")


def test_message_passing_layer_under_graph_capture(device):
    from equitorch_amd.nn.functional import EdgePlan
    torch.manual_seed(0)
    n_nodes, n_edges, channels = 256, 4096, 64
    layer = Layer(channels, num_basis=8, r_max=3.0).to(device)
    g = torch.Generator().manual_seed(3)
    src = torch.randint(0, n_nodes, (n_edges,), generator=g).to(device)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g).to(device)
    plan = EdgePlan(src, dst, n_nodes)
    params = [layer.mix.weight, layer.radial[2].weight, layer.norm.weight]

    def inputs(seed):
        gg = torch.Generator().manual_seed(100 + seed)
        x = torch.randn(n_nodes, 9, channels, generator=gg)
        vec = torch.randn(n_edges, 3, generator=gg)
        vec = vec / vec.norm(dim=-1, keepdim=True) * (0.5 + 2.0 * torch.rand(n_edges, 1, generator=gg))
        ct = torch.randn(n_nodes, 9, channels, generator=gg)
        return x.to(device), vec.to(device), ct.to(device)

    def run(x, vec, ct):
        out = layer(x, vec, plan, True)
        return (out, *torch.autograd.grad(out, [x, vec] + params, ct))

    x, vec, ct = inputs(-1)
    x.requires_grad_(True)
    vec.requires_grad_(True)
    graph, recorded = _capture(lambda: run(x, vec, ct))
    _check_replays(graph, recorded, (x, vec, ct), inputs, run)


def test_element_wise_modules_and_rotation_under_graph_capture(device):
    """Gate, squared norm, layer normalisation, harmonics with their gradient, and the fused Wigner rotation with the
    gradients of its angles' sincos tensors in one recorded graph."""
    from equitorch_amd import nn as enn
    torch.manual_seed(1)
    n, channels = 3000, 64
    gate = enn.Gate(IRR).to(device)
    sq = enn.SquaredNorm(IRR).to(device)
    norm = enn.LayerRMSNorm(IRR, channels).to(device)
    rot = enn.SparseWignerRotation(IRR).to(device)
    sincos = enn.SinCos(2)
    sh = enn.SphericalHarmonics(2, normalize_input=True).to(device)

    def inputs(seed):
        gg = torch.Generator().manual_seed(200 + seed)
        x = torch.randn(n, 9, channels, generator=gg)
        gates = torch.randn(n, 3, channels, generator=gg)
        angles = torch.rand(n, 3, generator=gg) * 6.0 - 3.0
        vec = torch.randn(n, 3, generator=gg)
        return x.to(device), gates.to(device), angles.to(device), vec.to(device)

    def run(x, gates, angles, vec):
        h = norm(gate(x, gates))
        h = rot(h, sincos(angles[:, 0]), sincos(angles[:, 1]), sincos(angles[:, 2]))
        y = sh(vec)
        loss = (h * y[:, :, None]).sum() + sq(h).square().mean()
        return (h, y, *torch.autograd.grad(loss, [x, gates, angles, vec, norm.weight]))

    statics = list(inputs(-1))
    for s in statics:
        s.requires_grad_(True)
    graph, recorded = _capture(lambda: run(*statics))
    _check_replays(graph, recorded, statics, inputs, run, tol=2e-6)
