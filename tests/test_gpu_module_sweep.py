"""Random sweep of the channel-mixing, gate, norm and SO(2) modules against the oracle's restatement of the
reference's forwards (``ref_ops.cpu_*`` on the oracle's own tables), gradients by autograd of the oracle: irreps,
channel counts (1 to 128, multiples of 4 or not), batch sizes, fp32 / fp64, shared and per-sample weights drawn at
random.  fp32 2e-5 norm-wise (sums over up to 128 input channels and several paths), fp64 1e-10.  The fixed cases of
the other test files cover the shapes the kernels were tuned on; this one covers the combinations nobody thought of
(it found the tables the reference's builder leaves incomplete, ``test_gpu_rotation.py``)."""
import random

import pytest
import torch

from oracle import ref_ops, ref_tables

pytestmark = pytest.mark.gpu

POOL = ["0e", "1o", "0e+1o", "0e+1o+2e", "0e+1o+2e+3o", "1o+2e", "0e+0e+1o", "2e+0e", "0e+1e+2e", "1o+1e",
        "2x0e+1o+3x2e", "0e+1o+1o+2e+0e", "0e+1o+2e+3o+4e"]


def _f32(d, keys):
    """Factors as the reference stores them: fp32 values (``torch.tensor(list)``), also under fp64 features."""
    d = dict(d)
    for k in keys:
        if d.get(k) is not None:
            d[k] = torch.tensor(d[k]).double().tolist()
    return d


def _worst(a, b):
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    assert a.shape == b.shape, (a.shape, b.shape)
    return 0.0 if b.numel() == 0 else float((a - b).abs().max() / max(1.0, float(b.abs().max())))


@pytest.mark.parametrize("seed", [31, 32, 33])
def test_modules_against_the_oracle(device, seed):
    from equitorch_amd import nn as enn
    from equitorch_amd.irreps import Irreps
    rnd, bad = random.Random(seed), []
    for it in range(40):
        kind = rnd.choice(["linear", "linear", "wise", "gate", "norms", "rms", "so2uu", "so2uv"])
        dtype = rnd.choice([torch.float32, torch.float32, torch.float64])
        tol = 2e-5 if dtype == torch.float32 else 1e-10
        n = rnd.choice([1, 2, 17, 64, 300, 1100])
        cin = rnd.choice([1, 2, 3, 4, 8, 12, 16, 20, 32, 33, 64, 128])
        cout = rnd.choice([1, 3, 4, 8, 16, 24, 32, 64, 65, 128])
        ii, io = rnd.choice(POOL), rnd.choice(POOL)
        per_sample = rnd.random() < 0.3
        tag = f"seed {seed} case {it}: {kind} {ii} -> {io}, {cin} -> {cout}, n {n}, {dtype}, per_sample {per_sample}"
        print(tag, flush=True)
        g = torch.Generator().manual_seed(seed * 1000 + it)
        rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
        dim_in, blocks = Irreps(ii).dim, len(Irreps(ii))
        info = _f32(ref_tables.irreps_info(ii), ["rdims", "rsqrt_dims"])
        if kind == "linear":
            try:
                mod = enn.IrrepsLinear(ii, io, cin, cout, internal_weights=False).to(device)
            except Exception:       # no path between these irreps: the reference's constructor raises as well
                continue
            lin = _f32(ref_tables.irreps_linear_infos(io, ii)[0], ["scale_MM0"])
            ops = (rd(n, dim_in, cin), rd(*((n,) if per_sample else ()), mod.num_paths, cin, cout))
            ref_fn, fn = (lambda x, w: ref_ops.cpu_irreps_linear(x, w, lin)), (lambda x, w: mod(x, w))
        elif kind == "wise":
            mod = enn.IrrepWiseLinear(ii, cin, cout, internal_weights=False).to(device)
            ops = (rd(n, dim_in, cin), rd(*((n,) if per_sample else ()), blocks, cin, cout))
            ref_fn, fn = (lambda x, w: ref_ops.cpu_irrep_wise_linear(x, w, info)), (lambda x, w: mod(x, w))
        elif kind == "gate":
            mod = enn.Gate(ii, activation=torch.nn.Sigmoid()).to(device)
            ops = (rd(n, dim_in, cin), rd(*(() if per_sample else (n,)), blocks, cin))      # a gate shared by the batch
            ref_fn, fn = (lambda x, gt: ref_ops.cpu_gating(x, torch.sigmoid(gt), info)), (lambda x, gt: mod(x, gt))
        elif kind == "norms":
            scaled, which = rnd.random() < 0.5, rnd.choice(["sq", "norm", "cm", "bm"])
            mod = {"sq": lambda: enn.SquaredNorm(ii, scaled), "norm": lambda: enn.Norm(ii, scaled),
                   "cm": lambda: enn.MeanSquaredNorm(ii, scaled, dim=-1),
                   "bm": lambda: enn.MeanSquaredNorm(ii, scaled, dim=0)}[which]().to(device)
            rf = {"sq": ref_ops.cpu_squared_norm, "norm": ref_ops.cpu_norm, "cm": ref_ops.cpu_channel_mean_squared_norm,
                  "bm": ref_ops.cpu_batch_mean_squared_norm}[which]
            ops = (rd(n, dim_in, cin),)
            ref_fn, fn = (lambda x: rf(x, info, scaled)), (lambda x: mod(x))
        elif kind == "rms":
            affine = rnd.random() < 0.6
            mod = enn.LayerRMSNorm(ii, cin, affine=affine).to(device).to(dtype)
            wt = rd(blocks, cin) if affine else None
            if affine:
                with torch.no_grad():
                    mod.weight.copy_(wt.to(device, dtype))
            ops = (rd(n, dim_in, cin),)
            ref_fn, fn = (lambda x: ref_ops.cpu_layer_rms_norm(x, info, wt)), (lambda x: mod(x))
        else:
            mode = kind[-2:]
            co = cin if mode == "uu" else cout
            mod = enn.SO2Linear(ii, io, cin, co, internal_weights=False, feature_mode=mode).to(device)
            so2 = _f32(ref_tables.so2_linear_infos(io, ii)[0], ["scale"])
            wshape = (mod.num_weights, co) if mode == "uu" else (mod.num_weights, cin, co)
            ops = (rd(n, dim_in, cin), rd(*((n,) if per_sample else ()), *wshape))
            ref_fn = lambda x, w: ref_ops.cpu_so2_linear(x, w, so2, per_sample=per_sample)
            fn = lambda x, w: mod(x, w)
        refs = [t.clone().requires_grad_(True) for t in ops]
        ref = ref_fn(*refs)
        ct = rd(*ref.shape)
        ref_grads = [torch.nan_to_num(t) for t in torch.autograd.grad(ref, refs, ct)]     # norm of a zero block: 0
        devs = [t.to(device, dtype).requires_grad_(True) for t in ops]
        scratch = [torch.full_like(t, 1e3) for t in devs]        # what the allocator hands out next is not zeros
        del scratch
        out = fn(*devs)
        grads = torch.autograd.grad(out, devs, ct.to(device, dtype))
        errs = [_worst(out, ref)] + [_worst(a, b) for a, b in zip(grads, ref_grads)]
        if max(errs) > tol or not all(bool(torch.isfinite(t).all()) for t in (out, *grads)):
            bad.append((tag, errs))
    assert not bad, "\n".join(map(str, bad))
