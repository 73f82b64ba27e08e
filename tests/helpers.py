"""Shared helpers of the test-suite: seeded inputs and the parity criterion."""
import torch

from equitorch_amd.utils._sh import spherical_harmonics


def assert_close(actual, expected, tol=1e-5, what=""):
    """``max|a - b| <= tol * max(1, max|b|)``: absolute ``tol`` for O(1) tensors, relative to the tensor's
    largest magnitude above that (rel/abs 1e-5 for fp32 results, per the parity bar of this path)."""
    a = actual.detach().double().cpu()
    b = expected.detach().double().cpu()
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    if b.numel() == 0:
        return
    scale = max(1.0, float(b.abs().max()))
    err = float((a - b).abs().max())
    assert err <= tol * scale, f"{what}: max abs err {err:.3e} > {tol:.0e} * {scale:.3e}"


def unit_vectors(n, gen):
    v = torch.randn(n, 3, generator=gen)
    return v / v.norm(dim=-1, keepdim=True)


def tp_inputs(n, d1, lmax2, n_paths, channels, shared_w, seed=0, dtype=torch.float32):
    """Seeded (x, sh, W) on the CPU: x ~ N(0,1) (n, d1, C); sh = harmonics of random unit vectors; W ~ N(0,1)."""
    gen = torch.Generator().manual_seed(seed)
    x = torch.randn(n, d1, channels, generator=gen)
    sh = spherical_harmonics(unit_vectors(n, gen), lmax2)
    w = torch.randn(*(() if shared_w else (n,)), n_paths, channels, generator=gen)
    return x.to(dtype), sh.to(dtype), w.to(dtype)
