"""Shared helpers of the test-suite: seeded inputs and the parity criterion."""
import os

import torch

from equitorch_amd.utils._sh import spherical_harmonics


PARITY_LOG = []      # (test id, what, tol, worst |a-b| / (1 + |b|), worst |a-b| / max(1, max|b|)) of every comparison


def assert_close(actual, expected, tol=1e-5, what="", norm="element"):
    """The parity criterion.  ``norm="element"`` (default): ``|a - b| <= tol * (1 + |b|)`` for every element — the
    rel/abs bound of this path (1e-5 for fp32 results and gradients).  ``norm="max"``: ``max|a - b| <= tol *
    max(1, max|b|)``, for results that are long fp32 sums (over a batch, over the edges of a node, over hundreds of
    coefficients): their rounding error scales with the magnitude of the sum's terms, not with the individual
    element, so entries that cancel to small values cannot meet an element-wise relative bound in fp32 arithmetic;
    every such call site says what is summed.  Either way the worst element-wise and norm-wise ratios of every
    comparison are kept in ``PARITY_LOG`` (written to a file by the suite when ``CGTP_PARITY_REPORT`` names one)."""
    a = actual.detach().double().cpu()
    b = expected.detach().double().cpu()
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    if b.numel() == 0:
        return
    diff = (a - b).abs()
    elem = float((diff / (1.0 + b.abs())).max())
    scale = max(1.0, float(b.abs().max()))
    err = float(diff.max())
    PARITY_LOG.append((os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0], what, tol, elem, err / scale))
    if norm == "element":
        assert elem <= tol, f"{what}: worst |a-b| / (1 + |b|) = {elem:.3e} > {tol:.0e} (max abs err {err:.3e})"
    else:
        assert norm == "max", norm
        assert err <= tol * scale, f"{what}: max abs err {err:.3e} > {tol:.0e} * {scale:.3e}"


def stable_seed(*key) -> int:
    """Seed derived from a test's parameters; the same in every process (``hash`` of a str is not)."""
    import zlib
    return zlib.crc32(repr(key).encode()) % 2 ** 31


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
