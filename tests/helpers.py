"""Shared helpers of the test-suite: seeded inputs and the parity criterion."""
import os

import torch

from equitorch_amd.utils._sh import spherical_harmonics


PARITY_LOG = []      # (test id, what, tol, worst |a-b| / (1 + |b|), worst |a-b| / max(1, max|b|)) of every comparison


def assert_close(actual, expected, tol=1e-5, what="", norm="element", fp32_ref=None):
    """The parity criterion.  ``norm="element"`` (default): ``|a - b| <= tol * (1 + |b|)`` for every element — the
    rel/abs bound of this path (1e-5 for fp32 results and gradients).  ``norm="max"``: ``max|a - b| <= tol *
    max(1, max|b|)``, for results that are long fp32 sums (over a batch, over the edges of a node, over hundreds of
    coefficients): their rounding error scales with the magnitude of the sum's terms, not with the individual
    element, so entries that cancel to small values cannot meet an element-wise relative bound in fp32 arithmetic;
    every such call site says what is summed.

    ``fp32_ref``: the same reference computation carried out in fp32 arithmetic on the same inputs (the oracle's
    functions run on float32 tensors, see :func:`fp32_twin`).  With it a norm-wise comparison does not rest on the
    tensor's maximum alone: every element must also satisfy ``|a - b| <= 3 * E32 + tol * (1 + |b|)``, where
    ``E32 = max|fp32_ref - b|`` is what plain fp32 arithmetic itself loses on this computation — the kernel may not
    err more than three times what the fp32 restatement of the reference does (a different but equally valid
    order of the same fp32 additions moves the worst element by a small factor: 2.6 is the largest seen), plus the
    element-wise allowance.

    Either way the worst element-wise and norm-wise ratios of every comparison, and the fp32 restatement's own worst
    element-wise ratio where one was given, are kept in ``PARITY_LOG`` (written to a file by the suite when
    ``CGTP_PARITY_REPORT`` names one)."""
    a = actual.detach().double().cpu()
    b = expected.detach().double().cpu()
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    if b.numel() == 0:
        return
    diff = (a - b).abs()
    elem = float((diff / (1.0 + b.abs())).max())
    scale = max(1.0, float(b.abs().max()))
    err = float(diff.max())
    ref_elem = None
    if fp32_ref is not None:
        r = fp32_ref.detach().double().cpu()
        assert r.shape == b.shape, f"{what}: fp32 reference has shape {tuple(r.shape)}, expected {tuple(b.shape)}"
        rdiff = (r - b).abs()
        ref_elem = float((rdiff / (1.0 + b.abs())).max())
        e32 = float(rdiff.max())
    PARITY_LOG.append((os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0], what, tol, elem, err / scale, ref_elem))
    if norm == "element":
        assert elem <= tol, f"{what}: worst |a-b| / (1 + |b|) = {elem:.3e} > {tol:.0e} (max abs err {err:.3e})"
    else:
        assert norm == "max", norm
        assert err <= tol * scale, f"{what}: max abs err {err:.3e} > {tol:.0e} * {scale:.3e}"
        if fp32_ref is not None:
            excess = float((diff - 3.0 * e32 - tol * (1.0 + b.abs())).max())
            assert excess <= 0.0, (f"{what}: an element errs {excess:.3e} more than 3 x the fp32 restatement's worst "
                                   f"error ({e32:.3e}) + {tol:.0e} * (1 + |b|)")


def fp32_twin(fn, *args, **kwargs):
    """``fn(*args, **kwargs)`` with every floating-point tensor among the arguments (also inside tuples, lists and
    dicts) cast to float32, leaves that require gradients again: the oracle's computation in the arithmetic the
    reference's own fp32 path uses.  Returns what ``fn`` returns."""
    def cast(v):
        if isinstance(v, torch.Tensor):
            if v.is_floating_point():
                t = v.detach().float()
                return t.requires_grad_(True) if v.requires_grad else t
            return v
        if isinstance(v, dict):
            return {k: cast(x) for k, x in v.items()}
        if isinstance(v, (tuple, list)):
            return type(v)(cast(x) for x in v)
        return v
    return fn(*cast(args), **cast(kwargs))


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
