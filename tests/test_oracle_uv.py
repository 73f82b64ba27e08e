"""Pins of the fully connected members of the numeric oracle (``dense_u1v``, ``dense_uvw``, ``dense_uuu``) and of
the structural restatement of the reference's CPU path for them (``cpu_outer``, ``cpu_vecmat``, ``cpu_mat_t_vec``,
``cpu_u1v_* / cpu_1vu_* / cpu_vu1_* / cpu_uvw_* / cpu_uuu_*``): special cases that reduce to library routines
(``x @ W``, ``torch.outer``, slices), and agreement of the two independent restatements in float64."""
import pytest
import torch

from helpers import assert_close, unit_vectors
from oracle import ref_ops, ref_tables

SH2 = "0e+1o+2e"
SH3 = "0e+1o+2e+3o"


def _rand(gen, *shape):
    return torch.randn(*shape, generator=gen, dtype=torch.float64)


def test_dense_u1v_at_lmax0_is_a_matrix_product():
    g = torch.Generator().manual_seed(0)
    T = ref_ops.dense_coupling("0e", "0e", "0e")
    assert T.shape == (1, 1, 1, 1) and float(T) == 1.0
    x, w = _rand(g, 9, 1, 7), _rand(g, 1, 7, 5)
    y = torch.ones(9, 1, dtype=torch.float64)
    torch.testing.assert_close(ref_ops.dense_u1v(T, x, y, w)[:, 0], x[:, 0] @ w[0])
    yv = _rand(g, 9, 1)
    torch.testing.assert_close(ref_ops.dense_u1v(T, x, yv, w)[:, 0], yv * (x[:, 0] @ w[0]))
    wn = _rand(g, 9, 1, 7, 5)                        # per-sample weight
    torch.testing.assert_close(ref_ops.dense_u1v(T, x, y, wn)[:, 0], torch.einsum("nu,nuv->nv", x[:, 0], wn[:, 0]))


@pytest.mark.parametrize("irreps", [SH2, SH3])
def test_dense_u1v_l2_zero_paths_are_scaled_block_products(irreps):
    """With the second operand reduced to its scalar part, path p: (l, l, 0) maps block l of x through W[p]:
    ``out[:, block] = y0 * x[:, block] @ W[p]`` (path_norm=False: each output irrep has a single such path)."""
    g = torch.Generator().manual_seed(1)
    T = ref_ops.dense_coupling(irreps, irreps, "0e", path_norm=False)
    lmax = T.shape[0] - 1
    d = (lmax + 1) ** 2
    x, y, w = _rand(g, 6, d, 5), _rand(g, 6, 1), _rand(g, lmax + 1, 5, 4)
    out = ref_ops.dense_u1v(T, x, y, w)
    for l in range(lmax + 1):
        s = slice(l * l, (l + 1) ** 2)
        torch.testing.assert_close(out[:, s], y[:, :, None] * (x[:, s] @ w[l]))


def test_dense_u1v_path_norm_scales_paths_by_count():
    """path_norm divides every path of output irrep k by sqrt(number of paths into k) (utils/_structs.py:177-206)."""
    T1 = ref_ops.dense_coupling(SH2, SH2, SH2, path_norm=True)
    T0 = ref_ops.dense_coupling(SH2, SH2, SH2, path_norm=False)
    counts = [3, 4, 4]                               # paths into l = 0, 1, 2 (lmax = 2)
    paths = ref_tables.fully_connected_paths(*(ref_tables.parse(SH2),) * 3)
    for p, (k, _, _) in enumerate(paths):
        torch.testing.assert_close(T1[p], T0[p] / counts[k] ** 0.5)


def test_dense_uvw_reductions():
    """uvw with one channel on the second operand is u1v; with 'diagonal' weights it is uuu; with one channel
    everywhere all three agree with u1u."""
    g = torch.Generator().manual_seed(2)
    T = ref_ops.dense_coupling(SH2, SH2, "0e+1o")
    p, n, u, w_ = T.shape[0], 5, 4, 3
    x, y, wt = _rand(g, n, 9, u), _rand(g, n, 4), _rand(g, p, u, w_)
    torch.testing.assert_close(ref_ops.dense_uvw(T, x, y[:, :, None], wt[:, :, None, :]), ref_ops.dense_u1v(T, x, y, wt))
    yc, wc = _rand(g, n, 4, u), _rand(g, p, u)
    diag = torch.zeros(p, u, u, u, dtype=torch.float64)
    idx = torch.arange(u)
    diag[:, idx, idx, idx] = wc
    torch.testing.assert_close(ref_ops.dense_uvw(T, x, yc, diag), ref_ops.dense_uuu(T, x, yc, wc))
    torch.testing.assert_close(ref_ops.dense_uuu(T, x[:, :, :1], yc[:, :, :1], wc[:, :1]),
                               ref_ops.dense_u1u(T, x[:, :, :1], yc[:, :, 0], wc[:, :1]))
    # per-sample weights: the shared result with the weight repeated
    wn = wt.unsqueeze(0).expand(n, -1, -1, -1).contiguous()
    torch.testing.assert_close(ref_ops.dense_u1v(T, x, y, wn), ref_ops.dense_u1v(T, x, y, wt))


def test_cpu_outer_and_vecmat_against_library_routines():
    """Identity tables: the operators reduce to ``torch.outer`` / ``@`` row by row; with a table, to a loop over
    its entries."""
    g = torch.Generator().manual_seed(3)
    n, m, u, v = 4, 6, 3, 5
    ident = dict(scale=None, index1=None, index2=None, seg_out=None)
    x, y = _rand(g, n, m, u), _rand(g, n, m, v)
    out = ref_ops.cpu_outer(x, y, ident)
    for i in range(n):
        for j in range(m):
            torch.testing.assert_close(out[i, j], torch.outer(x[i, j], y[i, j]))
    mat = _rand(g, m, u, v)
    out = ref_ops.cpu_vecmat(x, mat, ident)
    for j in range(m):
        torch.testing.assert_close(out[:, j], x[:, j] @ mat[j])
    torch.testing.assert_close(ref_ops.cpu_mat_t_vec(mat, x, ident), out)
    torch.testing.assert_close(ref_ops.cpu_outer(x, y, ident, out_accumulated=True), out.new_zeros(()) +
                               torch.einsum("nmu,nmv->muv", x, y))
    # a table with repeated and skipped indices, two entries per output row except an empty one
    info = dict(scale=torch.tensor([0.5, -2.0, 3.0, 1.5], dtype=torch.float64), index1=torch.tensor([0, 5, 2, 2]),
                index2=torch.tensor([1, 1, 4, 0]), seg_out=torch.tensor([0, 2, 2, 4]))
    out = ref_ops.cpu_vecmat(x, mat, info)
    want0 = 0.5 * x[:, 0] @ mat[1] - 2.0 * x[:, 5] @ mat[1]
    want2 = 3.0 * x[:, 2] @ mat[4] + 1.5 * x[:, 2] @ mat[0]
    torch.testing.assert_close(out[:, 0], want0)
    torch.testing.assert_close(out[:, 1], torch.zeros_like(want0))
    torch.testing.assert_close(out[:, 2], want2)
    out = ref_ops.cpu_outer(x, y, info)
    want0 = 0.5 * torch.einsum("nu,nv->nuv", x[:, 0], y[:, 1]) - 2.0 * torch.einsum("nu,nv->nuv", x[:, 5], y[:, 1])
    torch.testing.assert_close(out[:, 0], want0)


TRIPLES = [(SH2, SH2, SH2), ("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e"), ("1o+2e+1e", "0e+1o+2e", "0e+1o"), (SH3, SH3, SH3)]


@pytest.mark.parametrize("irreps", TRIPLES)
@pytest.mark.parametrize("shared_w", [True, False])
def test_structural_u1v_chain_matches_dense(irreps, shared_w):
    """vecsca -> vecmat and the reference's backward chain (1vu, vu1 with its weight-first order, accumulated
    outer) against the dense einsum and autograd, float64, 1e-12."""
    io, i1, i2 = irreps
    fwd, b1, b2, n_paths = ref_tables.tp_infos(io, i1, i2)
    fwd, b1, b2 = (ref_ops.tables_to_torch(t, torch.float64) for t in (fwd, b1, b2))
    d1, d2 = fwd["info_Mij_bwd1"]["out_size"], fwd["info_Mij_bwd2"]["out_size"]
    g = torch.Generator().manual_seed(5)
    n, u, v = 7, 4, 3
    x, y = _rand(g, n, d1, u), _rand(g, n, d2)
    w = _rand(g, *(() if shared_w else (n,)), n_paths, u, v)
    ct = _rand(g, n, fwd["out_size"], v)
    out, inter = ref_ops.cpu_u1v_forward(x, y, w, fwd)
    gx, gy, gw = ref_ops.cpu_u1v_backward(ct, x, y, w, inter, fwd, b1, b2)
    T = ref_ops.dense_coupling(io, i1, i2)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1v, T, (x, y, w), ct)
    for name, a, b in (("out", out, ref_out), ("gx", gx, ref_grads[0]), ("gy", gy, ref_grads[1]),
                       ("gw", gw, ref_grads[2])):
        assert_close(a, b, 1e-12, name)


@pytest.mark.parametrize("irreps", TRIPLES[:3])
@pytest.mark.parametrize("shared_w", [True, False])
def test_structural_uvw_and_uuu_chains_match_dense(irreps, shared_w):
    io, i1, i2 = irreps
    fwd, b1, b2, n_paths = ref_tables.tp_infos(io, i1, i2)
    fwd, b1, b2 = (ref_ops.tables_to_torch(t, torch.float64) for t in (fwd, b1, b2))
    d1, d2 = fwd["info_Mij_bwd1"]["out_size"], fwd["info_Mij_bwd2"]["out_size"]
    g = torch.Generator().manual_seed(6)
    n, u, v, w_ = 5, 3, 2, 4
    lead = () if shared_w else (n,)
    x, y = _rand(g, n, d1, u), _rand(g, n, d2, v)
    w = _rand(g, *lead, n_paths, u, v, w_)
    ct = _rand(g, n, fwd["out_size"], w_)
    out, inter = ref_ops.cpu_uvw_forward(x, y, w, fwd)
    gx, gy, gw = ref_ops.cpu_uvw_backward(ct, x, y, w, inter, fwd, b1, b2)
    T = ref_ops.dense_coupling(io, i1, i2)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_uvw, T, (x, y, w), ct)
    for name, a, b in (("out", out, ref_out), ("gx", gx, ref_grads[0]), ("gy", gy, ref_grads[1]),
                       ("gw", gw, ref_grads[2])):
        assert_close(a, b, 1e-12, "uvw " + name)
    yc, wc = _rand(g, n, d2, u), _rand(g, *lead, n_paths, u)
    out, _ = ref_ops.cpu_uuu_forward(x, yc, wc, fwd)
    assert_close(out, ref_ops.dense_uuu(T, x, yc, wc), 1e-12, "uuu out")


def test_dense_u1v_is_equivariant():
    """O(3) equivariance of the fully connected product for arbitrary weights (Wigner-D from the harmonics)."""
    from oracle.ref_sh import spherical_harmonics
    from test_oracle import _wigner_from_harmonics
    q, _ = torch.linalg.qr(torch.randn(3, 3, generator=torch.Generator().manual_seed(9), dtype=torch.float64))
    rot = -q * torch.sign(torch.linalg.det(q))       # improper: parities matter
    d = _wigner_from_harmonics(rot, 3)
    g = torch.Generator().manual_seed(10)
    v = unit_vectors(8, g).double()
    x, w = _rand(g, 8, 16, 3), _rand(g, 23, 3, 2)
    T = ref_ops.dense_coupling(SH3, SH3, SH3)
    out = ref_ops.dense_u1v(T, x, spherical_harmonics(v, 3), w)
    out_rot = ref_ops.dense_u1v(T, torch.einsum("ab,nbc->nac", d, x), spherical_harmonics(v @ rot.T, 3), w)
    torch.testing.assert_close(out_rot, torch.einsum("ab,nbc->nac", d, out), atol=1e-10, rtol=1e-10)
