"""Pins of the numeric oracle: the dense float64 einsum oracle against textbook identities, O(3)
equivariance and autograd's own gradcheck, and the structural restatement of the reference's CPU path against
the dense oracle."""
import pytest
import torch

from helpers import assert_close, tp_inputs, unit_vectors
from oracle import ref_ops, ref_tables

SH2 = "0e+1o+2e"


def test_l2_zero_paths_scale_x():
    """Every path with l2 = 0 multiplies x by y0 * W (times the path normalisation)."""
    T = ref_ops.dense_coupling(SH2, SH2, "0e", path_norm=False)
    x, _, w = tp_inputs(7, 9, 0, 3, 5, True, seed=1, dtype=torch.float64)
    y = torch.randn(7, 1, dtype=torch.float64)
    out = ref_ops.dense_u1u(T, x, y, w)
    blocks = [(0, 1, 0), (1, 4, 1), (4, 9, 2)]
    for lo, hi, p in blocks:
        torch.testing.assert_close(out[:, lo:hi], x[:, lo:hi] * y[:, :, None] * w[p])


def test_dot_and_cross_product_paths():
    g = torch.Generator().manual_seed(3)
    a, b = torch.randn(6, 3, generator=g, dtype=torch.float64), torch.randn(6, 3, generator=g, dtype=torch.float64)
    yzx = [1, 2, 0]
    T0 = ref_ops.dense_coupling("0e", "1o", "1o", path_norm=False)
    out = ref_ops.dense_u1u(T0, a[:, yzx, None], b[:, yzx], torch.ones(1, 1, dtype=torch.float64))
    torch.testing.assert_close(out[:, 0, 0], (a * b).sum(-1) / 3 ** 0.5)
    T1 = ref_ops.dense_coupling((1, 1), (1, 1), (1, 1), path_norm=False)   # SO(3), no parity: 1 x 1 -> 1 exists
    out = ref_ops.dense_u1u(T1, a[:, yzx, None], b[:, yzx], torch.ones(1, 1, dtype=torch.float64))
    torch.testing.assert_close(out[:, :, 0], torch.linalg.cross(a, b)[:, yzx] / 2 ** 0.5)


def _wigner_from_harmonics(rot, lmax):
    """Block-diagonal D with Y(R v) = D Y(v), solved by least squares from the harmonics themselves."""
    from oracle.ref_sh import spherical_harmonics
    v = unit_vectors(400, torch.Generator().manual_seed(11)).double()
    y, yr = spherical_harmonics(v, lmax), spherical_harmonics(v @ rot.T, lmax)
    d = torch.zeros((lmax + 1) ** 2, (lmax + 1) ** 2, dtype=torch.float64)
    for l in range(lmax + 1):
        s = slice(l * l, (l + 1) ** 2)
        d[s, s] = torch.linalg.lstsq(y[:, s], yr[:, s]).solution.T
    return d


def test_dense_oracle_is_equivariant():
    q, _ = torch.linalg.qr(torch.randn(3, 3, generator=torch.Generator().manual_seed(5), dtype=torch.float64))
    for rot in (q * torch.sign(torch.linalg.det(q)), -q * torch.sign(torch.linalg.det(q))):  # proper, improper
        d = _wigner_from_harmonics(rot, 2)
        from oracle.ref_sh import spherical_harmonics
        g = torch.Generator().manual_seed(6)
        v = unit_vectors(9, g).double()
        x = torch.randn(9, 9, 4, generator=g, dtype=torch.float64)
        w = torch.randn(11, 4, generator=g, dtype=torch.float64)
        T = ref_ops.dense_coupling(SH2, SH2, SH2)
        out = ref_ops.dense_u1u(T, x, spherical_harmonics(v, 2), w)
        out_rot = ref_ops.dense_u1u(T, torch.einsum("ab,nbc->nac", d, x), spherical_harmonics(v @ rot.T, 2), w)
        torch.testing.assert_close(out_rot, torch.einsum("ab,nbc->nac", d, out), atol=1e-10, rtol=1e-10)


@pytest.mark.parametrize("irreps", [(SH2, SH2, SH2), ("0e+1e+2e+3e", "0e+1e+2e", "0e+1e+2e"),
                                    ("1o+2e+1e", "0e+1o+2e", "0e+1o")])
@pytest.mark.parametrize("shared_w", [False, True])
def test_structural_cpu_path_matches_dense(irreps, shared_w):
    io, i1, i2 = irreps
    fwd, b1, b2, n_paths = ref_tables.tp_infos(io, i1, i2)
    fwd, b1, b2 = (ref_ops.tables_to_torch(t, torch.float64) for t in (fwd, b1, b2))
    d1, d2 = fwd["info_Mij_bwd1"]["out_size"], fwd["info_Mij_bwd2"]["out_size"]
    g = torch.Generator().manual_seed(2)
    n, c = 13, 6
    x = torch.randn(n, d1, c, generator=g, dtype=torch.float64)
    y = torch.randn(n, d2, generator=g, dtype=torch.float64)
    w = torch.randn(*(() if shared_w else (n,)), n_paths, c, generator=g, dtype=torch.float64)
    ct = torch.randn(n, fwd["out_size"], c, generator=g, dtype=torch.float64)
    out, inter = ref_ops.cpu_u1u_forward(x, y, w, fwd)
    gx, gy, gw = ref_ops.cpu_u1u_backward(ct, x, y, w, inter, fwd, b1, b2)
    T = ref_ops.dense_coupling(io, i1, i2)
    ref_out, ref_grads = ref_ops.dense_grads(ref_ops.dense_u1u, T, (x, y, w), ct)
    for name, a, b in (("out", out, ref_out), ("gx", gx, ref_grads[0]), ("gy", gy, ref_grads[1]),
                       ("gw", gw, ref_grads[2])):
        assert_close(a, b, 1e-12, name)


def test_structural_edge_path_matches_dense():
    fwd, b1, b2, _ = ref_tables.tp_infos(SH2, SH2, SH2)
    fwd, b1, b2 = (ref_ops.tables_to_torch(t, torch.float64) for t in (fwd, b1, b2))
    g = torch.Generator().manual_seed(4)
    n_nodes, n_edges, c = 9, 50, 4
    src = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g)
    info, _ = ref_tables.sparse_scale_infos(index=list(range(n_edges)), index_out=dst.tolist(), out_size=n_nodes,
                                            in_size=n_edges)
    perm, ptr = torch.tensor(info["index"]), torch.tensor(info["seg_out"])
    x = torch.randn(n_nodes, 9, c, generator=g, dtype=torch.float64)
    y = torch.randn(n_edges, 9, generator=g, dtype=torch.float64)
    w = torch.randn(n_edges, 11, c, generator=g, dtype=torch.float64)
    ct = torch.randn(n_nodes, 9, c, generator=g, dtype=torch.float64)
    out, inter = ref_ops.cpu_edge_forward(x, y, w, src, perm, ptr, fwd)
    gx, gy, gw = ref_ops.cpu_edge_backward(ct, x, y, w, inter, src, dst, fwd, b1, b2)
    T = ref_ops.dense_coupling(SH2, SH2, SH2)

    def fn(T, x, y, w):
        return ref_ops.scatter_sum(ref_ops.dense_u1u(T, x.index_select(0, src), y, w), dst, n_nodes)
    ref_out, ref_grads = ref_ops.dense_grads(fn, T, (x, y, w), ct)
    for name, a, b in (("out", out, ref_out), ("gx", gx, ref_grads[0]), ("gy", gy, ref_grads[1]),
                       ("gw", gw, ref_grads[2])):
        assert_close(a, b, 1e-12, name)


def test_segment_csr_against_index_add():
    g = torch.Generator().manual_seed(8)
    src = torch.randn(3, 20, 5, generator=g)
    ptr = torch.tensor([0, 0, 4, 4, 9, 20])
    out = ref_ops.segment_csr(src, ptr, 1)
    for i in range(5):
        torch.testing.assert_close(out[:, i], src[:, ptr[i]:ptr[i + 1]].sum(1))
