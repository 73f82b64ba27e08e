"""Host side of the per-sample-weight streaming kernels on the CPU: the walk ``PswTable`` builds from a product table
(blocks = output irreps, slots = walked paths, entry words) is replayed in numpy exactly as the kernels read it and
compared with the dense oracle — u1v, 1vu (operands exchanged), uvw and channel mixing."""
import numpy as np
import pytest
import torch

from oracle import ref_ops


def _replay(table, x, y, w):
    """``out[n, m0 + j, :] = sum over the block's slots and k of t[k][j] * W[n, p, k, :]`` with ``t`` formed from the
    entry words (j | a << 8 | b << 16 | end-of-run << 24)."""
    d1, d2, d_out, n_paths = table.dims
    n, _, cu = x.shape
    cv = y.shape[2]
    out = np.zeros((n, d_out, w.shape[-1]))
    words, coef = table.entries.numpy().astype(np.int64), table.coef(torch.float64).numpy()
    for m0, rows, q0, q1 in table.blocks.tolist():
        for p, e0, e1 in table.slots[q0:q1].tolist():
            t = np.zeros((n, cu * cv, rows))
            val = np.zeros((n, cu, cv))
            seen = []
            for e in range(e0, e1):
                j, a, b = words[e] & 255, (words[e] >> 8) & 255, (words[e] >> 16) & 255
                val += coef[e] * x[:, a, :, None] * y[:, b, None, :]
                if words[e] >> 24 & 1:
                    t[:, :, j] = val.reshape(n, -1)
                    val[:] = 0
                    seen.append(int(j))
            assert seen == list(range(rows)), "every row of the block must close exactly one run, in order"
            out[:, m0:m0 + rows] += np.einsum("nkj,nkw->njw", t, w[:, p])
    return out


def _sh(lmax):
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


@pytest.mark.parametrize("irreps", [(_sh(2),) * 3, ("1o+2e+1e", "0e+1o+2e", "0e+1o"), ("2x0e+1o+1e", "0e+2x1o", "0e+1o+1e"),
                                    ("0e+4e", "2e+3o", "2e+3o")])
@pytest.mark.parametrize("channelled", [1, 2])
def test_walk_reproduces_the_dense_product(irreps, channelled):
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn.functional import _psw
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    io, i1, i2 = irreps
    info = tp_infos(Irreps(io), Irreps(i1), Irreps(i2))[0]
    coo = kernels.coo_of(info)
    table = _psw.table_of_coo(coo, info.info_Mij_fwd.scale, channelled, "cpu")
    assert table is not None and table.covers_output
    T = ref_ops.dense_coupling(io, i1, i2).float().double()
    rng = np.random.default_rng(0)
    n, cu, cout = 5, 3, 4
    if channelled == 1:       # u1v and, with channels on y, uvw
        for cv in (1, 2):
            x, y = rng.standard_normal((n, T.shape[2], cu)), rng.standard_normal((n, T.shape[3], cv))
            w = rng.standard_normal((n, T.shape[0], cu * cv, cout))
            ref = ref_ops.dense_uvw(T, torch.from_numpy(x), torch.from_numpy(y),
                                    torch.from_numpy(w).reshape(n, -1, cu, cv, cout)).numpy()
            np.testing.assert_allclose(_replay(table, x, y, w), ref, atol=1e-12)
    else:                     # 1vu: the channelled operand is the product's second
        x, y = rng.standard_normal((n, T.shape[2])), rng.standard_normal((n, T.shape[3], cu))
        w = rng.standard_normal((n, T.shape[0], cu, cout))
        ref = ref_ops.dense_u1v(T.transpose(2, 3), torch.from_numpy(y), torch.from_numpy(x), torch.from_numpy(w)).numpy()
        np.testing.assert_allclose(_replay(table, y, x[:, :, None], w), ref, atol=1e-12)


def test_rows_without_a_term_and_tables_the_kernels_do_not_walk():
    """A (path, row) pair without a coefficient gets a zero entry, so the coupled operand's row is defined; row ranges
    of different paths that overlap are merged into one block; a block beyond two passes of rows is refused."""
    from equitorch_amd.nn.functional._psw import PswTable
    # path 0 writes rows 0..2 but has no term for row 1
    t = PswTable([0, 2], [0, 1], [0, 0], [0, 0], [1.0, 2.0], 2, 1, 3, 1, "cpu")
    assert t.entries.tolist() == [0 | 1 << 24, 1 | 1 << 24 | 1 << 25, 2 | 1 << 8 | 1 << 24]
    assert t.coef(torch.float64).tolist() == [1.0, 0.0, 2.0]
    assert t.blocks.tolist() == [[0, 3, 0, 1]] and t.slots.tolist() == [[0, 0, 3]]
    # rows 0..1 and 1..2 overlap without coinciding: one block of three rows, zero entries where a path has no term
    t = PswTable([0, 1, 1, 2], [0, 0, 0, 0], [0, 0, 0, 0], [0, 0, 1, 1], [1.0] * 4, 1, 1, 3, 2, "cpu")
    assert t.blocks.tolist() == [[0, 3, 0, 2]] and t.slots.tolist() == [[0, 0, 3], [1, 3, 6]]
    assert t.coef(torch.float64).tolist() == [1.0, 1.0, 0.0, 0.0, 1.0, 1.0]
    with pytest.raises(ValueError):     # a block of more rows than two passes take
        PswTable([0, 40], [0, 0], [0, 0], [0, 0], [1.0, 1.0], 1, 1, 41, 1, "cpu")
    t = PswTable([2, 0], [0, 0], [0, 0], [0, 0], [1.0, 1.0], 1, 1, 4, 1, "cpu")     # row 3 is never written
    assert not t.covers_output and t.blocks.tolist() == [[0, 3, 0, 1]]
