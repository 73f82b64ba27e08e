"""Small host-side helpers of the public API: the index helpers of ``irreps`` against the reference's docstring
examples (``equitorch/irreps/__init__.py:841-974``), the random-rotation utilities against what defines them,
and the block / SO(2) table builders against entries written out by hand."""
import math

import torch

from equitorch_amd import irreps as I
from equitorch_amd import utils as U


def test_irreps_index_helpers_match_the_reference_docstrings():
    uniq, where = I.unique_irreps(I.Irreps("0+0e+1o+0e+0e"))
    assert repr(uniq) == "Irreps(0+0e+1o)"
    assert {repr(k): v for k, v in where.items()} == {"0": [0], "0e": [1, 3, 4], "1o": [2]}
    uniq, where = I.unique_irreps(I.Irreps("2x1e+0o+1e"))
    assert repr(uniq) == "Irreps(1e+0o)"
    assert {repr(k): v for k, v in where.items()} == {"1e": [0, 1, 3], "0o": [2]}
    assert I.irrep_indices(I.Irreps("1o")).tolist() == [0, 0, 0]
    assert I.irrep_indices(I.Irreps((0, 3))).tolist() == [0, 1, 1, 1, 2, 2, 2, 2, 2, 3, 3, 3, 3, 3, 3, 3]
    assert I.irrep_indices("0+2x1e+2e").tolist() == [0, 1, 1, 1, 2, 2, 2, 3, 3, 3, 3, 3]
    assert I.irrep_degrees("0+2x1e+2e").tolist() == [0, 1, 1, 2]
    assert I.element_degrees("0e+1o+2e").tolist() == [0, 1, 1, 1, 2, 2, 2, 2, 2]
    assert I.element_orders("0e+1o+2e").tolist() == [0, -1, 0, 1, -2, -1, 0, 1, 2]
    for t in (I.irrep_indices("1o"), I.irrep_degrees("1o"), I.element_degrees("1o"), I.element_orders("1o")):
        assert t.dtype == torch.long
    assert I.p_mapping["e"] == 1 and I.p_mapping["o"] == -1 and I.p_mapping[None] == 0


def test_random_rotation_utilities():
    g = torch.Generator().manual_seed(0)
    R = U.rand_rotation_matrices((4, 5), dtype=torch.float64, generator=g)
    assert R.shape == (4, 5, 3, 3)
    eye = torch.eye(3, dtype=torch.float64).expand(4, 5, 3, 3)
    torch.testing.assert_close(R @ R.transpose(-1, -2), eye)
    torch.testing.assert_close(torch.linalg.det(R), torch.ones(4, 5, dtype=torch.float64))
    theta, phi = U.rand_spherical_angles((1000,), dtype=torch.float64, generator=g)
    assert theta.min() >= 0 and theta.max() <= math.pi and phi.min() >= 0 and phi.max() < 2 * math.pi
    assert abs(torch.cos(theta).mean()) < 0.1            # cos(theta) is uniform on [-1, 1]
    a, b, c = U.rand_rotation_angles((1000,), dtype=torch.float64, generator=g)
    assert b.min() >= 0 and b.max() <= math.pi and a.max() < 2 * math.pi and c.max() < 2 * math.pi
    assert abs(torch.cos(b).mean()) < 0.1


def test_irreps_blocks_and_so2_linear_tables():
    fwd, bwd1, bwd2 = U.irreps_blocks_infos("0e+1o")
    # 1 + 9 matrix elements, block after block and row-major: element q acts on input M_in(q) into output M_out(q)
    assert fwd.index1 is None and fwd.index2.tolist() == [0, 1, 2, 3, 1, 2, 3, 1, 2, 3]
    assert fwd.seg_out.tolist() == [0, 1, 4, 7, 10] and fwd.out_size == 4
    x = torch.randn(4, dtype=torch.float64)
    blocks = [torch.randn(1, 1, dtype=torch.float64), torch.randn(3, 3, dtype=torch.float64)]
    flat = torch.cat([b.reshape(-1) for b in blocks])
    prod = flat * x[fwd.index2]
    out = torch.stack([prod[a:b].sum() for a, b in zip(fwd.seg_out[:-1], fwd.seg_out[1:])])
    torch.testing.assert_close(out, torch.block_diag(*blocks) @ x)
    assert bwd1.out_size is None or bwd1.out_size >= 0     # gradient tables exist for both operands
    assert bwd2 is not None
    one, n = U.so2_linear_info(I.Irreps("0e+1o"), I.Irreps("0e+1o"))
    three = U.so2_linear_infos(I.Irreps("0e+1o"), I.Irreps("0e+1o"))
    assert n == three[3]
    for f in ("scale", "index1", "index2", "seg_out", "gather_index", "index_out"):
        a, b = getattr(one, f), getattr(three[0], f)
        assert (a is None and b is None) or torch.equal(a, b)


def test_transforms_without_pyg():
    """The data transforms on a plain attribute container: the radius graph against a double loop (centres in index
    order, first ``max_num_neighbors`` neighbours, examples of a batch kept apart), norms and length embeddings."""
    from types import SimpleNamespace

    from equitorch_amd import transforms as T
    g = torch.Generator().manual_seed(3)
    pos = torch.rand(40, 3, generator=g, dtype=torch.float64)
    batch = (torch.arange(40) >= 25).long()
    data = SimpleNamespace(pos=pos, batch=batch)
    out = T.RadiusGraph(0.45, max_num_neighbors=4)(data)
    assert not hasattr(data, "edge_index")                       # applied to a shallow copy
    want = []
    for i in range(40):
        nb = [j for j in range(40) if j != i and batch[i] == batch[j] and (pos[i] - pos[j]).norm() < 0.45][:4]
        want += [(j, i) for j in nb]
    assert out.edge_index.dtype == torch.long
    assert sorted(map(tuple, out.edge_index.t().tolist())) == sorted(want)
    torch.testing.assert_close(out.edge_vec, pos[out.edge_index[1]] - pos[out.edge_index[0]])
    flipped = T.RadiusGraph(0.45, max_num_neighbors=4, flow="target_to_source")(data)
    assert torch.equal(flipped.edge_index, out.edge_index.flip(0))
    loops = T.RadiusGraph(0.2, loop=True, max_num_neighbors=64)(SimpleNamespace(pos=pos, batch=None))
    assert ((loops.edge_index[0] == loops.edge_index[1]).sum()) == 40
    out = T.AddVectorNorm()(out)
    torch.testing.assert_close(out.edge_norm, out.edge_vec.norm(dim=-1))
    out = T.AddVectorLengthEmbedding(lambda d: torch.stack([d, d * d], dim=-1))(out)
    torch.testing.assert_close(out.edge_emb[:, 1], out.edge_norm ** 2)
    assert repr(T.RadiusGraph(0.5)) == "RadiusGraph(r=0.5)"
