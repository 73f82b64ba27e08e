"""Tables of the irreps-preserving channel mixing (``irreps_linear_infos``, ``irreps_info``): the product's
builders against the oracle's list-based restatement, bit for bit, and both against what the construction fixes in
closed form (equitorch/utils/_structs.py:336-459)."""
import pytest
import torch

from equitorch_amd.irreps import Irreps
from equitorch_amd.utils import irreps_info, irreps_linear_infos
from oracle import ref_ops, ref_tables

CASES = [
    ("0e+1o+2e", "0e+1o+2e", {}),
    ("0e+1o+2e", "0e+1o+1o+2e+0e", {}),
    ("2x0e+1o+3x2e", "0e+2x1o+2e+3e", {}),
    ("0e+1o", "0e+1e+2e", {"path_norm": False}),
    ("0e+1o+2e", "0e+1o+2e", {"channel_norm": True, "channel_scale": 64}),
    ("0e+1o+2e", "0e+1o+1o+2e", {"path_norm": False, "channel_norm": True, "channel_scale": 16}),
    ("0e+1o+2e", "0e+1o+1o+2e", {"path": [(0, 0), (1, 2), (2, 3)]}),
    ((0, 3), (0, 4), {}),
]


def _same(tensor, lst, what):
    ref = torch.tensor(lst)
    assert tensor.dtype == ref.dtype, f"{what}: dtype {tensor.dtype} vs {ref.dtype}"
    assert torch.equal(tensor, ref), what


@pytest.mark.parametrize("io,ii,kw", CASES)
def test_builder_matches_oracle_bit_for_bit(io, ii, kw):
    mine = irreps_linear_infos(io, ii, **kw)
    ref = ref_tables.irreps_linear_infos(io, ii, **kw)
    assert mine[2] == ref[2]
    for info, r in zip(mine[:2], ref[:2]):
        for field in info._fields:
            if field == "out_size":
                assert info.out_size == r["out_size"]
            else:
                _same(getattr(info, field), r[field], field)


def test_closed_form_structure():
    """One entry per component of every path, sorted by output component; scale = count(paths into the output
    irrep)^-1/2 as fp32; the backward table is the forward one with input and output components exchanged."""
    io, ii = Irreps("0e+1o+2e"), Irreps("0e+1o+1o+2e+2e+2e")
    f, b, n = irreps_linear_infos(io, ii)
    assert n == 6 and f.M_MM0.shape[0] == 1 + 2 * 3 + 3 * 5
    assert torch.equal(f.M_MM0, torch.sort(f.M_MM0).values)
    count = {0: 1, 1: 2, 2: 3}
    deg = [0, 1, 1, 1, 2, 2, 2, 2, 2]
    expect = torch.tensor([count[deg[M]] ** -0.5 for M in f.M_MM0.tolist()])
    assert torch.equal(f.scale_MM0, expect) and f.scale_MM0.dtype == torch.float32
    assert torch.equal(f.M_out, torch.arange(9)) and f.out_size == 9 and b.out_size == ii.dim
    pairs_f = sorted(zip(f.M_MM0.tolist(), f.M0_MM0.tolist(), f.ii0_MM0.tolist()))
    pairs_b = sorted(zip(b.M0_MM0.tolist(), b.M_MM0.tolist(), b.ii0_MM0.tolist()))
    assert pairs_f == pairs_b
    # without path_norm the reference's scale list holds the Python int 1: integer-typed scale tensors
    f2, _, _ = irreps_linear_infos("0e+1o", "0e+1o", path_norm=False)
    assert f2.scale_MM0.dtype == torch.int64 and f2.scales_ii0.tolist() == [1, 1]


def test_irreps_info_matches_oracle_and_closed_form():
    for irr in ("0e+1o+2e", "2x0e+3x1o", (0, 4)):
        mine, ref = irreps_info(irr), ref_tables.irreps_info(irr)
        for field in ("rsqrt_dims", "rdims", "irrep_index", "irrep_seg"):
            _same(getattr(mine, field), ref[field], field)
        assert mine.num_irreps == ref["num_irreps"]
    info = irreps_info("0e+1o+2e")
    assert info.irrep_seg.tolist() == [0, 1, 4, 9] and info.irrep_index.tolist() == [0, 1, 1, 1, 2, 2, 2, 2, 2]
    assert torch.equal(info.rdims, torch.tensor([1.0, 1 / 3, 1 / 5]))


def test_oracle_forward_reduces_to_plain_matmul():
    """With one path into every output irrep the layer is ``x[:, rows of l] @ W[l]``; with two input copies of an
    irrep it is the normalised sum of both — checked against torch.matmul written out by hand."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 9, 4, generator=g, dtype=torch.float64)
    w = torch.randn(3, 4, 6, generator=g, dtype=torch.float64)
    f, _, _ = ref_tables.irreps_linear_infos("0e+1o+2e", "0e+1o+2e")
    expect = torch.cat([x[:, 0:1] @ w[0], x[:, 1:4] @ w[1], x[:, 4:9] @ w[2]], dim=1)
    torch.testing.assert_close(ref_ops.cpu_irreps_linear(x, w, f), expect)
    torch.testing.assert_close(ref_ops.cpu_irrep_wise_linear(x, w, ref_tables.irreps_info("0e+1o+2e")), expect)
    x2 = torch.randn(5, 7, 4, generator=g, dtype=torch.float64)            # 0e + 1o + 1o
    w2 = torch.randn(3, 4, 6, generator=g, dtype=torch.float64)
    f2, _, _ = ref_tables.irreps_linear_infos("0e+1o", "0e+1o+1o")
    expect2 = torch.cat([x2[:, 0:1] @ w2[0], (x2[:, 1:4] @ w2[1] + x2[:, 4:7] @ w2[2]) / 2 ** 0.5], dim=1)
    torch.testing.assert_close(ref_ops.cpu_irreps_linear(x2, w2, f2), expect2)
    # per-sample weights
    wn = torch.randn(5, 3, 4, 6, generator=g, dtype=torch.float64)
    expect3 = torch.cat([torch.einsum("nmu,nuw->nmw", x[:, a:b], wn[:, p]) for p, (a, b) in
                         enumerate([(0, 1), (1, 4), (4, 9)])], dim=1)
    torch.testing.assert_close(ref_ops.cpu_irreps_linear(x, wn, f), expect3)
