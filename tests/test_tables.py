"""Constant tables: the oracle's restatement and the product's builders against the golden fixtures written by
the reference's own ``tp_infos`` / ``sparse_scale_infos`` (tests/golden/make_tables.py), bit for bit, plus
closed-form counts and hand-checked small cases."""
import json
import os

import numpy as np
import pytest
import torch

from equitorch_amd.irreps import Irreps, irrep_segments
from equitorch_amd.utils import (extract_batch_segments, extract_scatter_indices, generate_fully_connected_tp_paths,
                                 sort_by_column_key, sparse_product_info, sparse_scale_infos, tp_infos)
from oracle import ref_tables

GOLD = os.path.join(os.path.dirname(__file__), "golden")
FX = np.load(os.path.join(GOLD, "tp_tables.npz"))
FS = np.load(os.path.join(GOLD, "scale_tables.npz"))
META = json.load(open(os.path.join(GOLD, "tp_tables_meta.json")))


def _case_args(name):
    m = META[name]
    irr = [m["irreps_out"], m["irreps1"], m["irreps2"]]
    if name == "so3_13":
        irr = [(1, 3)] * 3
    kw = dict(m["kwargs"])
    if "path" in kw:
        kw["path"] = [tuple(p) for p in kw["path"]]
    return irr, kw, m["num_paths"]


def _check_field(fx, prefix, field, value):
    """value: tensor | list | int | None, compared with the fixture bit for bit (scale as fp32 bits)."""
    none = set(fx[prefix + "/__none__"].tolist())
    key = f"{prefix}/{field}"
    if value is None:
        assert field in none, f"{key}: reference has a tensor here"
        return
    assert field not in none, f"{key}: reference has None here"
    gold = fx[key]
    if isinstance(value, int):
        assert int(gold) == value, key
        return
    if isinstance(value, torch.Tensor):
        assert str(value.dtype) == str(fx[key + "/dtype"]), f"{key}: dtype {value.dtype}"
        value = value.numpy()
    elif field == "scale":
        value = np.asarray(value, dtype=np.float64).astype(np.float32)  # what torch.tensor(list) stores
    else:
        value = np.asarray(value, dtype=np.int64)
    assert value.shape == gold.shape, f"{key}: shape {value.shape} vs {gold.shape}"
    assert value.tobytes() == gold.tobytes(), f"{key}: bits differ"


INFO_FIELDS = {
    "product": ("scale", "index1", "index2", "seg_out", "gather_index", "index_out", "out_size"),
    "scale": ("scale", "index", "seg_out", "index_out", "out_size"),
}


@pytest.mark.parametrize("name", sorted(META))
def test_oracle_tables_match_reference(name):
    irr, kw, n_paths = _case_args(name)
    fwd, b1, b2, n = ref_tables.tp_infos(*irr, **kw)
    assert n == n_paths
    for dname, tp in (("fwd", fwd), ("bwd1", b1), ("bwd2", b2)):
        assert int(FX[f"{name}/{dname}/out_size"]) == tp["out_size"]
        for fld in ref_tables.TP_FIELDS:
            kind = "scale" if fld.startswith("info_M_kM1M2") else "product"
            for f in INFO_FIELDS[kind]:
                _check_field(FX, f"{name}/{dname}/{fld}", f, tp[fld][f])


@pytest.mark.parametrize("name", sorted(META))
def test_product_tables_match_reference(name):
    irr, kw, n_paths = _case_args(name)
    fwd, b1, b2, n = tp_infos(*[Irreps(i) for i in irr], **kw)
    assert n == n_paths
    for dname, tp in (("fwd", fwd), ("bwd1", b1), ("bwd2", b2)):
        assert int(FX[f"{name}/{dname}/out_size"]) == tp.out_size
        for fld in tp._fields[:-1]:
            info = getattr(tp, fld)
            for f in info._fields:
                _check_field(FX, f"{name}/{dname}/{fld}", f, getattr(info, f))


@pytest.mark.parametrize("name", ["g8_40", "g5_12_scaled", "g64_700", "g6_4_sparse"])
def test_scale_tables_match_reference(name):
    dst = FS[name + "/dst"].tolist()
    n = int(FS[name + "/n_nodes"])
    scale = FS[name + "/scale_in"].tolist() if name + "/scale_in" in FS else None
    args = dict(index=list(range(len(dst))), index_out=dst, scale=scale, out_size=n, in_size=len(dst))
    for builder, get in ((ref_tables.sparse_scale_infos, lambda i, f: i[f]),
                         (sparse_scale_infos, lambda i, f: getattr(i, f))):
        fwd, bwd = builder(**args)
        for dname, info in (("fwd", fwd), ("bwd", bwd)):
            for f in INFO_FIELDS["scale"]:
                _check_field(FS, f"{name}/{dname}", f, get(info, f))


def test_edge_plan_tables_are_the_scale_info_tables():
    """A stable sort by dst + histogram scan gives the index / seg_out of sparse_scale_info(index_out=dst)."""
    name = "g64_700"
    dst = torch.from_numpy(FS[name + "/dst"])
    n = int(FS[name + "/n_nodes"])
    perm = torch.sort(dst, stable=True).indices
    ptr = torch.zeros(n + 1, dtype=torch.int64)
    ptr[1:] = torch.cumsum(torch.bincount(dst, minlength=n), 0)
    assert perm.numpy().tobytes() == FS[name + "/fwd/index"].tobytes()
    assert ptr.numpy().tobytes() == FS[name + "/fwd/seg_out"].tobytes()
    # transposed table: one entry per edge, index = dst, no segmentation
    assert dst.numpy().tobytes() == FS[name + "/bwd/index"].tobytes()
    assert "seg_out" in set(FS[name + "/bwd/__none__"].tolist())


@pytest.mark.parametrize("lmax,paths,nnz,s1", [(2, 11, 83, 35), (3, 23, 353, 99), (6, 106, 6460, 826)])
def test_closed_form_counts(lmax, paths, nnz, s1):
    """Triangle + parity rule and the exact sparsity pattern of the real-basis coefficients."""
    irr = Irreps.spherical_harmonics(lmax)
    plist = generate_fully_connected_tp_paths(irr, irr, irr)
    expect = [(k, i, j) for k in range(lmax + 1) for i in range(lmax + 1) for j in range(lmax + 1)
              if abs(i - j) <= k <= i + j and (i + j + k) % 2 == 0]
    assert plist == expect and len(plist) == paths
    fwd = tp_infos(irr, irr, irr)[0]
    assert fwd.info_Mij_fwd.scale.numel() == nnz
    assert fwd.info_Mij_fwd.out_size == s1 == sum(2 * k + 1 for k, _, _ in plist)


def test_lmax2_path_list_and_nnz():
    irr = Irreps("0e+1o+2e")
    assert generate_fully_connected_tp_paths(irr, irr, irr) == [
        (0, 0, 0), (0, 1, 1), (0, 2, 2), (1, 0, 1), (1, 1, 0), (1, 1, 2), (1, 2, 1), (2, 0, 2), (2, 1, 1), (2, 2, 0),
        (2, 2, 2)]
    from equitorch_amd._tables import tp_coo
    coo = tp_coo(tp_infos(irr, irr, irr)[0])
    assert np.bincount(coo.p).tolist() == [1, 3, 5, 3, 3, 11, 11, 5, 11, 5, 25]


def test_tiny_table_by_hand():
    """0e+1o x 0e+1o -> 0e+1o: paths (0,0,0),(0,1,1),(1,0,1),(1,1,0); 1+3+3+3 = 10 coefficients."""
    irr = Irreps("0e+1o")
    fwd, _, _, n = tp_infos(irr, irr, irr)
    assert n == 4
    s = fwd.info_Mij_fwd
    r2, r6 = np.float32(2 ** -0.5), np.float32(2 ** -0.5 * 3 ** -0.5)
    # sorted by (k, M, i, j, M1, M2): M=0: path(0,0,0) then path (0,1,1) x3; then M=1..3: paths (1,0,1),(1,1,0)
    assert s.index1.tolist() == [0, 1, 2, 3, 0, 1, 0, 2, 0, 3]
    assert s.index2.tolist() == [0, 1, 2, 3, 1, 0, 2, 0, 3, 0]
    np.testing.assert_array_equal(s.scale.numpy(), np.array([r2, r6, r6, r6] + [r2] * 6, dtype=np.float32))
    assert s.seg_out.tolist() == [0, 1, 4, 5, 6, 7, 8, 9, 10]
    assert fwd.info_M_fwd.index2.tolist() == [0, 1, 2, 3, 2, 3, 2, 3]
    assert fwd.info_M_fwd.seg_out.tolist() == [0, 2, 4, 6, 8]


def test_index_helpers_examples():
    """The worked examples in the reference docstrings (equitorch/utils/_indices.py:36-57,115-123,160-181)."""
    assert extract_batch_segments([[1, 1, 2, 2], [1, 1, 2, 2]]) == ([0, 0, 1, 1], [0, 2, 4], [[1, 2], [1, 2]])
    assert extract_batch_segments([[5, 5, 5], [5, 5, 5]]) == ([0, 0, 0], [0, 3], [[5], [5]])
    assert extract_batch_segments([[1, 1, 2, 3, 3], [1, 2, 2, 3, 3]]) == (
        [0, 1, 2, 3, 3], [0, 1, 2, 3, 5], [[1, 1, 2, 3], [1, 2, 2, 3]])
    assert sort_by_column_key([[1, 2, 3], [4, 5, 6]], [[2, 1, 3], [1, 3, 2]]) == [[2, 1, 3], [5, 4, 6]]
    assert extract_scatter_indices([[1, 1, 2, 3, 3], [1, 2, 2, 3, 3]]) == (
        [0, 1, 2, 3, 3], [[1, 1, 2, 3], [1, 2, 2, 3]])
    for mine, ref in ((extract_batch_segments, ref_tables.batch_segments),
                      (extract_scatter_indices, ref_tables.scatter_indices)):
        keys = [[0, 0, 1, 1, 1, 4], [2, 3, 3, 3, 5, 5]]
        assert tuple(mine(keys)) == tuple(ref(keys))


def test_irreps_doc_examples():
    """Stored expected values from the reference's docstrings (equitorch/irreps/__init__.py:172-173,274-277,
    522-531,906-911)."""
    assert irrep_segments(Irreps("1o")) == [0, 3]
    assert irrep_segments(Irreps((0, 4))) == [0, 1, 4, 9, 16, 25]
    assert irrep_segments("0+2x1e+3x2e+4") == [0, 1, 4, 7, 12, 17, 22, 31]
    assert repr(Irreps.spherical_harmonics(2, "e")) == "Irreps(0e+1o+2e)"
    assert repr(Irreps.spherical_harmonics(3, "o")) == "Irreps(0o+1e+2o+3e)"
    assert repr(Irreps("1x0e + 1x1o") * Irreps("1x0o + 1x1e")) == "Irreps(2x0o+2x1e+1o+2o)"
    assert repr(Irreps((0, 2)) * Irreps((0, 2))) == "Irreps(3x0+6x1+6x2+3x3+4)"
    assert [repr(i) for i in Irreps("2x0+2x0+2x0e+3x1o+2")] == ["0", "0", "0", "0", "0e", "0e", "1o", "1o", "1o", "2"]
    assert Irreps("2x0e + 3x1o").dim == 11 and len(Irreps("2x0e + 3x1o")) == 5
    assert repr(Irreps("0o+3x0o+0e+3x1+3x2e+4x1").simplified()) == "Irreps(0e+4x0o+7x1+3x2e)"
    assert repr(Irreps("128x0e + 64x1o + 32x2e").squeeze_max_channels()[0]) == "Irreps(4x0e+2x1o+2e)"


def test_leading_empty_row_quirk_is_reproduced():
    """sparse_product_info pads its boundary list for empty leading rows before indexing it
    (equitorch/utils/_structs.py:103-121); product and oracle must reproduce the resulting pointer."""
    args = dict(index1=[0, 1, 2, 3], index2=[1, 0, 1, 0], index=[2, 2, 3, 5], out_size=7)
    mine = sparse_product_info(**args)
    ref = ref_tables.sparse_product_info(**args)
    assert mine.seg_out.tolist() == ref["seg_out"]
    assert mine.index1 is None and ref["index1"] is None
    assert mine.index2.tolist() == ref["index2"]
