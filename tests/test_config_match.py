"""Which compiled table a module's ``TensorProductInfo`` runs on must not depend on options that only rescale the
coefficients: the match is by entries (output row, input rows) with one factor per weight path, and an explicit
``path=`` subset maps onto the paths it keeps.  Host-only (the library describes its compiled tables)."""
import os

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "equitorch_amd", "lib", "libcgtp.so")
pytestmark = pytest.mark.skipif(not os.path.exists(LIB), reason="libcgtp.so not built (run __graft_entry__.build())")

SH2, SH3 = "0e+1o+2e", "0e+1o+2e+3o"


def _infos(irr, **kw):
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    i = Irreps(irr)
    return tp_infos(i, i, i, **kw)[0]


def test_default_tables_match_exactly():
    from equitorch_amd.ops import kernels
    for irr, paths in ((SH2, 11), (SH3, 23), ("0e+1o+2e+3o+4e+5o+6e", 106), ("0e+1e+2e+3e+4e", None)):
        cfg = kernels.uvu_config_of(_infos(irr))
        assert cfg >= 0 and cfg.path_scale is None and cfg.w_rows is None, irr
        if paths:
            assert kernels.uvu_dims(cfg)[3] == paths
    cfg = kernels.uv_config_of(_infos(SH3))
    assert cfg >= 0 and cfg.path_scale is None and cfg.w_rows is None


def test_path_norm_and_channel_scale_change_only_the_factors():
    from equitorch_amd.ops import kernels
    base = kernels.uvu_config_of(_infos(SH2))
    raw = kernels.uvu_config_of(_infos(SH2, path_norm=False))
    assert int(raw) == int(base) and raw.w_rows is None
    # default tables divide the paths into output degree k by sqrt(number of such paths): 3, 4, 4 at lmax = 2
    counts = np.array([3, 3, 3, 4, 4, 4, 4, 4, 4, 4, 4], dtype=np.float64)
    np.testing.assert_allclose(raw.path_scale, np.sqrt(counts), rtol=1e-6)
    scaled = kernels.uv_config_of(_infos(SH3, channel_norm=True, channel_scale=128 ** -0.5))
    assert int(scaled) == int(kernels.uv_config_of(_infos(SH3)))
    np.testing.assert_allclose(scaled.path_scale, np.full(23, 128 ** -0.5), rtol=1e-6)
    both = kernels.uv_config_of(_infos(SH3, path_norm=False, channel_norm=True, channel_scale=0.25))
    assert int(both) == int(scaled) and abs(both.path_scale[0] - 0.25 * 2.0) < 1e-6    # 4 paths into l = 0


def test_path_subset_maps_onto_the_compiled_paths():
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    from oracle import ref_tables
    irr = Irreps(SH2)
    full = ref_tables.fully_connected_paths(*(ref_tables.parse(SH2),) * 3)
    keep = [p for n, p in enumerate(full) if n not in (1, 4, 7)]
    info = tp_infos(irr, irr, irr, path=keep)[0]
    cfg = kernels.uvu_config_of(info)
    assert cfg >= 0 and int(cfg) == int(kernels.uvu_config_of(_infos(SH2)))
    rows = cfg.w_rows.tolist()
    assert [r for r in rows if r >= 0] == list(range(len(keep))) and [rows[i] for i in (1, 4, 7)] == [-1, -1, -1]
    assert all(cfg.path_scale[i] == 0.0 for i in (1, 4, 7)) and all(cfg.path_scale[i] > 0 for i in (0, 2, 3))
    w = torch.arange(len(keep) * 2, dtype=torch.float32).reshape(len(keep), 2)
    wf = kernels.expand_paths(w, cfg, -2)
    assert wf.shape == (11, 2) and torch.equal(wf[[0, 2, 3]], w[:3]) and float(wf[[1, 4, 7]].abs().sum()) == 0.0
    assert torch.equal(kernels.contract_paths(wf, cfg, -2), w)


def test_other_tables_do_not_match():
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    info = tp_infos(Irreps("1o+2e+1e"), Irreps(SH2), Irreps("0e+1o"))[0]
    assert kernels.uvu_config_of(info) == -1 and kernels.uv_config_of(info) == -1
    # same dims as sh2 but other parities: entries differ
    assert kernels.uv_config_of(_infos("0e+1e+2e")) == -1


def test_exactness_of_a_match_decides_what_float64_operands_run_on():
    """``Cfg.exact``: every coefficient equals the compiled one times its path's factor to the last bit.  The default
    tables are exact; a subset of the paths of a larger table with another normalisation matches only to an fp32
    rounding (ratios within 1e-6 of each other, not equal), which float64 operands are not given."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    assert kernels.uvu_config_of(_infos(SH2)).exact and kernels.uvu_config_of(_infos(SH3)).exact
    sub = kernels.uvu_config_of(tp_infos(Irreps(SH3), Irreps(SH2), Irreps(SH2))[0])
    assert sub >= 0 and sub.w_rows is not None and sub.path_scale is not None and not sub.exact
    x = torch.zeros(4, 9, 8, dtype=torch.float64)
    assert not kernels.uvu_launchable(sub, x, torch.zeros(4, 9, dtype=torch.float64), torch.zeros(4, 13, 8, dtype=torch.float64))


def test_host_logic_for_tables_the_reference_builder_leaves_incomplete():
    """``sparse_product_info`` (``equitorch/utils/_structs.py:105-123``) shifts its segments when the first output row
    has no entry: the general contraction's spec keeps what the segments reach, the streaming kernels' walk lists the
    weight paths it never visits, and a weight without elements is a weight per sample of an empty batch."""
    from equitorch_amd.nn import SO2Linear
    from equitorch_amd.nn.functional import _irreps_gemm as G, _psw
    from equitorch_amd.nn.functional._tri import spec_from_product_info
    from equitorch_amd.nn.linears import _view_weight
    mod = SO2Linear("1o+1e", "2e+0e", 4, 4, internal_weights=False, feature_mode="uu")
    info = mod.info_forward
    spec = spec_from_product_info(info, mod.irreps_in.dim, mod.num_weights)
    reached, entries = int(info.seg_out[-1]), info.scale.shape[0]
    assert reached < entries and spec.out_idx.shape[0] == reached == spec.idx[0].shape[0] == spec.coef.shape[0]
    mod = SO2Linear("0e", "1o+2e", 4, 4, internal_weights=False, feature_mode="uv")
    plan = G.plan_of_product_info(mod.info_forward, 1, mod.num_weights)
    assert len(plan.paths) == 1 and plan.n_paths == 2                      # the second weight is used by no row
    table = _psw.PswTable([p.o0 for p in plan.paths], [p.i0 for p in plan.paths], [0] * len(plan.paths),
                          [p.w for p in plan.paths], [p.scale for p in plan.paths], 1, 1, plan.out_size, plan.n_paths, "cpu")
    assert table.unwalked_paths == [1]
    empty = SO2Linear("0e", "2e+0e", 4, 4, internal_weights=False, feature_mode="uv")
    assert not G.plan_of_product_info(empty.info_forward, 1, empty.num_weights).paths
    assert _view_weight(torch.zeros(0, 3, 4, 5), (3, 4, 5), 60).shape == (0, 3, 4, 5)
    assert _view_weight(torch.zeros(60), (3, 4, 5), 60).shape == (3, 4, 5)
    assert _view_weight(torch.zeros(2, 60), (3, 4, 5), 60).shape == (2, 3, 4, 5)
