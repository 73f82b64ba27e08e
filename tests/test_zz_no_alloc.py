"""The row-summing contraction through the entry point that allocates nothing (``cgtp_tri_contract_static``: partial
rows in the library's fixed per-device array) against ``cgtp_tri_contract`` with a caller-provided workspace: the
same kernels, so the results must be bit-identical; two calls in a row, the second on a smaller input, which reuses
the array with the first call's contents still in it."""
import ctypes as C

import pytest
import torch

from oracle import ref_ops, ref_tables

pytestmark = pytest.mark.gpu


def _launch(static, x, y, table, n_out, out):
    from equitorch_amd._lib import OPERAND_NONE, OPERAND_VEC
    from equitorch_amd.ops import kernels
    n, _, ch = x.shape
    return kernels.tri_contract(table, n_out, (x, OPERAND_VEC), (y, OPERAND_VEC), (None, OPERAND_NONE), n, ch, x.dtype,
                                x.device, reduce_rows=True, out=out, static_scratch=static)


CASES = [  # table, dtype, channels, rows of the first and of the second call
    ("info_Mij_fwd", torch.float32, 64, 400, 100),      # operands staged in LDS, per-row results + two passes
    ("info_M_fwd", torch.float32, 64, 3000, 1100),      # light table, 16-byte lanes
    ("info_M_fwd", torch.float32, 97, 3000, 1100),      # row-by-row kernel: 1024 wavefronts with uneven shares
    ("info_Mij_fwd", torch.float64, 20, 300, 64),
]


@pytest.mark.parametrize("name,dtype,channels,n1,n2", CASES)
def test_static_scratch_entry_matches_workspace_entry(device, name, dtype, channels, n1, n2):
    from equitorch_amd import _lib
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    irr = Irreps((1, 3))
    info = getattr(tp_infos(irr, irr, irr)[0], name).to(device)
    ref = dict(ref_ops.tables_to_torch(ref_tables.tp_infos((1, 3), (1, 3), (1, 3))[0], torch.float64)[name])
    if ref["scale"] is not None:
        ref["scale"] = ref["scale"].float().double()
    nnz = int(ref["scale"].shape[0] if ref["scale"] is not None else ref["seg_out"][-1])
    size = lambda idx: nnz if idx is None else int(idx.max()) + 1
    d1, d2 = size(ref["index1"]), size(ref["index2"])
    table, n_out = kernels.product_tri_table(info.scale, info.index1, info.index2, info.seg_out, nnz, dtype, device)
    g = torch.Generator().manual_seed(channels)
    for n in (n1, n2):                                        # the second call is smaller and follows at once
        x = torch.randn(n, d1, channels, generator=g, dtype=torch.float64).to(dtype)
        y = torch.randn(n, d2, channels, generator=g, dtype=torch.float64).to(dtype)
        xd, yd = x.to(device), y.to(device)
        out_ws = torch.empty(n_out, channels, dtype=dtype, device=device)
        out_st = torch.full_like(out_ws, float("nan"))
        _launch(False, xd, yd, table, n_out, out_ws)
        before = torch.cuda.memory_allocated(device)
        _launch(True, xd, yd, table, n_out, out_st)
        assert torch.cuda.memory_allocated(device) == before
        assert torch.equal(out_st, out_ws), f"n={n}: static-scratch result differs from the workspace result"
        want = ref_ops.cpu_mul(x.double(), y.double(), ref, out_accumulated=True)
        err = float((out_st.double().cpu() - want).abs().max())
        assert err <= (1e-5 if dtype == torch.float32 else 1e-11) * max(1.0, float(want.abs().max())), err
    # beyond the fixed array: refused with its own status, nothing launched
    assert _lib.lib.cgtp_tri_static_scratch_bytes() == 16 << 20
    big = kernels.TriArgs()
    big.dtype, big.C, big.n_out, big.nnz, big.n_rows, big.reduce_rows = 0, 64, n_out, nnz, 1 << 20, 1
    big.idx, big.seg, big.out = table["idx"].data_ptr(), table["seg"].data_ptr(), out_st.data_ptr()
    assert _lib.lib.cgtp_tri_contract_static(C.byref(big), None) == 9
