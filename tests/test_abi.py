"""The C-ABI library: loads, exports every symbol declared in include/cgtp.h, and its host-only validation
entry points report the documented status codes (no kernel is launched here)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "equitorch_amd", "lib", "libcgtp.so")
pytestmark = pytest.mark.skipif(not os.path.exists(LIB), reason="libcgtp.so not built (run __graft_entry__.build())")


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "cgtp.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cgtp_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    lib = C.CDLL(LIB)
    names = declared_symbols()
    assert len(names) >= 15
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/cgtp.h but not exported"


def test_struct_layouts_match_the_ctypes_mirror():
    """The argument structs are mirrored by hand in ``equitorch_amd/_lib.py``; the library reports sizeof and every
    field offset as compiled, in declaration order."""
    from equitorch_amd import _lib
    for which, cls in enumerate((_lib.Operand, _lib.TriArgs, _lib.GenOperand, _lib.GenArgs, _lib.UvuArgs, _lib.UvtItem,
                                _lib.UvtArgs, _lib.UvtGwArgs, _lib.UvtGyArgs, _lib.UvuTab, _lib.PswTable,
                                _lib.PswArgs)):
        n = _lib.lib.cgtp_abi_layout(which, None, 0)
        assert n == 1 + len(cls._fields_), f"{cls.__name__}: {n - 1} fields in the library, {len(cls._fields_)} here"
        buf = (C.c_int64 * n)()
        assert _lib.lib.cgtp_abi_layout(which, buf, n) == n
        assert buf[0] == C.sizeof(cls), f"sizeof {cls.__name__}"
        for k, (name, _) in enumerate(cls._fields_):
            assert buf[1 + k] == getattr(cls, name).offset, f"{cls.__name__}.{name}"
    assert _lib.lib.cgtp_abi_layout(99, None, 0) == -1


def test_version_and_status_strings():
    from equitorch_amd import _lib
    assert _lib.lib.cgtp_version() >= 1
    assert _lib.lib.cgtp_status_string(0) == b"ok"
    assert len({_lib.lib.cgtp_status_string(i) for i in range(10)}) == 10


def test_compiled_tables_match_python_fingerprints():
    from equitorch_amd import _lib
    from equitorch_amd._tables import fingerprint, tp_coo
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    n = _lib.lib.cgtp_uvu_num_configs()
    assert n >= 3
    irr = Irreps("0e+1o+2e")
    coo = tp_coo(tp_infos(irr, irr, irr)[0])
    cfg = _lib.lib.cgtp_uvu_find(C.c_uint64(fingerprint(coo)))
    assert cfg >= 0
    dims = (C.c_int32 * 5)()
    assert _lib.lib.cgtp_uvu_describe(cfg, dims) == fingerprint(coo)
    assert tuple(dims) == (9, 9, 9, 11, 83)
    assert _lib.lib.cgtp_uvu_find(C.c_uint64(12345)) == -1


def test_host_side_validation_codes():
    from equitorch_amd import _lib
    L = _lib.lib
    a = _lib.UvuArgs()
    assert L.cgtp_uvu_validate(None, 0) == 1                        # CGTP_ERR_NULL
    a.cfg = 999
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 5                  # CGTP_ERR_CONFIG
    a.cfg, a.dtype = 1, 7
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 4                  # CGTP_ERR_DTYPE
    a.dtype, a.C = 0, 0
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2                  # CGTP_ERR_SHAPE
    a.C, a.n_rows, a.n_x_rows = 64, 10, 10
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 1                  # x / y / w missing
    a.x = a.y = a.w = a.out = 256
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0
    a.n_x_rows = 9
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2                  # rows of x without a gather table
    a.n_x_rows, a.C = 10, 512
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0                  # forward tiles channels over the grid
    a.grad_out = 256
    assert L.cgtp_uvu_validate(C.byref(a), 1) == 0                  # fp32 row mode: so does the backward ...
    a.grad_y = 256
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 1) == 8 * 10 * 9 * 4  # ... with grad_y partials of 8 channel chunks
    a.dtype = _lib.F64
    assert L.cgtp_uvu_validate(C.byref(a), 1) == 2                  # fp64 backward keeps a row inside one wavefront
    a.dtype, a.grad_y = _lib.F32, None
    a.C, a.w_shared, a.grad_w = 64, 1, 256
    # fp32 row mode runs on the block-wise kernels: 10 per-row weight gradients + 1 chunk partial of (P, C)
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 1) == (10 + 1) * 11 * 64 * 4
    a.dtype = _lib.F64
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 1) == 5 * 11 * 64 * 8   # fp64: 10 rows / 2 slots = 5 partial rows
    a.dtype = _lib.F32
    assert L.cgtp_uvu_bwd(C.byref(a), None) == 8                    # CGTP_ERR_WORKSPACE, nothing launched

    t = _lib.TriArgs()
    assert L.cgtp_tri_validate(C.byref(t)) == 2                     # C == 0
    t.C, t.n_out, t.nnz, t.n_rows = 8, 4, 30000, 3
    t.idx = t.seg = t.out = 256
    assert L.cgtp_tri_validate(C.byref(t)) == 6                     # 30000 * 8 B of table > 160 KB of LDS
    t.nnz = 100
    assert L.cgtp_tri_validate(C.byref(t)) == 0
    t.a.kind = 1
    assert L.cgtp_tri_validate(C.byref(t)) == 1                     # operand declared but no data
    assert L.cgtp_segment_sum(None, None, None, None, None, 1, 1, 1, 1, 0, None) == 1


def test_large_table_configs_and_row_gathers_validate_on_the_host():
    """lmax = 4..6 tables are served by the block-wise kernels only: fp32, row mode; a shared weight's gradient goes
    through per-row gradients in the workspace.  The row-mode backward accepts a separate gather for the rows of x."""
    from equitorch_amd import _lib
    from equitorch_amd._tables import fingerprint, tp_coo
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    L = _lib.lib
    sh6 = "0e+1o+2e+3o+4e+5o+6e"
    coo = tp_coo(tp_infos(Irreps(sh6), Irreps(sh6), Irreps(sh6))[0])
    cfg = L.cgtp_uvu_find(C.c_uint64(fingerprint(coo)))
    assert 0 <= cfg < L.cgtp_uvu_num_configs()
    dims = (C.c_int32 * 5)()
    assert L.cgtp_uvu_describe(cfg, dims) == fingerprint(coo) and tuple(dims) == (49, 49, 49, 106, 6460)
    a = _lib.UvuArgs()
    a.cfg, a.dtype, a.C, a.n_rows, a.n_x_rows = cfg, _lib.F32, 32, 10, 10
    a.x = a.y = a.w = a.out = a.grad_out = a.grad_x = a.grad_y = a.grad_w = 4096
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0 and L.cgtp_uvu_validate(C.byref(a), 1) == 0
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 1) == 0
    a.dtype = _lib.F64
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 4                  # fp32 only
    a.dtype, a.w_shared = _lib.F32, 1
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0 and L.cgtp_uvu_validate(C.byref(a), 1) == 0
    # shared weight: 10 per-row gradients + 1 chunk partial of (P, C) floats
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 1) == (10 + 1) * 106 * 32 * 4
    assert L.cgtp_uvu_bwd(C.byref(a), None) == 8                    # workspace missing, nothing launched
    a.w_shared, a.grad_w, a.n_seg, a.ptr, a.seg_ids, a.gather = 0, 4096, 10, 4096, 4096, 4096
    # segment mode on the block-wise kernels: one range per group of 32 lanes (C = 32: two per wavefront), at least
    # 4 positions each -> 3 ranges, 2 wavefronts, 2 partial rows per range slot
    assert L.cgtp_uvu_blockwise_only(cfg) == 1 and L.cgtp_uvu_blockwise_only(0) == 0
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0 and L.cgtp_uvu_validate(C.byref(a), 1) == 0
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 0) == 2 * 2 * 2 * 49 * 32 * 4
    a.pos_per_wave = 1                                              # here: positions per range -> 10 ranges, 5 wavefronts
    assert L.cgtp_uvu_workspace_bytes(C.byref(a), 1) == 5 * 2 * 2 * 49 * 32 * 4
    a.pos_per_wave = 0
    a.w_shared = 1
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0 and L.cgtp_uvu_validate(C.byref(a), 1) == 2   # no shared-weight gradient
    a.w_shared, a.C = 0, 65
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2                  # one wavefront wide at most
    a.C, a.wave_seg, a.n_waves = 32, 4096, 3
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2                  # ranges by position only
    a.wave_seg, a.n_waves = None, 0
    # row-mode backward with gathered x rows: x may then have any number of rows
    a.n_seg, a.ptr, a.seg_ids = 0, None, None
    a.n_x_rows = 4
    assert L.cgtp_uvu_validate(C.byref(a), 1) == 2
    a.x_gather = 4096
    assert L.cgtp_uvu_validate(C.byref(a), 1) == 0
    # channelled second operand ("uuu"): block-wise kernels, fp32, row mode, backward one wavefront wide
    b = _lib.UvuArgs()
    b.cfg, b.dtype, b.C, b.n_rows, b.n_x_rows, b.y_channels = cfg, _lib.F32, 64, 10, 10, 1
    b.x = b.y = b.w = b.out = b.grad_out = b.grad_x = b.grad_y = b.grad_w = 4096
    assert L.cgtp_uvu_validate(C.byref(b), 0) == 0 and L.cgtp_uvu_validate(C.byref(b), 1) == 0
    b.C = 128
    assert L.cgtp_uvu_validate(C.byref(b), 0) == 0 and L.cgtp_uvu_validate(C.byref(b), 1) == 0   # chunks of 64
    b.C, b.dtype = 64, _lib.F64
    assert L.cgtp_uvu_validate(C.byref(b), 0) == 4
    b.dtype, b.n_seg, b.ptr, b.seg_ids, b.gather = _lib.F32, 10, 4096, 4096, 4096
    assert L.cgtp_uvu_validate(C.byref(b), 0) == 2                  # no segment mode


def test_uv_matrix_core_entry_points_validate_on_the_host():
    """cgtp_uv_*: config lookup by fingerprint and argument checks, no launch (n_rows = 0 or a failing check)."""
    from equitorch_amd import _lib
    from equitorch_amd._tables import fingerprint, tp_coo
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    L = _lib.lib
    sh3 = "0e+1o+2e+3o"
    coo = tp_coo(tp_infos(Irreps(sh3), Irreps(sh3), Irreps(sh3))[0])
    cfg = L.cgtp_uv_find(C.c_uint64(fingerprint(coo)))
    assert 0 <= cfg < L.cgtp_uv_num_configs()
    assert L.cgtp_uv_find(C.c_uint64(12345)) == -1
    p16 = 4096  # any non-null, 16-byte aligned address: nothing is dereferenced by the checks
    assert L.cgtp_uv_validate(cfg, 0, p16, p16, p16, p16, 100, 128, 128, _lib.BF16) == 0
    assert L.cgtp_uv_validate(cfg, 2, p16, p16, p16, p16, 100, 128, 128, _lib.BF16) == 2       # direction
    assert L.cgtp_uv_validate(cfg, 0, p16, p16, p16, p16, 100, 128, 128, _lib.F32) == 4        # dtype
    assert L.cgtp_uv_validate(cfg, 0, p16, p16, p16, p16, 100, 48, 128, _lib.BF16) == 2        # C_in not 32/64/128
    assert L.cgtp_uv_validate(cfg, 0, p16, p16, p16, p16, 100, 128, 80, _lib.BF16) == 2        # C_out % 32
    assert L.cgtp_uv_validate(cfg, 0, p16 + 2, p16, p16, p16, 100, 128, 128, _lib.BF16) == 3   # alignment
    assert L.cgtp_uv_validate(cfg, 0, None, p16, p16, p16, 100, 128, 128, _lib.BF16) == 1      # null
    assert L.cgtp_uv_validate(99, 0, p16, p16, p16, p16, 100, 128, 128, _lib.BF16) == 5        # config
    assert L.cgtp_uv_apply(cfg, 0, p16, p16, p16, p16, 0, 128, 128, _lib.BF16, None) == 0      # empty batch
    assert L.cgtp_uv_grad_y(cfg, p16, p16, p16, p16, 0, 128, 128, _lib.BF16, None) == 0
    assert L.cgtp_uv_grad_y(cfg, p16, p16, p16, p16, 10, 128, 256, _lib.BF16, None) == 2       # C_out > 128
    assert L.cgtp_uv_pack_weights(0, p16, p16, 0, 128, 128, _lib.BF16, None, None) == 0
    assert L.cgtp_uv_pack_weights(0, p16, p16, 23, 100, 128, _lib.BF16, None, None) == 2
    assert L.cgtp_uv_pack_weights(3, p16, p16, 23, 128, 128, _lib.BF16, None, None) == 2
    # weight gradient: one fp32 partial of (P, C_in, C_out) per chunk of 512 samples
    assert L.cgtp_uv_grad_w_workspace_bytes(cfg, 32768, 128, 128) == 64 * 23 * 128 * 128 * 4
    assert L.cgtp_uv_grad_w_workspace_bytes(cfg, 513, 32, 64) == 2 * 23 * 32 * 64 * 4
    assert L.cgtp_uv_grad_w(cfg, p16, p16, p16, p16, None, 100, 128, 128, _lib.BF16, None, None) == 8  # workspace missing
    assert L.cgtp_uv_grad_w(cfg, p16, p16, p16, p16, p16, 100, 128, 160, _lib.BF16, None, None) == 2


def test_spherical_harmonics_entry_points_validate_on_the_host():
    from equitorch_amd import _lib
    L = _lib.lib
    assert L.cgtp_sh_max_degree() == 17
    assert L.cgtp_sh_forward(None, None, 0, 3, 1, 1.0, _lib.F32, None) == 0          # empty batch: no launch
    assert L.cgtp_sh_forward(None, 4096, 5, 3, 1, 1.0, _lib.F32, None) == 1          # null
    assert L.cgtp_sh_forward(4096, 4096, 5, 18, 1, 1.0, _lib.F32, None) == 2         # degree above 17
    assert L.cgtp_sh_forward(4096, 4096, -1, 2, 1, 1.0, _lib.F32, None) == 2
    assert L.cgtp_sh_forward(4096, 4096, 5, 2, 1, 1.0, _lib.BF16, None) == 4         # fp32 / fp64 only
    assert L.cgtp_sh_backward(4096, None, 4096, 5, 2, 1, 1.0, _lib.F64, None) == 1
    assert L.cgtp_sh_backward(4096, 4096, 4096, 0, 2, 1, 1.0, _lib.F64, None) == 0


def test_cpu_tensors_are_rejected_loudly():
    import torch
    from equitorch_amd import _lib
    from equitorch_amd.nn import SO3Linear
    m = SO3Linear("0e+1o", "0e+1o", "0e+1o", 4, 4)
    with pytest.raises(_lib.CgtpError, match="GPU only"):
        m(torch.randn(2, 4, 4), torch.randn(2, 4))


def test_tables_of_a_module_in_reduced_precision_find_their_config():
    """``module.to(torch.bfloat16)`` moves the coefficient tables too; such a table matches the compiled config whose
    fp32 coefficients round to it (cgtp_uvu_find_rounded / cgtp_uv_find_rounded), and only that one."""
    import torch
    from equitorch_amd import _lib
    from equitorch_amd._tables import fingerprint, round_coefficients, tp_coo
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import tp_infos
    L = _lib.lib
    # the rounding is torch's
    c = torch.randn(1000, dtype=torch.float64).numpy()
    for name, dt in (("bf16", torch.bfloat16), ("f16", torch.float16)):
        want = torch.from_numpy(c).float().to(dt).float().numpy()
        assert (round_coefficients(c, name) == want).all()
    for irreps, find, find_rounded, of in (
            ("0e+1o+2e", L.cgtp_uvu_find, L.cgtp_uvu_find_rounded, kernels.uvu_config_of),
            ("0e+1o+2e+3o", L.cgtp_uv_find, L.cgtp_uv_find_rounded, kernels.uv_config_of)):
        irr = Irreps(irreps)
        info = tp_infos(irr, irr, irr)[0]
        cfg = find(C.c_uint64(fingerprint(tp_coo(info))))
        assert cfg >= 0
        for name, dt, code in (("bf16", torch.bfloat16, _lib.BF16), ("f16", torch.float16, 3)):
            low = info._apply(lambda t: t.to(dt) if t.is_floating_point() else t)
            assert low.info_Mij_fwd.scale.dtype == dt
            fp = fingerprint(tp_coo(low), name)
            assert fp == fingerprint(tp_coo(info), name) != fingerprint(tp_coo(info))
            assert find_rounded(C.c_uint64(fp), code) == cfg == of(low)
            assert find(C.c_uint64(fp)) == -1                            # not an fp32 table
            assert find_rounded(C.c_uint64(fp), _lib.F32) == -1
        assert find_rounded(C.c_uint64(fingerprint(tp_coo(info), "bf16")), 3) == -1


def test_table_driven_matrix_core_entry_points_validate_on_the_host():
    """cgtp_uvt_*: launch shape queries and argument checks of the fp32 fully connected kernels, no launch."""
    from equitorch_amd import _lib
    L = _lib.lib
    p16 = 4096
    # lmax = 3, 128 -> 128 channels: four blocks of 16 k per ring turn; 16 output rows over 4 item groups (the other
    # two wavefronts of a sample block split the 128 output channels)
    assert L.cgtp_uvt_chunk(32768, 16, 16, 16, 128, 0, 128, _lib.F32) == 4
    assert L.cgtp_uvt_item_groups(32768, 16, 16, 16, 128, 0, 128, _lib.F32) == 4
    assert L.cgtp_uvt_item_groups(32768, 9, 9, 1, 32, 0, 64, _lib.F32) == 1           # a single output row
    assert L.cgtp_uvt_item_groups(32768, 9, 9, 9, 32, 0, 32, _lib.F64) == 8           # one wavefront covers the channels
    assert L.cgtp_uvt_chunk(100, 16, 16, 16, 130, 0, 128, _lib.F32) == -2             # channels not a multiple of 4
    assert L.cgtp_uvt_chunk(100, 49, 49, 49, 128, 0, 128, _lib.F32) == -6   # 16 samples x 49 rows x 128 floats > LDS
    assert L.cgtp_uvt_chunk(100, 16, 16, 16, 128, 0, 128, _lib.F64) == -6   # the same rows as doubles do not fit either
    assert L.cgtp_uvt_chunk(100, 16, 16, 16, 64, 0, 128, _lib.F64) == 2
    assert L.cgtp_uvt_chunk(100, 16, 16, 16, 64, 0, 128, _lib.BF16) == -4
    assert L.cgtp_uvt_packed_elems(23, 128, 128) == 23 * 8 * 8 * 256
    assert L.cgtp_uvt_packed_elems(2, 20, 12) == 2 * 2 * 4 * 256            # padded to whole ring turns / 4 blocks
    assert L.cgtp_uvt_packed_elems(2, 40, 12) == 2 * 4 * 4 * 256            # three blocks of k: two turns of a ring of two
    assert L.cgtp_uvt_packed_elems(2, 72, 12) == 2 * 6 * 4 * 256            # five blocks of k: three turns of a ring of two
    assert L.cgtp_uvt_packed_elems(2, 104, 12) == 2 * 8 * 4 * 256           # seven blocks: two turns of a ring of four
    assert L.cgtp_uvt_chunk(32768, 16, 16, 16, 32, 0, 128, _lib.F32) == 2
    assert L.cgtp_uvt_chunk(32768, 9, 9, 9, 4, 8, 16, _lib.F32) == 2         # K = 4 x 8
    assert L.cgtp_uvt_chunk(32768, 9, 9, 9, 8, 8, 16, _lib.F64) == 2         # K = 64
    assert L.cgtp_uvt_chunk(32768, 9, 9, 9, 8, 16, 16, _lib.F64) == 4
    a = _lib.UvtArgs()
    a.dtype = _lib.BF16
    assert L.cgtp_uvt_validate(C.byref(a)) == 4                             # fp32 only
    a.dtype = _lib.F32
    a.n_rows, a.dx, a.dy, a.dout, a.cx, a.cy, a.cout = 100, 9, 9, 9, 32, 0, 32
    assert L.cgtp_uvt_validate(C.byref(a)) == 2                             # kbi / groups not set
    a.kbi, a.n_groups = 4, 8
    assert L.cgtp_uvt_validate(C.byref(a)) == 2                             # up to 64 contracted channels: a ring of two
    a.kbi = 2
    a.n_items, a.n_terms = 35, 83
    for i in range(9):
        a.group_ptr[i] = min(5 * i, 35)
    assert L.cgtp_uvt_validate(C.byref(a)) == 1                             # null pointers
    a.x = a.y = a.wp = a.out = a.items = a.term_a = a.term_b = a.term_c = p16
    assert L.cgtp_uvt_validate(C.byref(a)) == 0
    a.group_ptr[8] = 34
    assert L.cgtp_uvt_validate(C.byref(a)) == 2                             # groups do not cover the items
    a.group_ptr[8] = 35
    a.x = p16 + 4
    assert L.cgtp_uvt_validate(C.byref(a)) == 3                             # alignment
    assert L.cgtp_uvt_pack_weights(p16, p16, 2, 0, 16, 1, 1, 1, _lib.F32, None) == 2
    assert L.cgtp_uvt_pack_weights(None, p16, 2, 16, 16, 1, 1, 1, _lib.F32, None) == 1
    # weight gradient: at most 128 chunks of samples; chunks of 256 samples, down to 32 while the launch would have
    # fewer than three workgroups per compute unit
    assert L.cgtp_uvt_grad_w_workspace_bytes(32768, 23, 128, 128, _lib.F32) == 128 * 23 * 128 * 128 * 4
    assert L.cgtp_uvt_grad_w_workspace_bytes(300, 4, 32, 16, _lib.F64) == 10 * 4 * 32 * 16 * 8
    assert L.cgtp_uvt_grad_w_workspace_bytes(8192, 23, 128, 128, _lib.F32) == 64 * 23 * 128 * 128 * 4
    # single precision weights of at most 64 x 64: one wavefront per (path, chunk), chunks of 32 samples or more, at
    # most 512 chunks and 8192 wavefronts
    assert L.cgtp_uvt_grad_w_workspace_bytes(4096, 3, 64, 64, _lib.F32) == 128 * 3 * 64 * 64 * 4
    assert L.cgtp_uvt_grad_w_workspace_bytes(65536, 3, 64, 64, _lib.F32) == 512 * 3 * 64 * 64 * 4
    assert L.cgtp_uvt_grad_w_workspace_bytes(4096, 100, 32, 48, _lib.F32) == 64 * 100 * 32 * 48 * 4
    assert L.cgtp_uvt_grad_w_workspace_bytes(4096, 3, 64, 64, _lib.F64) == 128 * 3 * 64 * 64 * 8
    g = _lib.UvtGwArgs()
    g.dtype = _lib.F32
    g.n_rows, g.n_paths, g.dx, g.dy, g.dg, g.cx, g.cy, g.cout = 10, 4, 9, 9, 9, 32, 0, 30
    g.x = g.y = g.g = g.gw = g.path_ptr = g.items = g.term_a = g.term_b = g.term_c = p16
    g.n_items = 1
    assert L.cgtp_uvt_grad_w(C.byref(g), None) == 2                         # cout not a multiple of 4
    g.cout = 32
    assert L.cgtp_uvt_grad_w(C.byref(g), None) == 8                         # workspace missing
    y = _lib.UvtGyArgs()
    y.dtype = _lib.F32
    y.n_rows, y.n_items, y.n_terms, y.dx, y.dy, y.dg, y.cx, y.cout = 0, 5, 9, 9, 9, 9, 32, 32
    assert L.cgtp_uvt_grad_y(C.byref(y), None) == 1                         # null pointers
    y.x = y.g = y.wp = y.gy = y.items = y.term_m = y.term_b = y.term_c = p16
    assert L.cgtp_uvt_grad_y(C.byref(y), None) == 0                         # empty batch: no launch
    y.dx, y.cx = 49, 128
    assert L.cgtp_uvt_grad_y(C.byref(y), None) == 6                         # 16 samples do not fit the LDS


def test_radial_mode_validates_on_the_host():
    """Per-edge weights formed in the kernel: segment mode, fp32, 64 channels, 4 | R <= 16, configs that keep four
    channels per lane (lmax <= 2 here)."""
    from equitorch_amd import _lib
    from equitorch_amd._tables import fingerprint, tp_coo
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.utils import tp_infos
    L = _lib.lib
    p16 = 4096

    def cfg_of(irr):
        return L.cgtp_uvu_find(C.c_uint64(fingerprint(tp_coo(tp_infos(Irreps(irr), Irreps(irr), Irreps(irr))[0]))))
    c2, c3 = cfg_of("0e+1o+2e"), cfg_of("0e+1o+2e+3o")
    assert L.cgtp_uvu_radial_supported(c2) == 1 and L.cgtp_uvu_radial_supported(c3) == 0
    assert L.cgtp_uvu_radial_supported(-1) == 0 and L.cgtp_uvu_radial_supported(999) == 0
    a = _lib.UvuArgs()
    a.cfg, a.dtype, a.C, a.n_rows, a.n_x_rows, a.n_seg = c2, _lib.F32, 64, 100, 10, 10
    a.ptr = a.seg_ids = a.gather = a.x = a.y = a.out = p16
    a.radial_h, a.radial_w, a.radial_r = p16, p16, 16
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 0                          # no weight tensor needed
    a.radial_r = 6
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2
    a.radial_r, a.C = 8, 32
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2                          # 64 channels only
    a.C, a.dtype = 64, _lib.F64
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 4
    a.dtype, a.radial_w = _lib.F32, None
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 1
    a.radial_w, a.cfg = p16, c3
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 5                          # no such kernels for this table
    a.cfg, a.path_scale = c2, p16
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 2                          # fold the factors into radial_w
    a.path_scale, a.radial_h = None, p16 + 4
    assert L.cgtp_uvu_validate(C.byref(a), 0) == 3
    # gradients of the features and the shared matrix: at most 512 partial sums of (R, P, 64) floats
    assert L.cgtp_uvu_radial_grad_workspace_bytes(65536, 16, 11) == 512 * 16 * 11 * 64 * 4
    assert L.cgtp_uvu_radial_grad_workspace_bytes(100, 8, 4) == 7 * 8 * 4 * 64 * 4
    assert L.cgtp_uvu_radial_grad(p16, p16, p16, p16, p16, None, 100, 16, 11, _lib.F32, None) == 8
    assert L.cgtp_uvu_radial_grad(p16, p16, p16, p16, p16, p16, 100, 20, 11, _lib.F32, None) == 2
    assert L.cgtp_uvu_radial_grad(p16, p16, p16, p16, p16, p16, 100, 16, 3, _lib.F32, None) == 2
    assert L.cgtp_uvu_radial_grad(p16, p16, p16, None, p16, p16, 100, 16, 11, _lib.F32, None) == 1
    assert L.cgtp_uvu_radial_grad(p16, p16, p16, p16, p16, p16, 100, 16, 11, _lib.F64, None) == 4


def test_radial_basis_and_cutoff_entry_points_validate_on_the_host():
    """``cgtp_bessel`` / ``cgtp_bessel_grad`` / ``cgtp_cutoff``: argument checks return before any launch."""
    from equitorch_amd import _lib
    L = _lib.lib
    p = 4096
    assert L.cgtp_bessel(p, p, p, 0, 8, 4.0, _lib.F32, None) == 0                 # nothing to do
    assert L.cgtp_bessel(None, p, p, 10, 8, 4.0, _lib.F32, None) == 1             # null
    assert L.cgtp_bessel(p, None, p, 10, 8, 4.0, _lib.F64, None) == 1
    assert L.cgtp_bessel(p, p, p, 10, 8, 4.0, _lib.BF16, None) == 4               # dtype
    assert L.cgtp_bessel(p, p, p, 10, 0, 4.0, _lib.F32, None) == 2                # no basis functions
    assert L.cgtp_bessel(p, p, p, 10, 8, 0.0, _lib.F32, None) == 2                # r_max
    assert L.cgtp_bessel(p, p, p, -1, 8, 4.0, _lib.F32, None) == 2
    assert L.cgtp_bessel_grad(p, p, p, None, None, 10, 8, 4.0, _lib.F32, None) == 0   # no gradient wanted
    assert L.cgtp_bessel_grad(p, p, None, p, None, 10, 8, 4.0, _lib.F32, None) == 1
    assert L.cgtp_cutoff(0, p, None, p, 0, 0.0, 4.0, 6.0, _lib.F64, None) == 0
    assert L.cgtp_cutoff(3, p, None, p, 10, 0.0, 4.0, 6.0, _lib.F32, None) == 2   # kind
    assert L.cgtp_cutoff(1, p, None, p, 10, 0.0, 0.0, 0.0, _lib.F32, None) == 2   # empty interval
    assert L.cgtp_cutoff(1, p, None, None, 10, 0.0, 4.0, 0.0, _lib.F32, None) == 1
    assert L.cgtp_cutoff(2, p, None, p, 10, 0.0, 4.0, 1e-7, _lib.F16, None) == 4


def test_torch_extension_loads_and_matches_the_library():
    """The PyTorch C++ extension over the C ABI imports without a GPU, was built against this libcgtp (ABI version),
    and takes a plan's index tensors as they are."""
    import torch

    from equitorch_amd import _lib, _shim
    mod = _shim.module()
    assert mod is not None, "equitorch_amd/lib/_cgtp_torch.so is not built"
    assert mod.abi_version() == _lib.lib.cgtp_version()
    i = torch.zeros(3, dtype=torch.int64)
    mod.EdgeHandle(0, 9, 0, None, i, None, i, i, None, i, i, i, i, i, torch.zeros(2, dtype=torch.int32), None)
