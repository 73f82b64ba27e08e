"""ctypes binding of ``libcgtp.so`` (the C ABI declared in ``include/cgtp.h``).

The library is built in-tree by ``python -m equitorch_amd.csrc.build``; importing this module without it
raises — there is no fallback implementation.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libcgtp.so")

F32, F64, BF16, F16 = 0, 1, 2, 3
OPERAND_NONE, OPERAND_VEC, OPERAND_SCALAR = 0, 1, 2
_DTYPES = {torch.float32: F32, torch.float64: F64, torch.bfloat16: BF16, torch.float16: F16}


class CgtpError(RuntimeError):
    pass


class Operand(C.Structure):
    _fields_ = [("data", C.c_void_p), ("rows", C.c_void_p), ("row_stride", C.c_int64),
                ("idx_stride", C.c_int64), ("kind", C.c_int32), ("size", C.c_int32)]


class TriArgs(C.Structure):
    _fields_ = [("a", Operand), ("b", Operand), ("w", Operand),
                ("coef", C.c_void_p), ("idx", C.c_void_p), ("seg", C.c_void_p),
                ("n_out", C.c_int32), ("nnz", C.c_int32),
                ("out", C.c_void_p), ("workspace", C.c_void_p), ("n_rows", C.c_int64),
                ("C", C.c_int32), ("dtype", C.c_int32), ("reduce_c", C.c_int32), ("reduce_rows", C.c_int32)]


class GenOperand(C.Structure):
    _fields_ = [("data", C.c_void_p), ("row_stride", C.c_int64), ("idx_stride", C.c_int64),
                ("u_stride", C.c_int64), ("w_stride", C.c_int64), ("present", C.c_int32), ("_pad", C.c_int32)]


class GenArgs(C.Structure):
    _fields_ = [("a", GenOperand), ("b", GenOperand), ("w", GenOperand),
                ("coef", C.c_void_p), ("idx", C.c_void_p), ("seg", C.c_void_p),
                ("n_out", C.c_int32), ("nnz", C.c_int32), ("out", C.c_void_p), ("n_rows", C.c_int64),
                ("U", C.c_int32), ("W", C.c_int32), ("out_has_u", C.c_int32), ("out_has_w", C.c_int32),
                ("reduce_rows", C.c_int32), ("dtype", C.c_int32)]


class UvuArgs(C.Structure):
    _fields_ = [("cfg", C.c_int32), ("dtype", C.c_int32), ("C", C.c_int32), ("w_shared", C.c_int32),
                ("n_rows", C.c_int64), ("n_x_rows", C.c_int64), ("n_seg", C.c_int64),
                ("ptr", C.c_void_p), ("perm", C.c_void_p), ("seg_ids", C.c_void_p), ("gather", C.c_void_p),
                ("pos_per_wave", C.c_int32), ("y_vec", C.c_int32),
                ("wave_seg", C.c_void_p), ("n_waves", C.c_int64),
                ("x", C.c_void_p), ("y", C.c_void_p), ("w", C.c_void_p),
                ("out", C.c_void_p),
                ("grad_out", C.c_void_p), ("grad_x", C.c_void_p), ("grad_y", C.c_void_p),
                ("grad_w", C.c_void_p), ("workspace", C.c_void_p), ("x_gather", C.c_void_p),
                ("y_channels", C.c_int32), ("reserved_", C.c_int32), ("path_scale", C.c_void_p),
                ("radial_h", C.c_void_p), ("radial_w", C.c_void_p), ("radial_r", C.c_int32), ("reserved2_", C.c_int32),
                ("wave_pos", C.c_void_p)]


class UvuTab(C.Structure):
    _fields_ = [("coef", C.c_void_p), ("idx", C.c_void_p), ("paths", C.c_void_p),
                ("nnz", C.c_int32), ("n_segments", C.c_int32),
                ("D1", C.c_int32), ("D2", C.c_int32), ("DO", C.c_int32), ("P", C.c_int32)]


class PswTable(C.Structure):
    _fields_ = [("entries", C.c_void_p), ("coef", C.c_void_p), ("slots", C.c_void_p), ("blocks", C.c_void_p),
                ("n_entries", C.c_int32), ("n_slots", C.c_int32), ("n_blocks", C.c_int32), ("max_rows", C.c_int32),
                ("D1", C.c_int32), ("D2", C.c_int32), ("DO", C.c_int32), ("P", C.c_int32)]


class PswArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("w", C.c_void_p), ("out", C.c_void_p),
                ("g", C.c_void_p), ("gx", C.c_void_p), ("gy", C.c_void_p), ("gw", C.c_void_p),
                ("n_rows", C.c_int64), ("cx", C.c_int32), ("cy", C.c_int32), ("cout", C.c_int32),
                ("dtype", C.c_int32)]


class UvtItem(C.Structure):
    _fields_ = [("p", C.c_int32), ("kb0", C.c_int32), ("nkb", C.c_int32), ("t0", C.c_int32), ("t1", C.c_int32),
                ("out_row", C.c_int32), ("flags", C.c_int32), ("reserved_", C.c_int32)]


class UvtArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("wp", C.c_void_p), ("out", C.c_void_p),
                ("items", C.c_void_p), ("term_a", C.c_void_p), ("term_b", C.c_void_p), ("term_c", C.c_void_p),
                ("n_rows", C.c_int64), ("n_items", C.c_int32),
                ("dx", C.c_int32), ("dy", C.c_int32), ("dout", C.c_int32),
                ("cx", C.c_int32), ("cy", C.c_int32), ("cout", C.c_int32),
                ("kbi", C.c_int32), ("dtype", C.c_int32), ("n_terms", C.c_int32),
                ("n_groups", C.c_int32), ("group_ptr", C.c_int32 * 9)]


class UvtGwArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("y", C.c_void_p), ("g", C.c_void_p), ("gw", C.c_void_p), ("workspace", C.c_void_p),
                ("items", C.c_void_p), ("path_ptr", C.c_void_p), ("term_a", C.c_void_p), ("term_b", C.c_void_p),
                ("term_c", C.c_void_p), ("n_rows", C.c_int64),
                ("n_items", C.c_int32), ("n_terms", C.c_int32), ("n_paths", C.c_int32),
                ("dx", C.c_int32), ("dy", C.c_int32), ("dg", C.c_int32),
                ("cx", C.c_int32), ("cy", C.c_int32), ("cout", C.c_int32), ("dtype", C.c_int32),
                ("reserved_", C.c_int32)]


class UvtGyArgs(C.Structure):
    _fields_ = [("x", C.c_void_p), ("g", C.c_void_p), ("wp", C.c_void_p), ("gy", C.c_void_p),
                ("items", C.c_void_p), ("term_m", C.c_void_p), ("term_b", C.c_void_p), ("term_c", C.c_void_p),
                ("n_rows", C.c_int64), ("n_items", C.c_int32), ("n_terms", C.c_int32),
                ("dx", C.c_int32), ("dy", C.c_int32), ("dg", C.c_int32),
                ("cx", C.c_int32), ("cout", C.c_int32), ("dtype", C.c_int32)]


def _load():
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            f"{_LIB_PATH} is missing: build the HIP library first (python -m equitorch_amd.csrc.build). "
            "equitorch_amd has no non-HIP implementation of its operators.")
    lib = C.CDLL(_LIB_PATH)
    lib.cgtp_status_string.restype = C.c_char_p
    lib.cgtp_status_string.argtypes = [C.c_int]
    lib.cgtp_version.restype = C.c_int
    lib.cgtp_tri_workspace_bytes.restype = C.c_int64
    lib.cgtp_tri_workspace_bytes.argtypes = [C.POINTER(TriArgs)]
    lib.cgtp_tri_validate.argtypes = [C.POINTER(TriArgs)]
    lib.cgtp_tri_contract.argtypes = [C.POINTER(TriArgs), C.c_void_p]
    lib.cgtp_tri_contract_static.argtypes = [C.POINTER(TriArgs), C.c_void_p]
    lib.cgtp_tri_static_scratch_bytes.restype = C.c_int64
    lib.cgtp_gen_validate.argtypes = [C.POINTER(GenArgs)]
    lib.cgtp_gen_contract.argtypes = [C.POINTER(GenArgs), C.c_void_p]
    lib.cgtp_segment_sum.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                     C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_void_p]
    lib.cgtp_uvu_num_configs.restype = C.c_int
    lib.cgtp_uvu_find.argtypes = [C.c_uint64]
    lib.cgtp_uvu_find_rounded.argtypes = [C.c_uint64, C.c_int]
    lib.cgtp_uvu_describe.restype = C.c_uint64
    lib.cgtp_uvu_describe.argtypes = [C.c_int, C.POINTER(C.c_int32)]
    lib.cgtp_uvu_sh_degree.argtypes = [C.c_int]
    lib.cgtp_uvu_radial_supported.argtypes = [C.c_int]
    lib.cgtp_uvu_slots.argtypes = [C.c_int, C.c_int, C.c_int, C.c_int]
    lib.cgtp_uvu_blockwise_only.argtypes = [C.c_int]
    lib.cgtp_uvu_blockwise_only.restype = C.c_int
    lib.cgtp_uvu_radial_grad_workspace_bytes.restype = C.c_int64
    lib.cgtp_uvu_radial_grad_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int32]
    lib.cgtp_uvu_radial_grad.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]
    lib.cgtp_uvu_table.argtypes = [C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_int32)]
    lib.cgtp_uv_table.argtypes = [C.c_int, C.POINTER(C.c_int32), C.POINTER(C.c_float), C.POINTER(C.c_int32)]
    lib.cgtp_uvu_validate.argtypes = [C.POINTER(UvuArgs), C.c_int]
    lib.cgtp_uvu_workspace_bytes.restype = C.c_int64
    lib.cgtp_uvu_workspace_bytes.argtypes = [C.POINTER(UvuArgs), C.c_int]
    lib.cgtp_uvu_fwd.argtypes = [C.POINTER(UvuArgs), C.c_void_p]
    lib.cgtp_uvu_bwd.argtypes = [C.POINTER(UvuArgs), C.c_void_p]
    lib.cgtp_uvu_tab_workspace_bytes.restype = C.c_int64
    lib.cgtp_uvu_tab_workspace_bytes.argtypes = [C.POINTER(UvuArgs), C.POINTER(UvuTab), C.c_int]
    lib.cgtp_uvu_tab_validate.argtypes = [C.POINTER(UvuArgs), C.POINTER(UvuTab), C.c_int]
    lib.cgtp_uvu_tab_fwd.argtypes = [C.POINTER(UvuArgs), C.POINTER(UvuTab), C.c_void_p]
    lib.cgtp_uvu_tab_bwd.argtypes = [C.POINTER(UvuArgs), C.POINTER(UvuTab), C.c_void_p]
    lib.cgtp_bessel.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_double, C.c_int32, C.c_void_p]
    lib.cgtp_bessel_grad.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32,
                                     C.c_double, C.c_int32, C.c_void_p]
    lib.cgtp_cutoff.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_double, C.c_double, C.c_double,
                                C.c_int32, C.c_void_p]
    lib.cgtp_psw_validate.argtypes = [C.POINTER(PswArgs), C.POINTER(PswTable), C.c_int]
    lib.cgtp_psw_fwd.argtypes = [C.POINTER(PswArgs), C.POINTER(PswTable), C.c_void_p]
    lib.cgtp_psw_bwd.argtypes = [C.POINTER(PswArgs), C.POINTER(PswTable), C.c_void_p]
    lib.cgtp_uv_find.argtypes = [C.c_uint64]
    lib.cgtp_uv_find_rounded.argtypes = [C.c_uint64, C.c_int]
    _uv = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32,
           C.c_int32]
    lib.cgtp_uv_pack_weights.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
                                         C.c_void_p, C.c_void_p]
    lib.cgtp_uv_grad_y.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32,
                                   C.c_int32, C.c_int32, C.c_void_p]
    lib.cgtp_uv_grad_w_workspace_bytes.restype = C.c_int64
    lib.cgtp_uv_grad_w_workspace_bytes.argtypes = [C.c_int, C.c_int64, C.c_int32, C.c_int32]
    lib.cgtp_uv_grad_w.argtypes = [C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64,
                                   C.c_int32, C.c_int32, C.c_int32, C.c_void_p, C.c_void_p]
    lib.cgtp_uv_validate.argtypes = _uv
    lib.cgtp_uv_apply.argtypes = _uv + [C.c_void_p]
    lib.cgtp_uvt_packed_elems.restype = C.c_int64
    lib.cgtp_uvt_packed_elems.argtypes = [C.c_int32, C.c_int64, C.c_int32]
    lib.cgtp_uvt_pack_weights.argtypes = [C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_int64, C.c_int64,
                                          C.c_int64, C.c_int32, C.c_void_p]
    lib.cgtp_uvt_chunk.argtypes = [C.c_int64] + [C.c_int32] * 7
    lib.cgtp_uvt_item_groups.argtypes = [C.c_int64] + [C.c_int32] * 7
    lib.cgtp_uvt_validate.argtypes = [C.POINTER(UvtArgs)]
    lib.cgtp_uvt_apply.argtypes = [C.POINTER(UvtArgs), C.c_void_p]
    lib.cgtp_uvt_grad_w_workspace_bytes.restype = C.c_int64
    lib.cgtp_uvt_grad_w_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int64, C.c_int32, C.c_int32]
    lib.cgtp_uvt_grad_w.argtypes = [C.POINTER(UvtGwArgs), C.c_void_p]
    lib.cgtp_uvt_grad_y.argtypes = [C.POINTER(UvtGyArgs), C.c_void_p]
    lib.cgtp_sh_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_double, C.c_int,
                                    C.c_void_p]
    lib.cgtp_sh_backward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int, C.c_int, C.c_double,
                                     C.c_int, C.c_void_p]
    _seg = C.POINTER(C.c_int32)
    lib.cgtp_layer_rms_supported.argtypes = [_seg, C.c_int, C.c_int, C.c_int]
    lib.cgtp_layer_rms_workspace_bytes.argtypes = [C.c_int64, C.c_int, C.c_int, C.c_int]
    lib.cgtp_layer_rms_workspace_bytes.restype = C.c_int64
    _rd = C.POINTER(C.c_float)
    lib.cgtp_layer_rms_forward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, _seg, _rd, C.c_int,
                                           C.c_int64, C.c_int, C.c_int, C.c_int, C.c_double, C.c_int, C.c_void_p]
    lib.cgtp_layer_rms_backward.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.c_void_p, _seg, _rd, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_int,
                                            C.c_int, C.c_void_p]
    lib.cgtp_wigner_rotate_supported.argtypes = [_seg, _seg, C.c_int, C.c_int, C.c_int]
    lib.cgtp_wigner_rotate.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, _seg,
                                       _seg, C.c_int, C.c_int64, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p]
    lib.cgtp_wigner_rotate_backward.argtypes = [C.c_void_p] * 6 + [_seg, _seg, C.c_int, C.c_int64, C.c_int, C.c_int] + \
        [C.c_void_p] * 4 + [C.c_int, C.c_void_p]
    lib.cgtp_abi_layout.argtypes = [C.c_int, C.POINTER(C.c_int64), C.c_int]
    return lib


lib = _load()


def check(status: int, what: str = "cgtp"):
    if status != 0:
        raise CgtpError(f"{what}: {lib.cgtp_status_string(status).decode()} (status {status})")


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPES[dtype]
    except KeyError:
        raise CgtpError(f"unsupported dtype {dtype}") from None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def stream_ptr(device) -> int:
    """The current stream of ``device`` as a raw handle.  Asked from torch directly where it offers that (a tenth of the
    time of building a ``torch.cuda.Stream`` object per launch)."""
    if _raw_stream is not None:
        index = device.index if isinstance(device, torch.device) else device
        return _raw_stream(torch.cuda.current_device() if index is None else index)
    return torch.cuda.current_stream(device).cuda_stream


def ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise CgtpError("equitorch_amd operators run on the GPU only (got a CPU tensor); "
                            "there is no CPU implementation in this package")
