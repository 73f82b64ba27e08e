"""Constant-table containers of the sparse tensor-product path.

Field names, order and defaults follow ``equitorch/structs/__init__.py:50-102`` so tables built here can be
passed wherever the reference's NamedTuples are expected; ``_apply`` / ``to`` / ``cuda`` / ``cpu`` behave as
the decorator at ``:7-48`` (``to(dtype)`` converts floating tensors only, index tensors keep ``int64``).
"""
from typing import Any, Callable, NamedTuple, Optional

import torch
from torch import Tensor


def _movable(cls):
    def _apply(self, fn: Callable[[Any], Any]):
        vals = []
        for v in self:
            if isinstance(v, Tensor):
                vals.append(fn(v))
            elif hasattr(v, "_apply") and isinstance(v, tuple):
                vals.append(v._apply(fn))
            else:
                vals.append(v)
        return type(self)(*vals)

    def to(self, *args, **kwargs):
        device, dtype, non_blocking, _ = torch._C._nn._parse_to(*args, **kwargs)

        def conv(t: Tensor):
            return t.to(device=device, dtype=dtype if (dtype is not None and t.is_floating_point()) else None,
                        non_blocking=non_blocking)
        return self._apply(conv)

    cls._apply = _apply
    cls.to = to
    cls.cuda = lambda self, *a, **k: self._apply(lambda t: t.cuda(*a, **k))
    cls.cpu = lambda self, *a, **k: self._apply(lambda t: t.cpu(*a, **k))
    return cls


add_operation_methods = _movable   # the reference's name for this class decorator (``structs/__init__.py:7-47``)


@_movable
class SparseScaleInfo(NamedTuple):
    """``z[M] = sum_{t in seg_out[M]..seg_out[M+1]} scale[t] * x[index[t]]``."""
    scale: Optional[Tensor] = None      # (T,) floating
    index: Optional[Tensor] = None      # (T,) int64 in [0, in_size); None = identity
    seg_out: Optional[Tensor] = None    # (out_size+1,) int64 CSR pointer; None = one term per output
    index_out: Optional[Tensor] = None  # never produced by the builders
    out_size: Optional[int] = None


@_movable
class SparseProductInfo(NamedTuple):
    """``z[M] = sum_{t in seg_out[M]..seg_out[M+1]} scale[t] * x[index1[t]] * y[index2[t]]``."""
    scale: Optional[Tensor] = None
    index1: Optional[Tensor] = None
    index2: Optional[Tensor] = None
    seg_out: Optional[Tensor] = None
    gather_index: Optional[Tensor] = None  # never produced by the builders
    index_out: Optional[Tensor] = None     # never produced by the builders
    out_size: Optional[int] = None


@_movable
class TensorProductInfo(NamedTuple):
    info_Mij_fwd: SparseProductInfo
    info_Mij_bwd1: SparseProductInfo
    info_Mij_bwd2: SparseProductInfo

    info_M_fwd: SparseProductInfo
    info_M_bwd1: SparseProductInfo
    info_M_bwd2: SparseProductInfo

    info_kM1j_fwd: SparseProductInfo
    info_kM1j_bwd1: SparseProductInfo
    info_kM1j_bwd2: SparseProductInfo
    info_kM1M2_fwd: SparseProductInfo
    info_kM1M2_bwd1: SparseProductInfo
    info_kM1M2_bwd2: SparseProductInfo
    info_M_kM1M2_fwd: SparseScaleInfo
    info_M_kM1M2_bwd: SparseScaleInfo
    out_size: int


@_movable
class IrrepsInfo(NamedTuple):
    """Per-irrep constants of an ``Irreps`` (``equitorch/structs/__init__.py:106-111``)."""
    rsqrt_dims: Tensor      # (num_irreps,) (2l+1)^-1/2
    rdims: Tensor           # (num_irreps,) 1/(2l+1)
    irrep_index: Tensor     # (dim,) irrep of every component
    irrep_seg: Tensor       # (num_irreps+1,) first component of every irrep
    num_irreps: int


@_movable
class IrrepsLinearInfo(NamedTuple):
    """Tables of the irreps-preserving channel mixing (``equitorch/structs/__init__.py:114-130``): entries
    ``(M, M0, path)`` sorted by output component, and the same entries sorted by path for the weight gradient."""
    scale_MM0: Tensor
    M_seg_MM0: Tensor
    ii0_MM0: Tensor
    M0_MM0: Tensor
    M_MM0: Tensor
    M_out: Tensor

    ii0_seg_ii0MM0: Tensor
    M_ii0MM0: Tensor
    M0_ii0MM0: Tensor
    scales_ii0: Tensor

    out_size: int


@_movable
class WignerRotationInfo(NamedTuple):
    """Tables of a rotation applied as ``Z(alpha) J Z(beta) J Z(gamma)``
    (``equitorch/structs/__init__.py:133-139``)."""
    j_matrix_info: SparseScaleInfo
    rotate_z_info_fwd: SparseProductInfo
    rotate_z_info_bwd_input: Optional[SparseProductInfo] = None
    rotate_z_info_bwd_cs: Optional[SparseProductInfo] = None
    sign: Optional[Tensor] = None
    max_m: Optional[int] = None
