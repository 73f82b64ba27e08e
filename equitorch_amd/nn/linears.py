"""``SO3Linear``: tensor product of a channelled feature with a channel-less one (edge harmonics);
``IrrepWiseLinear`` / ``IrrepsLinear``: channel mixing that leaves the irreps structure alone.

Constructors, attributes, ``forward`` contracts and ``repr`` follow ``equitorch/nn/linears.py:26-411``.
"""
import math
from typing import Optional

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn import Parameter

from .._lib import require_gpu as _lib_require
from ..irreps import check_irreps
from ..structs import IrrepsInfo, IrrepsLinearInfo, TensorProductInfo
from ..utils._structs import irreps_info, irreps_linear_infos, so2_linear_infos, tp_infos
from .functional.linears import irrep_wise_linear, irreps_linear, so3_linear_uu, so3_linear_uv
from .functional.sparse_product import sparse_mul, sparse_vecmat
from .init import initialize_linear, initialize_so3_so2_linear


class SO3Linear(nn.Module):
    r"""``feature_mode='uu'``: ``input1 (N, irreps_in1.dim, C)``, ``input2 (N, irreps_in2.dim)``, weight
    ``(num_paths, C)`` (shared) or ``(N, num_paths, C)`` (per sample) -> ``(N, irreps_out.dim, C)``.

    ``feature_mode='uv'``: weight ``(num_paths, C_in, C_out)`` (or with a leading ``N``), output
    ``(N, irreps_out.dim, C_out)``.
    """
    tp_info_forward: TensorProductInfo
    tp_info_backward1: TensorProductInfo
    tp_info_backward2: TensorProductInfo

    def __init__(self, irreps_in1, irreps_in2, irreps_out, channels_in=None, channels_out=None,
                 internal_weights=True, feature_mode='uu', path_norm=True, channel_norm=False, path=None):
        super().__init__()
        self.irreps_in1 = check_irreps(irreps_in1)
        self.irreps_in2 = check_irreps(irreps_in2)
        self.irreps_out = check_irreps(irreps_out)
        self.irreps_in1_dim = self.irreps_in1.dim
        self.irreps_in2_dim = self.irreps_in2.dim
        self.irreps_out_dim = self.irreps_out.dim
        assert not internal_weights or (channels_in is not None and channels_out is not None)
        if feature_mode not in ('uu', 'uv'):
            raise ValueError(f'Feature_mode should be in ["uv", "uu"], got {feature_mode}.')
        self.channels_in = channels_in
        self.channels_out = channels_out
        self.feature_mode = feature_mode
        self.path_norm = path_norm
        self.channel_norm = channel_norm and (feature_mode == 'uv')
        fan_in = self.channels_in if feature_mode == 'uv' else 1
        (self.tp_info_forward, self.tp_info_backward1, self.tp_info_backward2, self.num_paths) = tp_infos(
            self.irreps_out, self.irreps_in1, self.irreps_in2, path=path, path_norm=path_norm,
            channel_norm=self.channel_norm, channel_scale=fan_in ** (-0.5))
        if feature_mode == 'uv':
            self.weight_shape = (self.num_paths, self.channels_in, self.channels_out)
        else:
            self.weight_shape = (self.num_paths, self.channels_out)
        self.weight_numel = math.prod(self.weight_shape) if None not in self.weight_shape else None
        self.internal_weights = internal_weights
        if internal_weights:
            self.weight = Parameter(torch.empty(*self.weight_shape))
            initialize_so3_so2_linear(self.weight, feature_mode, channel_normed=self.channel_norm)
        else:
            self.weight = None

    def _resolve_weight(self, input1: Tensor, weight: Optional[Tensor]) -> Tensor:
        if self.internal_weights:
            assert weight is None, 'Do not pass the weight when self.internal_weights is True.'
            return self.weight
        assert weight is not None, 'Please pass the weight when self.internal_weights is False.'
        shape = self.weight_shape
        if None in shape:  # channels were not given at construction: take them from the input
            shape = ((self.num_paths, input1.shape[-1], weight.shape[-1]) if self.feature_mode == 'uv'
                     else (self.num_paths, input1.shape[-1]))
        return _view_weight(weight, shape, math.prod(shape))

    def forward(self, input1: Tensor, input2: Tensor, weight: Optional[Tensor] = None):
        assert input1.shape[-2] == self.irreps_in1_dim, \
            f"Input1 spherical dim mismatch: expected {self.irreps_in1_dim}, got {input1.shape[-2]}"
        assert input2.shape[-1] == self.irreps_in2_dim, \
            f"Input2 spherical dim mismatch: expected {self.irreps_in2_dim}, got {input2.shape[-1]}"
        assert input2.ndim == input1.ndim - 1, \
            f"Input2 should have one less dimension than Input1. Got input1 ndim={input1.ndim}, input2 ndim={input2.ndim}"
        assert self.channels_in is None or input1.shape[-1] == self.channels_in, \
            f"Input1 channel dim mismatch: expected {self.channels_in}, got {input1.shape[-1]}"
        weight = self._resolve_weight(input1, weight)
        infos = (self.tp_info_forward, self.tp_info_backward1, self.tp_info_backward2)
        if self.feature_mode == 'uu':
            return so3_linear_uu(input1, input2, weight, *infos)
        return so3_linear_uv(input1, input2, weight, *infos)

    def _apply(self, *args, **kwargs):
        mod = super()._apply(*args, **kwargs)
        mod.tp_info_forward = self.tp_info_forward._apply(*args, **kwargs)
        mod.tp_info_backward1 = self.tp_info_backward1._apply(*args, **kwargs)
        mod.tp_info_backward2 = self.tp_info_backward2._apply(*args, **kwargs)
        return mod

    def __repr__(self):
        ch = (f"channels={self.channels_in}" if self.feature_mode == 'uu'
              else f"channels_in={self.channels_in}, channels_out={self.channels_out}")
        return (f"{self.__class__.__name__}(irreps_in1={self.irreps_in1.short_repr()}, "
                f"irreps_in2={self.irreps_in2.short_repr()}, irreps_out={self.irreps_out.short_repr()}, {ch}, "
                f"feature_mode={self.feature_mode}, path_norm={self.path_norm}, "
                f"channel_norm={self.channel_norm}, internal_weights={self.internal_weights}, "
                f"num_paths={self.num_paths})")


def _view_weight(weight: Tensor, shape, numel: int) -> Tensor:
    """The reference's rule (``equitorch/nn/linears.py:163-168``): more elements than one set of weights means a set
    per sample.  A weight without elements (an empty batch with per-sample weights, which the reference's ``view``
    rejects as ambiguous) is per-sample with zero samples."""
    if weight.numel() == 0 and numel > 0:
        return weight.view(0, *shape)
    return weight.view(-1, *shape) if weight.numel() > numel else weight.view(*shape)


class IrrepWiseLinear(nn.Module):
    r"""One ``(channels_in, channels_out)`` matrix per irrep of ``irreps`` applied to the channels
    (``equitorch/nn/linears.py:215-300``): ``(..., irreps.dim, channels_in) -> (..., irreps.dim, channels_out)``,
    weight ``(len(irreps), channels_in, channels_out)`` (or with a leading sample axis).  ``channel_norm`` divides
    the output by ``sqrt(channels_in)``."""
    irreps_info: IrrepsInfo

    def __init__(self, irreps, channels_in, channels_out, internal_weights=True, channel_norm: bool = False):
        super().__init__()
        self.irreps = check_irreps(irreps)
        self.irreps_dim = self.irreps.dim
        self.channels_in = channels_in
        self.channels_out = channels_out
        self.irreps_info = irreps_info(self.irreps)
        self.channel_norm = channel_norm
        self.num_paths = len(self.irreps)
        self.weight_shape = (self.num_paths, self.channels_in, self.channels_out)
        self.weight_numel = math.prod(self.weight_shape)
        self.internal_weights = internal_weights
        if internal_weights:
            self.weight = Parameter(torch.empty(*self.weight_shape))
            initialize_linear(self.weight, channel_normed=self.channel_norm)
        else:
            self.weight = None

    def forward(self, input: Tensor, weight: Optional[Tensor] = None):
        assert input.shape[-2] == self.irreps_dim, \
            f"Input spherical dim mismatch: expected {self.irreps_dim}, got {input.shape[-2]}"
        assert input.shape[-1] == self.channels_in, \
            f"Input channel dim mismatch: expected {self.channels_in}, got {input.shape[-1]}"
        if self.internal_weights:
            assert weight is None, 'Do not pass the weight when self.internal_weights is True.'
            weight = self.weight
        else:
            assert weight is not None, 'Please pass the weight when self.internal_weights is False.'
            weight = _view_weight(weight, self.weight_shape, self.weight_numel)
        output = irrep_wise_linear(input, weight, self.irreps_info)
        if self.channel_norm:
            output = output / (self.channels_in ** 0.5)
        return output

    def _apply(self, *args, **kwargs):
        tp = super()._apply(*args, **kwargs)
        tp.irreps_info = self.irreps_info._apply(*args, **kwargs)
        return tp

    def __repr__(self):
        return (f"{self.__class__.__name__}(irreps={self.irreps.short_repr()}, channels_in={self.channels_in}, "
                f"channels_out={self.channels_out}, channel_norm={self.channel_norm}, "
                f"internal_weights={self.internal_weights})")


class IrrepsLinear(nn.Module):
    r"""Channel mixing between input and output irreps of equal degree and compatible parity
    (``equitorch/nn/linears.py:302-411``): ``(..., irreps_in.dim, channels_in) -> (..., irreps_out.dim,
    channels_out)``, weight ``(num_paths, channels_in, channels_out)`` (or with a leading sample axis), one path
    per allowed ``(irrep_out, irrep_in)`` pair.  ``path_norm`` scales each path by ``count(paths into its output
    irrep)^-1/2``.  As in the reference, ``channel_norm`` multiplies the table scales by ``channels_in`` (the
    value its constructor hands to the table builder) and switches the initialiser to the un-normalised range."""
    forward_info: IrrepsLinearInfo
    backward_info: IrrepsLinearInfo

    def __init__(self, irreps_in, irreps_out, channels_in, channels_out, internal_weights=True, path_norm=True,
                 channel_norm=False, path=None):
        super().__init__()
        self.irreps_in = check_irreps(irreps_in)
        self.irreps_out = check_irreps(irreps_out)
        self.irreps_in_dim = self.irreps_in.dim
        self.irreps_out_dim = self.irreps_out.dim
        self.channels_in = channels_in
        self.channels_out = channels_out
        self.channel_norm = channel_norm
        self.path_norm = path_norm
        self.forward_info, self.backward_info, self.num_paths = irreps_linear_infos(
            self.irreps_out, self.irreps_in, path, path_norm, channel_norm, self.channels_in)
        self.weight_shape = (self.num_paths, self.channels_in, self.channels_out)
        self.weight_numel = math.prod(self.weight_shape)
        self.internal_weights = internal_weights
        if internal_weights:
            self.weight = Parameter(torch.empty(*self.weight_shape))
            initialize_linear(self.weight, channel_normed=channel_norm)
        else:
            self.weight = None

    def forward(self, input: Tensor, weight: Optional[Tensor] = None):
        assert input.shape[-2] == self.irreps_in_dim, \
            f"Input spherical dim mismatch: expected {self.irreps_in_dim}, got {input.shape[-2]}"
        assert input.shape[-1] == self.channels_in, \
            f"Input channel dim mismatch: expected {self.channels_in}, got {input.shape[-1]}"
        if self.internal_weights:
            assert weight is None, 'Do not pass the weight when self.internal_weights is True.'
            weight = self.weight
        else:
            assert weight is not None, 'Please pass the weight when self.internal_weights is False.'
            weight = _view_weight(weight, self.weight_shape, self.weight_numel)
        return irreps_linear(input, weight, self.forward_info, self.backward_info)

    def _apply(self, *args, **kwargs):
        tp = super()._apply(*args, **kwargs)
        tp.forward_info = self.forward_info._apply(*args, **kwargs)
        tp.backward_info = self.backward_info._apply(*args, **kwargs)
        return tp

    def __repr__(self):
        return (f"{self.__class__.__name__}(irreps_in={self.irreps_in.short_repr()}, "
                f"irreps_out={self.irreps_out.short_repr()}, channels_in={self.channels_in}, "
                f"channels_out={self.channels_out}, path_norm={self.path_norm}, channel_norm={self.channel_norm}, "
                f"internal_weights={self.internal_weights}, num_paths={self.num_paths})")


class SO2Linear(nn.Module):
    r"""Linear map between features expressed in the frame where the edge points along z
    (``equitorch/nn/linears.py:413-571``): components of equal ``|m|`` mix, with one weight for ``m = 0`` and a
    ``(w_+, w_-)`` pair acting like a complex number on the ``(+m, -m)`` pair otherwise, for every path
    ``(irrep_out, irrep_in)`` and ``m <= min(l_out, l_in)``.  ``feature_mode='uu'``: weight ``(num_weights, C)``,
    channel-wise; ``'uv'``: weight ``(num_weights, C_in, C_out)``; either may carry a leading sample axis."""

    def __init__(self, irreps_in, irreps_out, channels_in=None, channels_out=None, internal_weights=True,
                 feature_mode='uu', path_norm=True, channel_norm=False, path=None):
        super().__init__()
        self.irreps_in = check_irreps(irreps_in)
        self.irreps_out = check_irreps(irreps_out)
        assert not internal_weights or (channels_in is not None and channels_out is not None)
        if feature_mode not in ('uu', 'uv'):
            raise ValueError(f'Feature_mode should be in ["uv", "uu"], got {feature_mode}.')
        self.channels_in, self.channels_out = channels_in, channels_out
        self.internal_weights = internal_weights
        self.feature_mode = feature_mode
        self.path_norm = path_norm
        self.channel_norm = channel_norm and feature_mode == 'uv'
        channel_scale = self.channels_in ** (-0.5) if self.channel_norm else 1.0
        self.info_forward, self.info_backward1, self.info_backward2, self.num_weights = so2_linear_infos(
            self.irreps_out, self.irreps_in, path=path, path_norm=path_norm, channel_norm=self.channel_norm,
            channel_scale=channel_scale)
        if feature_mode == 'uv':
            self.weight_shape = (self.num_weights, self.channels_in, self.channels_out)
        else:
            self.weight_shape = (self.num_weights, self.channels_out)
        self.weight_numel = math.prod(self.weight_shape) if None not in self.weight_shape else None
        if internal_weights:
            self.weight = Parameter(torch.empty(*self.weight_shape))
            initialize_so3_so2_linear(self.weight, feature_mode, channel_normed=self.channel_norm)
        else:
            self.weight = None

    def forward(self, input: Tensor, weight: Optional[Tensor] = None):
        assert input.shape[-2] == self.irreps_in.dim, \
            f"Input spherical dim mismatch: expected {self.irreps_in.dim}, got {input.shape[-2]}"
        if self.channels_in is not None:
            assert input.shape[-1] == self.channels_in, \
                f"Input channel dim mismatch: expected {self.channels_in}, got {input.shape[-1]}"
        if self.internal_weights:
            assert weight is None, 'Do not pass the weight when self.internal_weights is True.'
            weight = self.weight
        else:
            assert weight is not None, 'Please pass the weight when self.internal_weights is False.'
            if self.weight_numel is not None:
                weight = _view_weight(weight, self.weight_shape, self.weight_numel)
        if self.feature_mode == 'uu':
            return sparse_mul(input, weight, self.info_forward, self.info_backward1, self.info_backward2)
        if (input.is_floating_point() and input.dtype == weight.dtype and weight.ndim in (3, 4)
                and weight.shape[-3] == self.num_weights and input.ndim >= 3):
            if weight.ndim == 3:
                _lib_require(input, weight)
                # every table entry is one (C_in, C_out) product on one component: the table-driven matrix-core
                # kernels of the fully connected product take the table as it is (16-bit operands widened, channel
                # counts filled up to multiples of 4)
                from .functional import _irreps_gemm as G
                plan = G.plan_of_product_info(self.info_forward, self.irreps_in.dim, self.num_weights)
                anchor = next(t for t in (self.info_forward.seg_out, self.info_forward.index1,
                                          self.info_forward.index2, self.info_forward.scale) if t is not None)
                x3 = input.reshape(-1, *input.shape[-2:]).contiguous()
                if not plan.paths:
                    return G.no_paths(x3, weight, plan).reshape(*input.shape[:-2], plan.out_size, weight.shape[-1])
                out = G._table_driven_path(x3, weight.contiguous(), plan, self.irreps_in.dim, anchor)
                if out is None and x3.shape[0] > 0:
                    out = G._adapted_path(x3, weight.contiguous(), plan, self.irreps_in.dim, anchor)
                if out is not None:
                    return out.reshape(*input.shape[:-2], plan.out_size, out.shape[-1])
                # one GEMM per order |m| over the components of that order side by side
                from .functional._so2_gemm import so2_linear_uv_shared
                return so2_linear_uv_shared(input, weight, self.info_forward, self.irreps_in.dim, self.num_weights)
            # per-sample weights: every table entry is a (C_in, C_out) GEMM on one component, batched over samples
            from .functional import _irreps_gemm as G
            plan = G.plan_of_product_info(self.info_forward, self.irreps_in.dim, self.num_weights)
            anchor = next(t for t in (self.info_forward.seg_out, self.info_forward.index1,
                                      self.info_forward.index2, self.info_forward.scale) if t is not None)
            return G.mix(input, weight, plan, self.irreps_in.dim, anchor=anchor)
        return sparse_vecmat(input, weight, self.info_forward, self.info_backward1, self.info_backward2)

    def _apply(self, *args, **kwargs):
        lin = super()._apply(*args, **kwargs)
        lin.info_forward = self.info_forward._apply(*args, **kwargs)
        lin.info_backward1 = self.info_backward1._apply(*args, **kwargs)
        lin.info_backward2 = self.info_backward2._apply(*args, **kwargs)
        return lin

    def __repr__(self):
        channels = (f"channels={self.channels_in}" if self.feature_mode == 'uu'
                    else f"channels_in={self.channels_in}, channels_out={self.channels_out}")
        return (f"{self.__class__.__name__}(irreps_in={self.irreps_in.short_repr()}, "
                f"irreps_out={self.irreps_out.short_repr()}, {channels}, feature_mode={self.feature_mode}, "
                f"path_norm={self.path_norm}, channel_norm={self.channel_norm}, "
                f"internal_weights={self.internal_weights}, num_weights={self.num_weights})")
