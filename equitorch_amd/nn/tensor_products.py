"""``TensorProduct``: weighted tensor product of two channelled features
(``equitorch/nn/tensor_products.py:19-198``); ``TensorDot``: irrep-wise dot product (``:199-262``)."""
import math
from typing import Optional

import torch
import torch.nn as nn
from torch import Tensor
from torch.nn import Parameter

from ..irreps import check_irreps
from ..structs import IrrepsInfo, TensorProductInfo
from ..utils._structs import tp_infos
from ._irreps_module import IrrepsModule
from .linears import _view_weight
from .functional.tensor_products import tensor_dot_uu, tensor_dot_uv, tensor_product_uuu, tensor_product_uvw
from .init import initialize_tensor_product


class TensorProduct(nn.Module):
    r"""``feature_mode='uuu'``: inputs ``(N, irreps_in{1,2}.dim, C)``, weight ``(num_paths, C)`` or
    ``(N, num_paths, C)`` -> ``(N, irreps_out.dim, C)``.

    ``feature_mode='uvw'``: inputs with ``C1`` / ``C2`` channels, weight ``(num_paths, C1, C2, C_out)``.
    """
    tp_info_forward: TensorProductInfo
    tp_info_backward1: TensorProductInfo
    tp_info_backward2: TensorProductInfo

    def __init__(self, irreps_in1, irreps_in2, irreps_out, channels_in1=None, channels_in2=None,
                 channels_out=None, internal_weights=True, feature_mode='uuu', path_norm=True,
                 channel_norm=False, path=None):
        super().__init__()
        self.irreps_in1 = check_irreps(irreps_in1)
        self.irreps_in2 = check_irreps(irreps_in2)
        self.irreps_out = check_irreps(irreps_out)
        self.irreps_in1_dim = self.irreps_in1.dim
        self.irreps_in2_dim = self.irreps_in2.dim
        self.irreps_out_dim = self.irreps_out.dim
        if feature_mode not in ('uvw', 'uuu'):
            raise ValueError(f'Feature_mode should be in ["uvw", "uuu"], got {feature_mode}.')
        assert not internal_weights or (channels_in1 is not None and channels_in2 is not None
                                        and channels_out is not None)
        self.channels_in1, self.channels_in2, self.channels_out = channels_in1, channels_in2, channels_out
        self.feature_mode = feature_mode
        self.path_norm = path_norm
        self.channel_norm = channel_norm and (feature_mode == 'uvw')
        fan_in = self.channels_in1 * self.channels_in2 if feature_mode == 'uvw' else 1
        (self.tp_info_forward, self.tp_info_backward1, self.tp_info_backward2, self.num_paths) = tp_infos(
            self.irreps_out, self.irreps_in1, self.irreps_in2, path=path, path_norm=path_norm,
            channel_norm=self.channel_norm, channel_scale=fan_in ** (-0.5))
        if feature_mode == 'uvw':
            self.weight_shape = (self.num_paths, channels_in1, channels_in2, channels_out)
        else:
            self.weight_shape = (self.num_paths, channels_out)
        self.weight_numel = math.prod(self.weight_shape) if None not in self.weight_shape else None
        self.internal_weights = internal_weights
        if internal_weights:
            self.weight = Parameter(torch.empty(*self.weight_shape))
            initialize_tensor_product(self.weight, feature_mode, channel_normed=self.channel_norm)
        else:
            self.weight = None

    def forward(self, input1: Tensor, input2: Tensor, weight: Optional[Tensor] = None) -> Tensor:
        assert input1.shape[-2] == self.irreps_in1_dim, \
            f"Input1 spherical dim mismatch: expected {self.irreps_in1_dim}, got {input1.shape[-2]}"
        assert input2.shape[-2] == self.irreps_in2_dim, \
            f"Input2 spherical dim mismatch: expected {self.irreps_in2_dim}, got {input2.shape[-2]}"
        if self.feature_mode == 'uuu':
            assert input1.shape[-1] == input2.shape[-1], "uuu mode needs equal channel counts"
        if self.internal_weights:
            assert weight is None, 'Do not pass the weight when self.internal_weights is True.'
            weight = self.weight
        else:
            assert weight is not None, 'Please pass the weight when self.internal_weights is False.'
            shape = self.weight_shape
            if None in shape:
                shape = ((self.num_paths, input1.shape[-1], input2.shape[-1], weight.shape[-1])
                         if self.feature_mode == 'uvw' else (self.num_paths, input1.shape[-1]))
            weight = _view_weight(weight, shape, math.prod(shape))
        infos = (self.tp_info_forward, self.tp_info_backward1, self.tp_info_backward2)
        if self.feature_mode == 'uuu':
            return tensor_product_uuu(input1, input2, weight, *infos)
        return tensor_product_uvw(input1, input2, weight, *infos)

    def _apply(self, *args, **kwargs):
        mod = super()._apply(*args, **kwargs)
        mod.tp_info_forward = self.tp_info_forward._apply(*args, **kwargs)
        mod.tp_info_backward1 = self.tp_info_backward1._apply(*args, **kwargs)
        mod.tp_info_backward2 = self.tp_info_backward2._apply(*args, **kwargs)
        return mod

    def __repr__(self):
        ch = (f"channels={self.channels_in1}" if self.feature_mode == 'uuu' else
              f"channels_in1={self.channels_in1}, channels_in2={self.channels_in2}, channels_out={self.channels_out}")
        return (f"{self.__class__.__name__}(irreps_in1={self.irreps_in1.short_repr()}, "
                f"irreps_in2={self.irreps_in2.short_repr()}, irreps_out={self.irreps_out.short_repr()}, {ch}, "
                f"feature_mode={self.feature_mode}, path_norm={self.path_norm}, "
                f"channel_norm={self.channel_norm}, internal_weights={self.internal_weights}, "
                f"num_paths={self.num_paths})")


class TensorDot(IrrepsModule):
    r"""Irrep-wise dot product of two features with the same irreps (``equitorch/nn/tensor_products.py:199-262``).

    ``feature_mode='uu'``: ``(..., irreps.dim, C), (..., irreps.dim, C) -> (..., len(irreps), C)``;
    ``'uv'`` (``-> (..., len(irreps), C1, C2)``) is declared by the reference but raises ``NotImplementedError``
    there, and does so here.  ``scaled`` divides by ``sqrt(2l+1)``.
    """
    irreps_info: IrrepsInfo

    def __init__(self, irreps, feature_mode, scaled=False):
        super().__init__(irreps)
        assert feature_mode in ['uv', 'uu']
        self.feature_mode = feature_mode
        self.scaled = scaled

    def forward(self, input1: Tensor, input2: Tensor) -> Tensor:
        assert input1.shape[-2] == self.irreps_dim, \
            f"Input1 spherical dim mismatch: expected {self.irreps_dim}, got {input1.shape[-2]}"
        assert input2.shape[-2] == self.irreps_dim, \
            f"Input2 spherical dim mismatch: expected {self.irreps_dim}, got {input2.shape[-2]}"
        if self.feature_mode == 'uu':
            assert input1.shape[-1] == input2.shape[-1], \
                f"Input channel dims must match in 'uu' mode. Got {input1.shape[-1]} and {input2.shape[-1]}"
            return tensor_dot_uu(input1, input2, self.irreps_info, self.scaled)
        return tensor_dot_uv(input1, input2, self.irreps_info, self.scaled)

    def extra_repr(self) -> str:
        return f"irreps={self.irreps}, feature_mode={self.feature_mode}, scaled={self.scaled}"
