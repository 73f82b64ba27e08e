"""Weight initialisers of the tensor-product modules (``equitorch/nn/init.py:3-91``): uniform in
``[-a, a]`` with ``a = sqrt(3) * gain`` for the channel-wise modes (and for channel-normalised fully
connected modes), ``a = sqrt(3 / fan_in) * gain`` otherwise; ``initialize_linear`` (``:93-120``) is the
same rule for plain channel mixing."""
import math

import torch


def initialize_tensor_product(weight, feature_mode, gain=1, channel_normed=False):
    if feature_mode == 'uvw':
        fan_in = weight.shape[-2] * weight.shape[-3]
        a = math.sqrt(3.0) * gain if channel_normed else math.sqrt(3.0 / fan_in) * gain
    elif feature_mode == 'uuu':
        a = math.sqrt(3.0) * gain
    else:
        raise ValueError(f"Unknown feature_mode '{feature_mode}' for initialize_tensor_product")
    torch.nn.init.uniform_(weight, -a, a)


def initialize_so3_so2_linear(weight, feature_mode, gain=1, channel_normed=False):
    if feature_mode == 'uv':
        fan_in = weight.shape[-2]
        a = math.sqrt(3.0) * gain if channel_normed else math.sqrt(3.0 / fan_in) * gain
    elif feature_mode == 'uu':
        a = math.sqrt(3.0) * gain
    else:
        raise ValueError(f"Unknown feature_mode '{feature_mode}' for initialize_so3_so2_linear")
    torch.nn.init.uniform_(weight, -a, a)


def initialize_linear(weight, gain=1, channel_normed=False):
    fan_in = weight.shape[-2]
    a = math.sqrt(3.0) * gain if channel_normed else math.sqrt(3.0 / fan_in) * gain
    torch.nn.init.uniform_(weight, -a, a)
