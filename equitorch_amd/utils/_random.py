"""Random test inputs (``equitorch/utils/_random.py:5-18``)."""
import torch


def rand_spherical_xyz(shape, device=None, dtype=None, generator=None) -> torch.Tensor:
    """Gaussian-normalised random unit vectors of shape ``(*shape, 3)``."""
    xyz = torch.randn(*shape, 3, device=device, dtype=dtype, generator=generator)
    return xyz / xyz.norm(dim=-1, keepdim=True)
