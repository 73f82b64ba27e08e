"""Shared plumbing of the modules that act on one ``Irreps`` through its ``IrrepsInfo`` tables."""
from torch import Tensor, nn

from ..irreps import check_irreps
from ..structs import IrrepsInfo
from ..utils._structs import irreps_info


class IrrepsModule(nn.Module):
    """Holds ``irreps`` and ``irreps_info`` and moves the tables with the module (``.to()``, ``.cuda()``)."""
    irreps_info: IrrepsInfo

    def __init__(self, irreps):
        super().__init__()
        self.irreps = check_irreps(irreps)
        self.irreps_dim = self.irreps.dim
        self.irreps_info = irreps_info(self.irreps)

    def _check_dim(self, input_tensor: Tensor) -> None:
        if input_tensor.shape[-2] != self.irreps_dim:
            raise ValueError(f"Input tensor's irreps dimension ({input_tensor.shape[-2]}) does not match expected "
                             f"irreps dimension ({self.irreps_dim})")

    def _apply(self, *args, **kwargs):
        mod = super()._apply(*args, **kwargs)
        mod.irreps_info = self.irreps_info._apply(*args, **kwargs)
        return mod
