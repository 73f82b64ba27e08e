"""``Dropout`` (``equitorch/nn/dropout.py``)."""
import torch.nn.functional as F
from torch import Tensor, nn

from ..utils._structs import irreps_info
from .functional.dropout import irrep_wise_dropout


class Dropout(nn.Module):
    """Equivariant dropout on ``(N, irreps.dim, C)``: per (irrep, channel) when ``irrep_wise`` (needs ``irreps``),
    otherwise whole channels (``dropout1d`` on the transposed tensor).  ``work_on_eval`` keeps it active in
    evaluation mode."""

    def __init__(self, p: float = 0.5, irreps=None, irrep_wise: bool = True, work_on_eval: bool = False):
        super().__init__()
        if p < 0.0 or p > 1.0:
            raise ValueError(f"dropout probability has to be between 0 and 1, but got {p}")
        if irrep_wise and irreps is None:
            raise ValueError("irreps must be provided if irrep_wise is True")
        self.p, self.irrep_wise, self.work_on_eval = p, irrep_wise, work_on_eval
        self.irreps_info = irreps_info(irreps) if irrep_wise else None

    def forward(self, input: Tensor) -> Tensor:
        assert input.ndim >= 2, "Input tensor must have at least 2 dimensions (irreps_dim, channels)"
        active = self.training or self.work_on_eval
        if not active or self.p == 0.0:
            return input
        if self.irrep_wise:
            return irrep_wise_dropout(input, self.p, active, self.irreps_info)
        return F.dropout1d(input.transpose(-1, -2), self.p, active).transpose(-1, -2).contiguous()

    def extra_repr(self) -> str:
        return f"p={self.p}, irrep_wise={self.irrep_wise}, work_on_eval={self.work_on_eval}"

    def _apply(self, *args, **kwargs):
        mod = super()._apply(*args, **kwargs)
        if self.irreps_info is not None:
            mod.irreps_info = self.irreps_info._apply(*args, **kwargs)
        return mod
