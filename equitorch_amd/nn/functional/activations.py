"""``gating`` (``equitorch/nn/functional/activations.py:9-35``): every irrep block of the input scaled by its gate."""
from torch import Tensor

from ...structs import IrrepsInfo, SparseProductInfo
from .sparse_product import sparse_mul


def _broadcast_infos(irreps_info: IrrepsInfo):
    """Tables of ``z[n, M, c] = x[n, M, c] * s[(n,) irrep(M), c]`` and of its two gradients."""
    return (SparseProductInfo(index2=irreps_info.irrep_index), SparseProductInfo(index1=irreps_info.irrep_index),
            SparseProductInfo(seg_out=irreps_info.irrep_seg))


def gating(input: Tensor, gates: Tensor, irreps_info: IrrepsInfo) -> Tensor:
    """``out[n, M, c] = input[n, M, c] * gates[(n,) irrep_of(M), c]``; ``gates`` is ``(num_irreps, C)`` or
    ``(N, num_irreps, C)``.  One launch of the table-driven product kernel."""
    return sparse_mul(input, gates, *_broadcast_infos(irreps_info))
