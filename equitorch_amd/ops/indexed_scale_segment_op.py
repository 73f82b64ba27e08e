"""``indexed_scale_segment`` (``equitorch/ops/indexed_scale_segment_op.py:110-181``) on the HIP kernel."""
from torch import Tensor

from . import kernels


def indexed_scale_segment(input: Tensor, scale, index, seg, out_size=None, out=None,
                          block_size_n=64, block_size_c=64) -> Tensor:
    r"""``out[n, m, c] = sum_{t in [seg[m], seg[m+1])} scale[t] * input[n, index[t], c]``.

    ``input`` is ``(N, in_size, C)``; ``scale`` / ``index`` / ``seg`` may each be ``None`` (no scaling /
    identity gather / one term per output row, in which case ``out_size`` gives the number of rows).
    ``block_size_*`` are accepted for signature compatibility and ignored.
    """
    if seg is not None:
        n_seg = seg.shape[0] - 1
    elif out_size is not None:
        n_seg = out_size
    else:
        n_seg = index.shape[0] if index is not None else input.shape[1]
    out_size = out_size or n_seg
    res = kernels.segment_sum(input, scale, index, seg, out_size)
    if out is not None:
        out.copy_(res)
        return out
    return res
