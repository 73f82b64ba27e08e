"""``SO2Linear('uv')`` with a shared weight as one library GEMM per order ``|m|``.

The table of the layer (``so2_linear_infos``, reference ``equitorch/utils/_structs.py:673-786``) couples an output
component only with input components of the same ``|m|``: ``m = 0`` components through one weight per (output irrep,
input irrep), the ``(+m, -m)`` pairs through a ``(w_+, w_-)`` pair acting like a complex number.  The components
therefore fall into blocks (the connected components of the table's input-output graph, found from the table
itself), and inside a block the layer is a dense matrix

    out[n, (M, w)] = sum_(M0, u) x[n, (M0, u)] * B[(M0, u), (M, w)],      B[(M0, :), (M, :)] = scale_t * W[p_t]

for the one table entry ``t`` that links ``M0`` with ``M``.  ``B`` is assembled from the weight list by a small
matrix product with a constant 0 / scale matrix, the rows of a block are gathered side by side, and the block is
one GEMM with ``K = n_in * C_in`` and ``N = n_out * C_out`` instead of ``n_in * n_out`` GEMMs with ``K = C_in`` on
strided rows.  Everything is differentiable tensor algebra, so gradients of any order come from autograd.
The reference runs the layer on its table-driven vector-matrix kernel (``sparse_vecmat``).
"""
from typing import NamedTuple

import torch
from torch import Tensor

from ...ops.kernels import cached


class _Block(NamedTuple):
    rows_in: Tensor       # (n_in,) input components of the block
    rows_out: Tensor      # (n_out,) output components
    assemble: Tensor      # (n_in * n_out, P): entry [(i, o), p] = scale of the table entry in -> out through weight p


def _entries(info, in_size: int):
    n = next((t.shape[0] for t in (info.index1, info.index2, info.scale) if t is not None), None)
    if n is None:
        n = int(info.seg_out[-1]) if info.seg_out is not None else in_size
    i1 = list(range(n)) if info.index1 is None else info.index1.tolist()
    i2 = list(range(n)) if info.index2 is None else info.index2.tolist()
    sc = [1.0] * n if info.scale is None else info.scale.tolist()
    if info.seg_out is None:
        out_of, n_out = list(range(n)), n
    else:
        seg = info.seg_out.tolist()
        n_out = len(seg) - 1
        out_of = [m for m in range(n_out) for _ in range(seg[m], seg[m + 1])]
    if info.out_size is not None:
        n_out = max(n_out, int(info.out_size))
    return list(zip(out_of, i1, i2, sc)), n_out


def _blocks(info, in_size: int, n_weights: int, device, dtype):
    anchor = next(t for t in (info.seg_out, info.index1, info.index2, info.scale) if t is not None)

    def build():
        entries, n_out = _entries(info, in_size)
        # union-find over input nodes ('i', M0) and output nodes ('o', M)
        parent = {}

        def find(a):
            parent.setdefault(a, a)
            while parent[a] != a:
                parent[a] = parent[parent[a]]
                a = parent[a]
            return a

        for m, m0, _, _ in entries:
            parent[find(("o", m))] = find(("i", m0))
        groups = {}
        for m, m0, p, s in entries:
            groups.setdefault(find(("i", m0)), []).append((m, m0, p, s))
        blocks = []
        for ents in groups.values():
            rin = sorted({m0 for _, m0, _, _ in ents})
            rout = sorted({m for m, _, _, _ in ents})
            asm = torch.zeros(len(rin) * len(rout), n_weights, dtype=torch.float64)
            for m, m0, p, s in ents:
                asm[rin.index(m0) * len(rout) + rout.index(m), p] += s
            blocks.append(_Block(torch.tensor(rin, dtype=torch.int64, device=device),
                                 torch.tensor(rout, dtype=torch.int64, device=device),
                                 asm.to(device=device, dtype=dtype)))
        blocks.sort(key=lambda b: int(b.rows_out[0]))
        order = torch.cat([b.rows_out for b in blocks]) if blocks else torch.zeros(0, dtype=torch.int64, device=device)
        # where every output component sits in the concatenation of the blocks' results (all covered), or None
        inverse = torch.argsort(order) if order.shape[0] == n_out else None
        return blocks, n_out, order, inverse
    return cached(anchor, ("so2_blocks", in_size, n_weights, str(device), dtype), build)


def so2_linear_uv_shared(input: Tensor, weight: Tensor, info, in_size: int, n_weights: int) -> Tensor:
    """``input (..., D_in, C_in)``, ``weight (P, C_in, C_out)`` -> ``(..., D_out, C_out)``."""
    lead = input.shape[:-2]
    x = input.reshape(-1, *input.shape[-2:])
    n, _, cin = x.shape
    cout = weight.shape[-1]
    blocks, n_out, order, inverse = _blocks(info, in_size, n_weights, x.device, weight.dtype)
    flat_w = weight.reshape(n_weights, cin * cout)
    pieces = []
    for blk in blocks:
        n_in, n_o = blk.rows_in.shape[0], blk.rows_out.shape[0]
        mat = (blk.assemble @ flat_w).view(n_in, n_o, cin, cout).permute(0, 2, 1, 3).reshape(n_in * cin, n_o * cout)
        xb = x.index_select(1, blk.rows_in).reshape(n, n_in * cin)
        pieces.append((xb @ mat).view(n, n_o, cout))
    if not pieces:
        return x.new_zeros(*lead, n_out, cout)
    stacked = torch.cat(pieces, dim=1)
    if inverse is not None:
        out = stacked.index_select(1, inverse)
    else:                                  # output components no entry reaches stay zero
        out = x.new_zeros(n, n_out, cout).index_copy(1, order, stacked)
    return out.reshape(*lead, n_out, cout)
