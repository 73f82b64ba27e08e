"""Structural helpers (``equitorch/nn/others.py``): splitting a feature tensor by groups of irreps and applying one
module per group."""
from typing import Iterable, List, Union

import torch
from torch import Tensor, nn

from ..irreps import Irreps, check_irreps


class SplitIrreps(nn.Module):
    """Splits along ``dim`` into consecutive groups of ``split_num_irreps`` irreps each; one entry may be ``-1`` or
    ``...`` and takes the rest.  ``irreps_out`` lists the (merged) irreps of every part."""

    def __init__(self, irreps, split_num_irreps: Iterable[int], dim: int = -2):
        super().__init__()
        self.irreps = check_irreps(irreps)
        self.dim = dim
        counts = list(split_num_irreps)
        rest = [i for i, c in enumerate(counts) if c in (-1, ...)]
        if len(rest) > 1:
            raise ValueError("split_num_irreps can contain at most one -1 or ...")
        if rest:
            counts[rest[0]] = len(self.irreps) - sum(c for c in counts if c not in (-1, ...))
        if sum(counts) != len(self.irreps):
            raise ValueError(f"Sum of split_num_irreps ({sum(counts)}) must equal to the number of total irreps "
                             f"({len(self.irreps)})")
        self.split_num_irreps = counts
        self.input_dim = self.irreps.dim
        self.split_sizes, self.irreps_out, at = [], [], 0
        for num in counts:
            part = [self.irreps[at + i] for i in range(num)]
            self.split_sizes.append(sum(ir.dim for ir in part))
            self.irreps_out.append(Irreps(part).merged())
            at += num

    def forward(self, x: Tensor) -> List[Tensor]:
        if x.shape[self.dim] != self.input_dim:
            raise ValueError(f"Input tensor dimension {x.shape[self.dim]} does not match expected irreps dimension "
                             f"{self.input_dim}")
        return torch.split(x, self.split_sizes, dim=self.dim)

    def __repr__(self):
        parts = ", ".join(ir.short_repr() for ir in self.irreps_out)
        return f"{self.__class__.__name__}(irreps_in={self.irreps.short_repr()}, irreps_out=[{parts}])"


class Separable(nn.Module):
    """Applies ``sub_modules[i]`` (or nothing, if ``None``) to the i-th part of :class:`SplitIrreps` and concatenates
    the results along ``dim`` (returns the list instead when ``cat_after`` is false)."""

    def __init__(self, irreps, split_num_irreps: Iterable[int], sub_modules: Iterable[nn.Module],
                 cat_after: bool = True, dim: int = -2):
        super().__init__()
        self.irreps = check_irreps(irreps)
        self.dim = dim
        split_num_irreps, sub_modules = list(split_num_irreps), list(sub_modules)
        self.split = SplitIrreps(self.irreps, split_num_irreps, dim=dim)
        self.cat_after = cat_after
        if len(split_num_irreps) != len(sub_modules):
            raise ValueError(f"Length of split_num_irreps ({len(split_num_irreps)}) must match length of "
                             f"sub_modules ({len(sub_modules)})")
        self.sub_modules = nn.ModuleList(sub_modules)

    def forward(self, x: Tensor) -> Union[Tensor, List[Tensor]]:
        if x.shape[self.dim] != self.split.input_dim:
            raise RuntimeError(f"Input dimension ({x.shape[self.dim]}) must match irreps dimension "
                               f"({self.split.input_dim})")
        parts = [m(part) if m is not None else part for m, part in zip(self.sub_modules, self.split(x))]
        return torch.cat(parts, dim=self.dim) if self.cat_after else parts

    def __repr__(self):
        parts = ", ".join(ir.short_repr() for ir in self.split.irreps_out)
        mods = ", ".join(str(m) if m is not None else "None" for m in self.sub_modules)
        return (f"{self.__class__.__name__}(irreps_in={self.irreps.short_repr()}, irreps_out=[{parts}], "
                f"sub_modules=[{mods}], cat_after={self.cat_after})")
