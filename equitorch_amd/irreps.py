"""O(3) / SO(3) irreducible-representation bookkeeping used by the tensor-product table builders.

Mirrors the public surface of ``equitorch/irreps/__init__.py`` that the sparse
Clebsch-Gordan path touches (``Irrep``, ``Irreps``, ``check_irreps``, ``has_path``,
``irrep_segments`` and the index helpers ``unique_irreps``, ``irrep_indices``, ``irrep_degrees``,
``element_degrees``, ``element_orders``; reference lines 12-158, 161-238, 240-338, 558-717, 841-974).

Conventions kept from the reference: a feature tensor is ``(batch, irreps.dim, channels)``
and the multiplicity of an ``Irreps`` entry is *not* the channel count; parity is stored as
``+1`` ('e'), ``-1`` ('o') or ``0`` (no parity, SO(3) only).
"""
from __future__ import annotations

import math
import re
from typing import Iterator, List, Sequence, Tuple, Union

_PARITY = {"e": 1, "o": -1, 1: 1, -1: -1, 0: 0, None: 0}
p_mapping = _PARITY   # the reference's public name (``:8-10``)
_TERM = re.compile(r"(?:(\d+)x)?(\d+)([eo]?)")


class Irrep:
    """One irreducible representation ``(l, p)``; ``Irrep(2, 'e')``, ``Irrep('3o')``, ``Irrep(1)``,
    ``Irrep((2, -1))`` are all accepted (reference ``irreps/__init__.py:12-96``)."""

    __slots__ = ("l", "p")

    def __init__(self, *args):
        if len(args) == 1:
            a = args[0]
            if isinstance(a, Irrep):
                l, p = a.l, a.p
            elif isinstance(a, str):
                m = _TERM.fullmatch(a.strip())
                if m is None or m.group(1) is not None:
                    raise ValueError(f"cannot parse irrep {a!r}")
                l, p = int(m.group(2)), (m.group(3) or None)
            elif isinstance(a, int):
                l, p = a, None
            elif isinstance(a, tuple):
                l, p = a
            else:
                raise TypeError("Invalid argument type")
        elif len(args) == 2:
            l, p = args
            if not isinstance(l, int) or p is None:
                raise TypeError("Cannot pass both string and (l, p) initialization")
        elif len(args) == 0:
            raise TypeError("Irrep requires at least one argument")
        else:
            raise TypeError("Irrep accepts at most two arguments")
        if p not in _PARITY:
            raise ValueError("p must be +1 ('e'), -1 ('o'), or 0 (None)")
        if not isinstance(l, int) or l < 0:
            raise ValueError("l must be a non-negative integer")
        self.l = l
        self.p = _PARITY[p]

    def __iter__(self):
        yield self.l
        yield self.p

    def __repr__(self):
        return f"{self.l}{'' if self.p == 0 else ('e' if self.p > 0 else 'o')}"

    def __eq__(self, other):
        if isinstance(other, str):
            return repr(self) == other
        if isinstance(other, int):
            return self.p == 0 and self.l == other
        if isinstance(other, (Irrep, tuple)):
            l, p = other
            return self.l == int(l) and self.p == _PARITY[p]
        return False

    def __hash__(self):
        return hash((self.l, self.p))

    @property
    def dim(self) -> int:
        return 2 * self.l + 1

    def __mul__(self, other: "Irrep") -> "Irreps":
        if not isinstance(other, Irrep):
            raise TypeError(f"Can only multiply Irrep with Irrep, got {type(other)}")
        p = self.p * other.p
        return Irreps([Irrep(l, p) for l in range(abs(self.l - other.l), self.l + other.l + 1)])


def parse_irreps(text: str) -> List[Tuple[Irrep, int]]:
    """``'6x0+1+2e+5x2o'`` -> ``[(0, 6), (1, 1), (2e, 1), (2o, 5)]`` (reference ``:161-207``)."""
    groups = []
    for term in text.replace(" ", "").split("+"):
        if not term:
            continue
        m = _TERM.fullmatch(term)
        if m is None:
            raise ValueError(f"Invalid term: {term}")
        mul = 1 if m.group(1) is None else int(m.group(1))
        if mul < 1:
            raise ValueError(f"Multiplicity must be ≥1 in '{term}'")
        groups.append((Irrep(m.group(2) + m.group(3)), mul))
    return groups


def show_irreps(groups: Sequence[Tuple[Irrep, int]]) -> str:
    return "+".join((f"{mul}x{ir}" if mul != 1 else f"{ir}") for ir, mul in groups)


class Irreps:
    """Ordered list of ``(Irrep, multiplicity)`` groups (reference ``:240-338``).

    Iteration, indexing and ``len`` run over the multiplicity-expanded sequence.
    """

    def __init__(self, irreps: Union[str, tuple, list, Irrep, "Irreps"]):
        if isinstance(irreps, str):
            groups = parse_irreps(irreps)
        elif isinstance(irreps, Irreps):
            groups = list(irreps.irrep_groups)
        elif isinstance(irreps, Irrep):
            groups = [(irreps, 1)]
        elif isinstance(irreps, tuple):
            if len(irreps) == 2 and all(isinstance(v, int) for v in irreps):
                groups = [(Irrep(l), 1) for l in range(irreps[0], irreps[1] + 1)]
            elif len(irreps) == 2 and isinstance(irreps[0], Irrep) and isinstance(irreps[1], int):
                groups = [irreps]
            else:
                raise ValueError("Invalid tuple format. Expected two integers for range.")
        elif isinstance(irreps, list):
            groups = []
            for item in irreps:
                if isinstance(item, Irrep):
                    groups.append((item, 1))
                elif isinstance(item, tuple) and isinstance(item[0], Irrep):
                    groups.append((item[0], item[1]))
                else:
                    groups.append((Irrep(item), 1))
        else:
            raise TypeError(f"Invalid type for irrep_groups: {type(irreps)}")
        self.irrep_groups: List[Tuple[Irrep, int]] = groups

    # -- constructors -------------------------------------------------------------------
    @staticmethod
    def spherical_harmonics(max_degree: int, parity_even_degree="e") -> "Irreps":
        """``0e+1o+2e+...`` (or the opposite assignment for ``'o'``); reference ``:262-284``."""
        if parity_even_degree not in ("e", "o"):
            raise ValueError("parity_even_degree must be 'e' or 'o'")
        other = "o" if parity_even_degree == "e" else "e"
        return Irreps([f"{l}{parity_even_degree if l % 2 == 0 else other}" for l in range(max_degree + 1)])

    @staticmethod
    def both_parities(max_degree: int, min_degree: int = 0) -> "Irreps":
        return Irreps("+".join(f"{l}e+{l}o" for l in range(min_degree, max_degree + 1)))

    # -- container protocol ---------------------------------------------------------------
    def __iter__(self) -> Iterator[Irrep]:
        for ir, mul in self.irrep_groups:
            for _ in range(mul):
                yield ir

    def __len__(self) -> int:
        return sum(mul for _, mul in self.irrep_groups)

    def __getitem__(self, index):
        flat = list(self)
        if isinstance(index, int):
            if not -len(flat) <= index < len(flat):
                raise IndexError("Irrep index out of range")
            return flat[index]
        if isinstance(index, slice):
            if index.indices(len(flat))[2] != 1:
                raise ValueError("Irreps slicing only supports a step of 1")
            return Irreps(flat[index])
        raise TypeError(f"Irreps indices must be integers or slices, not {type(index).__name__}")

    def __repr__(self):
        return f"Irreps({self.short_repr()})"

    def short_repr(self) -> str:
        return show_irreps(self.irrep_groups)

    def __eq__(self, other):
        if other is None:
            return False
        return self.irrep_groups == check_irreps(other).irrep_groups

    def __hash__(self):
        return hash(self.short_repr())

    # -- sizes --------------------------------------------------------------------------
    @property
    def dim(self) -> int:
        return sum(ir.dim * mul for ir, mul in self.irrep_groups)

    @property
    def l_max(self) -> int:
        return max(ir.l for ir, _ in self.irrep_groups)

    def dims(self):
        for ir in self:
            yield ir.dim

    # -- algebra ------------------------------------------------------------------------
    def __add__(self, other):
        return Irreps(self.irrep_groups + check_irreps(other).irrep_groups)

    def __radd__(self, other):
        return Irreps(check_irreps(other).irrep_groups + self.irrep_groups)

    def sorted(self, by=None) -> "Irreps":
        if by is None:
            # degree first, then no-parity < even < odd, then multiplicity
            def by(g):
                return (g[0].l, {0: 0, 1: 1, -1: 2}[g[0].p], g[1])
        return Irreps(sorted(self.irrep_groups, key=by))

    def merged(self) -> "Irreps":
        out: List[Tuple[Irrep, int]] = []
        for ir, mul in self.irrep_groups:
            if out and out[-1][0] == ir:
                out[-1] = (ir, out[-1][1] + mul)
            else:
                out.append((ir, mul))
        return Irreps(out)

    def simplified(self) -> "Irreps":
        totals = {}
        for ir, mul in self.irrep_groups:
            totals[ir] = totals.get(ir, 0) + mul
        return Irreps(list(totals.items())).sorted()

    def eliminate_parity(self, simplified: bool = False) -> "Irreps":
        out = Irreps([(Irrep(ir.l, 0), mul) for ir, mul in self.irrep_groups])
        return out.simplified() if simplified else out

    def __mul__(self, other) -> "Irreps":
        other = check_irreps(other)
        groups = [
            (ir, m1 * m2)
            for ir1, m1 in self.irrep_groups
            for ir2, m2 in other.irrep_groups
            for ir in ir1 * ir2
        ]
        return Irreps(groups).simplified()

    def isomorphic_to(self, other) -> bool:
        return self.simplified() == check_irreps(other).simplified()

    def channels_divided(self, mul: int) -> "Irreps":
        assert all(m % mul == 0 for _, m in self.irrep_groups), (
            f"All multiplicities must be divisible by {mul}, but got {self.irrep_groups}")
        return Irreps([(ir, m // mul) for ir, m in self.irrep_groups])

    def channels_multiplied(self, mul: int) -> "Irreps":
        return Irreps([(ir, m * mul) for ir, m in self.irrep_groups])

    def max_channels(self) -> int:
        return math.gcd(*(m for _, m in self.irrep_groups))

    def squeeze_max_channels(self):
        g = self.max_channels()
        return self.channels_divided(g), g


def check_irreps(irreps) -> Irreps:
    return irreps if isinstance(irreps, Irreps) else Irreps(irreps)


def has_path(irrep_out: Irrep, irrep_1: Irrep, irrep_2: Irrep = None) -> bool:
    """Selection rule of a coupling path (reference ``:220-238``): triangle inequality on the degrees
    and, unless the output carries no parity, ``p1 * p2 == p_out``."""
    if irrep_2 is None:
        return irrep_out.l == irrep_1.l and (irrep_out.p == 0 or irrep_1.p == irrep_out.p)
    triangle = abs(irrep_1.l - irrep_2.l) <= irrep_out.l <= irrep_1.l + irrep_2.l
    return triangle and (irrep_out.p == 0 or irrep_1.p * irrep_2.p == irrep_out.p)


def irrep_segments(irreps) -> List[int]:
    """Start offset of every (expanded) irrep block plus the total dim (reference ``:889-921``)."""
    seg = [0]
    for ir in check_irreps(irreps):
        seg.append(seg[-1] + ir.dim)
    return seg


def unique_irreps(irreps):
    """``(Irreps of the distinct irreps in order of first appearance, {irrep: positions in the expanded sequence})``
    (reference ``:841-887``): ``unique_irreps("0+0e+1o+0e+0e") -> (Irreps(0+0e+1o), {0: [0], 0e: [1, 3, 4], 1o: [2]})``."""
    positions = {}
    for i, ir in enumerate(check_irreps(irreps)):
        positions.setdefault(ir, []).append(i)
    return Irreps(list(positions)), positions


def _long_tensor(values):
    import torch   # only these helpers return tensors; the rest of the module is torch-free
    return torch.tensor(values, dtype=torch.long)


def irrep_indices(irreps):
    """For every component of the feature, the position of its irrep in the expanded sequence
    (reference ``:923-952``): ``"0+2x1e+2e" -> [0, 1, 1, 1, 2, 2, 2, 3, 3, 3, 3, 3]``."""
    return _long_tensor([i for i, ir in enumerate(check_irreps(irreps)) for _ in range(ir.dim)])


def irrep_degrees(irreps):
    """Degree ``l`` of every irrep of the expanded sequence (reference ``:954-959``)."""
    return _long_tensor([ir.l for ir in check_irreps(irreps)])


def element_degrees(irreps):
    """Degree ``l`` of every component (reference ``:961-966``)."""
    return _long_tensor([ir.l for ir in check_irreps(irreps) for _ in range(ir.dim)])


def element_orders(irreps):
    """Order ``m = -l .. l`` of every component (reference ``:968-974``)."""
    return _long_tensor([m for ir in check_irreps(irreps) for m in range(-ir.l, ir.l + 1)])
