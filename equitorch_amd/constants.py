"""Real-basis SO(3) Clebsch-Gordan coefficients in exact arithmetic (no computer-algebra dependency).

Same convention as ``equitorch/constants/__init__.py:40-105``: the complex (Condon-Shortley)
coefficients ``<j1 m1 j2 m2 | j3 m3>`` are rotated into the real basis with the unitary ``Q_l`` of
``_change_basis_real_to_complex`` (``:63-75``, including the global ``(-i)^l`` phase that makes the result
real), ``C[m, a, b] = sum_{n,i,k} conj(Q_l[n, m]) <l1 i l2 k | l n> Q_l1[i, a] Q_l2[k, b]``.

Every complex coefficient is ``sign * sqrt(rational)`` (Racah's closed form), and every entry of ``Q`` is a
fourth root of unity times ``1`` or ``1/sqrt(2)``, so each real-basis entry is a short signed sum of square
roots of rationals.  The sum is carried as ``{radicand: integer multiplicity}`` and evaluated once in
60-digit decimal arithmetic, which yields the correctly rounded double and an exact test for zero.
"""
from __future__ import annotations

import functools
from decimal import Decimal, localcontext
from fractions import Fraction
from math import factorial as _f
from typing import Dict, List, Tuple

import numpy as np


@functools.lru_cache(maxsize=None)
def _su2_cg(j1: int, m1: int, j2: int, m2: int, j3: int, m3: int) -> Tuple[int, Fraction]:
    """``<j1 m1 j2 m2 | j3 m3>`` for integer spins as ``(sign, radicand)`` with value ``sign*sqrt(radicand)``."""
    if m1 + m2 != m3 or not abs(j1 - j2) <= j3 <= j1 + j2:
        return 0, Fraction(0)
    if abs(m1) > j1 or abs(m2) > j2 or abs(m3) > j3:
        return 0, Fraction(0)
    pref = Fraction(
        (2 * j3 + 1) * _f(j3 + j1 - j2) * _f(j3 - j1 + j2) * _f(j1 + j2 - j3),
        _f(j1 + j2 + j3 + 1),
    ) * (_f(j3 + m3) * _f(j3 - m3) * _f(j1 - m1) * _f(j1 + m1) * _f(j2 - m2) * _f(j2 + m2))
    kmin = max(0, j2 - j3 - m1, j1 - j3 + m2)
    kmax = min(j1 + j2 - j3, j1 - m1, j2 + m2)
    s = Fraction(0)
    for k in range(kmin, kmax + 1):
        den = (_f(k) * _f(j1 + j2 - j3 - k) * _f(j1 - m1 - k) * _f(j2 + m2 - k)
               * _f(j3 - j2 + m1 + k) * _f(j3 - j1 - m2 + k))
        s += Fraction(-1 if k % 2 else 1, den)
    if s == 0:
        return 0, Fraction(0)
    return (1 if s > 0 else -1), s * s * pref


@functools.lru_cache(maxsize=None)
def _real_to_complex(l: int) -> Dict[Tuple[int, int], Tuple[int, int]]:
    """Non-zero entries of ``Q_l`` as ``{(row, col): (e, h)}`` meaning ``i**e * 2**(-h/2)``.

    Rows index the complex order ``m = row - l``; columns index the real component.
    """
    q: Dict[Tuple[int, int], Tuple[int, int]] = {}
    g = (3 * l) % 4  # (-i)^l = i^(3l)
    for m in range(-l, 0):
        q[(l + m, l - m)] = (g, 1)                  # 1/sqrt2
        q[(l + m, l + m)] = ((g + 3) % 4, 1)        # -i/sqrt2
    q[(l, l)] = (g, 0)
    for m in range(1, l + 1):
        q[(l + m, l + m)] = ((g + 2 * m) % 4, 1)      # (-1)^m/sqrt2
        q[(l + m, l - m)] = ((g + 1 + 2 * m) % 4, 1)  # i(-1)^m/sqrt2
    return q


def _eval_sqrt_sum(terms: Dict[Fraction, int]) -> float:
    terms = {r: c for r, c in terms.items() if c != 0}
    if not terms:
        return 0.0
    with localcontext() as ctx:
        ctx.prec = 60
        tot = Decimal(0)
        for r, c in terms.items():
            tot += c * (Decimal(r.numerator) / Decimal(r.denominator)).sqrt()
        if abs(tot) < Decimal("1e-40"):
            return 0.0
        return float(tot)


@functools.lru_cache(maxsize=None)
def so3_clebsch_gordan(l: int, l1: int, l2: int) -> np.ndarray:
    """Dense ``(2l+1, 2l1+1, 2l2+1)`` float64 array of real-basis coefficients coupling ``l1 x l2 -> l``.

    Normalisation is unitary: ``sum_{a,b} C[m,a,b] C[m',a,b] = delta_{mm'}`` (reference ``constants:40-61``).
    """
    ql, q1, q2 = _real_to_complex(l), _real_to_complex(l1), _real_to_complex(l2)
    cols_l: Dict[int, List[Tuple[int, int, int]]] = {}
    for (row, col), (e, h) in ql.items():
        cols_l.setdefault(col, []).append((row, (-e) % 4, h))  # conjugated
    cols_1: Dict[int, List[Tuple[int, int, int]]] = {}
    for (row, col), (e, h) in q1.items():
        cols_1.setdefault(col, []).append((row, e, h))
    cols_2: Dict[int, List[Tuple[int, int, int]]] = {}
    for (row, col), (e, h) in q2.items():
        cols_2.setdefault(col, []).append((row, e, h))

    out = np.zeros((2 * l + 1, 2 * l1 + 1, 2 * l2 + 1), dtype=np.float64)
    for m in range(2 * l + 1):
        for a in range(2 * l1 + 1):
            for b in range(2 * l2 + 1):
                re: Dict[Fraction, int] = {}
                im: Dict[Fraction, int] = {}
                for (n, e0, h0) in cols_l[m]:
                    for (i, e1, h1) in cols_1[a]:
                        for (k, e2, h2) in cols_2[b]:
                            sgn, rad = _su2_cg(l1, i - l1, l2, k - l2, l, n - l)
                            if sgn == 0:
                                continue
                            e = (e0 + e1 + e2) % 4
                            rad = rad / (1 << (h0 + h1 + h2))
                            if e >= 2:
                                sgn = -sgn
                            tgt = re if e % 2 == 0 else im
                            tgt[rad] = tgt.get(rad, 0) + sgn
                if _eval_sqrt_sum(im) != 0.0:
                    raise ArithmeticError(f"real-basis CG({l};{l1},{l2}) has an imaginary part")
                out[m, a, b] = _eval_sqrt_sum(re)
    out.setflags(write=False)
    return out


@functools.lru_cache(maxsize=None)
def j_matrix(l: int) -> np.ndarray:
    """Real-basis Wigner matrix of the rotation that exchanges the y and z axes and reverses x
    (``equitorch/constants/__init__.py:13-36``): ``J_1`` is written down, higher degrees follow from
    ``J_l = C(l; 1, l-1) (J_1 (x) J_{l-1}) C(l; 1, l-1)^T``.  With it every rotation is
    ``D(alpha, beta, gamma) = Z(alpha) J Z(beta) J Z(gamma)`` where ``Z`` mixes only the ``+-m`` pairs."""
    if l == 0:
        return np.ones((1, 1))
    if l == 1:
        return np.array([[0.0, 1.0, 0.0], [1.0, 0.0, 0.0], [0.0, 0.0, -1.0]])
    cg = so3_clebsch_gordan(l, 1, l - 1)
    return np.einsum("iI,jJ,kij,KIJ->kK", j_matrix(1), j_matrix(l - 1), cg, cg)
