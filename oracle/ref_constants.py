"""TEST INFRASTRUCTURE ONLY: the reference's symbolic real-basis Clebsch-Gordan construction.

Follows ``equitorch/constants/__init__.py``:
  * ``su2_cg``            <- ``_su2_clebsch_gordan`` (:77-105), entries from ``sympy.physics.wigner.clebsch_gordan``
  * ``real_to_complex``   <- ``_change_basis_real_to_complex`` (:63-75)
  * ``so3_cg``            <- ``so3_clebsch_gordan`` (:40-61), contraction ``"mn,nik,ij,kl->mjl"``

Pinned by: golden fixtures ``tests/golden/tp_tables_*.npz`` (coefficients as stored by the reference's
``tp_infos``), unitarity, the l2=0 identity, the 1x1->0 dot product, the 1x1->1 cross product and the
exchange symmetry (tests/test_cg.py).
"""
import functools

import sympy
from sympy import S
from sympy.physics.wigner import clebsch_gordan


@functools.lru_cache(maxsize=None)
def su2_cg(j3, j1, j2):
    rows = []
    for n in range(2 * j3 + 1):
        rows.append([[clebsch_gordan(j1, j2, j3, S(i - j1), S(k - j2), S(n - j3))
                      if (i - j1) + (k - j2) == n - j3 else S(0)
                      for k in range(2 * j2 + 1)] for i in range(2 * j1 + 1)])
    return rows


@functools.lru_cache(maxsize=None)
def real_to_complex(l):
    r = sympy.sqrt(2) / 2
    q = [[S(0)] * (2 * l + 1) for _ in range(2 * l + 1)]
    for m in range(-l, 0):
        q[l + m][l - m] = r
        q[l + m][l + m] = -sympy.I * r
    q[l][l] = S(1)
    for m in range(1, l + 1):
        q[l + m][l + m] = (-1) ** m * r
        q[l + m][l - m] = sympy.I * (-1) ** m * r
    ph = (-sympy.I) ** l
    return [[ph * v for v in row] for row in q]


@functools.lru_cache(maxsize=None)
def so3_cg(l, l1, l2):
    """Exact symbolic ``C[m][j][l']``; ``float()`` of an entry is what the table builder consumes."""
    q, q1, q2 = real_to_complex(l), real_to_complex(l1), real_to_complex(l2)
    c = su2_cg(l, l1, l2)
    out = [[[S(0)] * (2 * l2 + 1) for _ in range(2 * l1 + 1)] for _ in range(2 * l + 1)]
    for m in range(2 * l + 1):
        for j in range(2 * l1 + 1):
            for lp in range(2 * l2 + 1):
                acc = S(0)
                for n in range(2 * l + 1):
                    qt = sympy.conjugate(q[n][m])
                    if qt == 0:
                        continue
                    for i in range(2 * l1 + 1):
                        if q1[i][j] == 0:
                            continue
                        for k in range(2 * l2 + 1):
                            if q2[k][lp] == 0 or c[n][i][k] == 0:
                                continue
                            acc = acc + qt * c[n][i][k] * q1[i][j] * q2[k][lp]
                out[m][j][lp] = sympy.sympify(acc)
    return out


@functools.lru_cache(maxsize=None)
def j_matrix(l):
    """``j_matrix`` (equitorch/constants/__init__.py:13-36) in exact arithmetic: nested lists of sympy numbers.
    Pinned by the golden fixture ``tests/golden/rotation_tables.npz`` (entries as stored by the reference's
    ``j_matrix_info``), by ``J^2 = 1`` and by ``Y(J v) = J Y(v)`` for ``J v = (-x, z, y)``."""
    if l == 0:
        return [[S(1)]]
    if l == 1:
        return [[S(0), S(1), S(0)], [S(1), S(0), S(0)], [S(0), S(0), S(-1)]]
    cg, j1, jp = so3_cg(l, 1, l - 1), j_matrix(1), j_matrix(l - 1)
    n, n1 = 2 * l + 1, 2 * l - 1
    # 'iI,jJ,kij,KIJ->kK'
    half = [[[sum(j1[i][I] * jp[j][J] * cg[k][i][j] for i in range(3) for j in range(n1))
              for J in range(n1)] for I in range(3)] for k in range(n)]
    return [[sympy.nsimplify(sum(half[k][I][J] * cg[K][I][J] for I in range(3) for J in range(n1)))
             for K in range(n)] for k in range(n)]
