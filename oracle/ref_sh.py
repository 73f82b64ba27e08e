"""TEST INFRASTRUCTURE ONLY: real spherical harmonics as the reference defines them.

``equitorch/ops/spherical_harmonics.py:68-640`` evaluates, degree by degree, polynomials of the form
``sh_l_m = sum coef * sh_{l-1}_{m'} * {x, y, z}`` that its generator (commented out at ``:5-66``) obtained as
``Y_l = N_l * C(l; l-1, 1) . (Y_{l-1} (x) Y_1)`` with ``Y_0 = 1``, ``Y_1 = sqrt(3) (y, z, x)`` and ``N_l`` fixed by the
value at the north pole, ``|Y_l(0, 0, 1)| = sqrt(2l+1)``.  ``spherical_harmonics`` below restates that recursion
in float64 torch (differentiable, so autograd provides the gradient oracle) on the real-basis Clebsch-Gordan
coefficients of ``ref_constants.so3_cg``; the sign of ``N_l`` is the one the polynomial text shows: the
coefficient of ``sh_{l-1}_{l-1} * z`` in ``sh_l_l`` is positive for every ``l <= 17``, i.e.
``Y_{l,0}(0, 0, 1) = +sqrt(2l+1)``.  Like the polynomials, the result is homogeneous of degree ``l`` in the input.

``closed_form`` is an independent statement of the same functions from textbook formulas (associated Legendre
functions from ``scipy.special.lpmv`` without the Condon-Shortley phase, ``cos m phi`` for ``m > 0``, ``sin |m| phi``
for ``m < 0``, 4-pi normalisation); unit vectors only.

Pinned by (tests/test_sh.py): ``closed_form`` for every ``(l, m)`` up to degree 10; the hand-expanded polynomials
of degrees 0..3 (``sqrt(15) x y``, ``sqrt(5)/2 (2 z^2 - x^2 - y^2)``, ``sqrt(70)/4 ... (3 x^2 y - y^3)`` ...) as they
follow from ``:80-114``; ``Y_{l,+-l} = sqrt((2l+1)/(2l)) (x Y_{l-1,+-(l-1)} -+ y Y_{l-1,-+(l-1)})`` (``sh_l_0`` and
``sh_l_{2l}`` lines of every degree); ``|Y_l|^2 = 2l+1``; the addition theorem
``sum_m Y_lm(a) Y_lm(b) = (2l+1) P_l(a . b)``; homogeneity.
"""
import functools
import math

import numpy as np
import torch

from . import ref_constants


@functools.lru_cache(maxsize=None)
def _coupling(l: int) -> torch.Tensor:
    """C(l; l-1, 1) as a (2l+1, 2l-1, 3) float64 tensor."""
    c = ref_constants.so3_cg(l, l - 1, 1)
    return torch.tensor(np.array(c, dtype=np.float64).reshape(2 * l + 1, 2 * l - 1, 3))


@functools.lru_cache(maxsize=None)
def _norm(l: int) -> float:
    """N_l: makes Y_{l,0}(north pole) = +sqrt(2l+1)."""
    pole = torch.tensor([[0.0, 0.0, 1.0]], dtype=torch.float64)
    raw = _blocks(pole, l, normalised_last=False)[-1][0]
    assert abs(abs(float(raw[l])) - float(raw.norm())) < 1e-12   # only m = 0 survives at the pole
    return math.sqrt(2 * l + 1) / float(raw[l])


def _blocks(v: torch.Tensor, l_max: int, normalised_last: bool = True):
    y1 = math.sqrt(3.0) * v[:, [1, 2, 0]]
    blocks = [torch.ones(v.shape[0], 1, dtype=v.dtype)]
    if l_max >= 1:
        blocks.append(y1)
    for l in range(2, l_max + 1):
        raw = torch.einsum("mab,na,nb->nm", _coupling(l).to(v.dtype), blocks[-1], y1)
        blocks.append(raw if (l == l_max and not normalised_last) else _norm(l) * raw)
    return blocks


def spherical_harmonics(xyz: torch.Tensor, l_max: int) -> torch.Tensor:
    """``(n, 3)`` float64 -> ``(n, (l_max+1)^2)``, index ``l^2 + l + m``; no normalisation of the input."""
    return torch.cat(_blocks(xyz, l_max), dim=-1)


def normalize(xyz: torch.Tensor, eps: float = 1e-12) -> torch.Tensor:
    """``torch.nn.functional.normalize(xyz, dim=-1)`` as ``SphericalHarmonics.forward`` applies it
    (``equitorch/nn/sphericals.py:31-33``)."""
    return xyz / xyz.norm(dim=-1, keepdim=True).clamp_min(eps)


def closed_form(unit: np.ndarray, l_max: int) -> np.ndarray:
    """Textbook real harmonics of unit vectors ``(n, 3)`` (float64 numpy), same layout and normalisation."""
    from scipy.special import lpmv
    x, y, z = unit[:, 0], unit[:, 1], unit[:, 2]
    phi = np.arctan2(y, x)
    out = np.zeros((unit.shape[0], (l_max + 1) ** 2))
    for l in range(l_max + 1):
        for m in range(0, l + 1):
            k = math.sqrt((2 * l + 1) * math.factorial(l - m) / math.factorial(l + m))
            p = (-1) ** m * lpmv(m, l, z)            # lpmv carries the Condon-Shortley phase; remove it
            if m == 0:
                out[:, l * l + l] = k * p
            else:
                out[:, l * l + l + m] = math.sqrt(2.0) * k * p * np.cos(m * phi)
                out[:, l * l + l - m] = math.sqrt(2.0) * k * p * np.sin(m * phi)
    return out
