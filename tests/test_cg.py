"""Real-basis Clebsch-Gordan coefficients: the product's exact-arithmetic implementation and the oracle's
symbolic one, against each other and against what the mathematics fixes."""
import itertools

import numpy as np
import pytest

from equitorch_amd.constants import so3_clebsch_gordan
from oracle import ref_constants

TRIPLES = [(l, l1, l2) for l, l1, l2 in itertools.product(range(4), repeat=3) if abs(l1 - l2) <= l <= l1 + l2]


def _oracle(l, l1, l2):
    return np.array([[[float(v) for v in r] for r in m] for m in ref_constants.so3_cg(l, l1, l2)])


@pytest.mark.parametrize("l,l1,l2", TRIPLES + [(4, 2, 2), (5, 3, 2), (6, 3, 3), (2, 4, 6)])
def test_product_matches_symbolic_oracle(l, l1, l2):
    a, b = so3_clebsch_gordan(l, l1, l2), _oracle(l, l1, l2)
    assert a.shape == (2 * l + 1, 2 * l1 + 1, 2 * l2 + 1)
    assert np.array_equal(a != 0, b != 0), "sparsity pattern"
    assert np.abs(a - b).max() <= 2.3e-16, "more than one ulp apart"
    assert np.array_equal(a.astype(np.float32), b.astype(np.float32)), "fp32 bits"


@pytest.mark.parametrize("impl", [so3_clebsch_gordan, _oracle])
@pytest.mark.parametrize("l,l1,l2", TRIPLES + [(4, 2, 3), (6, 6, 6)])
def test_unitarity(impl, l, l1, l2):
    if impl is _oracle and l1 + l2 + l > 12:
        pytest.skip("symbolic evaluation too slow")
    c = impl(l, l1, l2).reshape(2 * l + 1, -1)
    np.testing.assert_allclose(c @ c.T, np.eye(2 * l + 1), atol=1e-14)


@pytest.mark.parametrize("impl", [so3_clebsch_gordan, _oracle])
def test_special_cases(impl):
    for l in range(4):
        # l x 0 -> l is the identity; l x l -> 0 is the normalised dot product
        np.testing.assert_allclose(impl(l, l, 0)[:, :, 0], np.eye(2 * l + 1), atol=1e-15)
        np.testing.assert_allclose(impl(0, l, l)[0], np.eye(2 * l + 1) / np.sqrt(2 * l + 1), atol=1e-15)
    # 1 x 1 -> 1 is the cross product / sqrt(2) on components ordered (y, z, x)
    c = impl(1, 1, 1)
    rng = np.random.default_rng(0)
    a, b = rng.normal(size=3), rng.normal(size=3)          # (x, y, z)
    to_yzx = [1, 2, 0]
    got = np.einsum("mab,a,b->m", c, a[to_yzx], b[to_yzx])
    np.testing.assert_allclose(got, np.cross(a, b)[to_yzx] / np.sqrt(2), atol=1e-14)


@pytest.mark.parametrize("l,l1,l2", [(1, 1, 2), (2, 1, 1), (3, 2, 1), (2, 2, 2), (3, 3, 2), (1, 1, 1)])
def test_exchange_symmetry(l, l1, l2):
    a, b = so3_clebsch_gordan(l, l1, l2), so3_clebsch_gordan(l, l2, l1)
    np.testing.assert_allclose(a, (-1) ** (l + l1 + l2) * b.transpose(0, 2, 1), atol=1e-15)


def test_nnz_counts_lmax2():
    nnz = {(0, 0, 0): 1, (0, 1, 1): 3, (0, 2, 2): 5, (1, 0, 1): 3, (1, 1, 0): 3, (1, 1, 2): 11, (1, 2, 1): 11,
           (2, 0, 2): 5, (2, 1, 1): 11, (2, 2, 0): 5, (2, 2, 2): 25}
    for t, n in nnz.items():
        assert np.count_nonzero(so3_clebsch_gordan(*t)) == n


def test_harmonics_consistent_with_coupling():
    """Y_l is proportional to C(l; l-1, 1) . Y_{l-1} (x) Y_1 and has |Y_l|^2 = 2l+1 on the sphere."""
    import torch
    from equitorch_amd.utils._sh import spherical_harmonics
    g = torch.Generator().manual_seed(0)
    v = torch.randn(50, 3, generator=g, dtype=torch.float64)
    v = v / v.norm(dim=-1, keepdim=True)
    y = spherical_harmonics(v, 6)
    assert torch.allclose(y[:, 1:4], 3 ** 0.5 * v[:, [1, 2, 0]])
    for l in range(7):
        blk = y[:, l * l:(l + 1) ** 2]
        assert torch.allclose((blk ** 2).sum(-1), torch.full((50,), 2.0 * l + 1, dtype=torch.float64))
