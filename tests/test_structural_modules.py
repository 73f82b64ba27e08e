"""SplitIrreps / Separable / AnglesToMatrix (plain tensor code) on the CPU."""
import math

import pytest
import torch

from equitorch_amd.nn.others import Separable, SplitIrreps
from equitorch_amd.nn.functional.rotations import angles_to_matrix


def test_split_and_separable():
    split = SplitIrreps("0e+1o+1o+2e", [1, -1, 1])
    assert split.split_sizes == [1, 6, 5] and [str(i.short_repr()) for i in split.irreps_out] == ["0e", "2x1o", "2e"]
    x = torch.randn(3, 12, 4)
    a, b, c = split(x)
    assert a.shape == (3, 1, 4) and b.shape == (3, 6, 4) and torch.equal(torch.cat([a, b, c], dim=1), x)
    sep = Separable("0e+1o+1o+2e", [1, 2, 1], [torch.nn.Identity(), None, torch.nn.Tanh()])
    y = sep(x)
    assert torch.equal(y[:, :7], x[:, :7]) and torch.equal(y[:, 7:], torch.tanh(x[:, 7:]))
    with pytest.raises(ValueError):
        SplitIrreps("0e+1o", [1, 2])
    with pytest.raises(ValueError):
        split(x[:, :5])


def test_angles_to_matrix_order_and_orthogonality():
    a, b, g = torch.tensor([0.3, -1.1]), torch.tensor([0.7, 2.0]), torch.tensor([-0.4, 0.9])
    R = angles_to_matrix(a, b, g)
    assert R.shape == (2, 3, 3)
    torch.testing.assert_close(R @ R.transpose(-1, -2), torch.eye(3).expand(2, 3, 3), atol=1e-6, rtol=0)
    # alpha acts first: a pure alpha rotation is R_z(alpha); gamma = pi/2 after beta = pi/2 takes z to y
    c, s = math.cos(0.3), math.sin(0.3)
    torch.testing.assert_close(angles_to_matrix(alpha=a)[0], torch.tensor([[c, -s, 0.0], [s, c, 0.0], [0.0, 0.0, 1.0]]))
    z = torch.tensor([0.0, 0.0, 1.0])
    Rzy = angles_to_matrix(beta=torch.tensor(math.pi / 2), gamma=torch.tensor(math.pi / 2))
    torch.testing.assert_close(Rzy @ z, torch.tensor([0.0, 1.0, 0.0]), atol=1e-6, rtol=0)
    with pytest.raises(ValueError):
        angles_to_matrix()
