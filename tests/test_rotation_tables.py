"""Tables of the Wigner rotation (z-rotation, J matrix) and of SO2Linear: the product's builders and the oracle's
restatement against the golden fixture written by the reference's own ``wigner_d_info`` / ``so2_linear_infos``
(tests/golden/make_rotation_tables.py), bit for bit; plus what the J matrix must satisfy mathematically."""
import os

import numpy as np
import pytest
import torch

from equitorch_amd.constants import j_matrix
from equitorch_amd.utils import so2_linear_infos, wigner_d_info
from oracle import ref_constants, ref_sh, ref_tables

FX = np.load(os.path.join(os.path.dirname(__file__), "golden", "rotation_tables.npz"))
WIGNER_CASES = {"sh2": "0e+1o+2e", "so3_04": (0, 4), "odd13": "1o+3o", "mult": "2x1o+2e"}
SO2_CASES = {
    "sh2": ("0e+1o+2e", "0e+1o+2e", {}),
    "sh3_to_2": ("0e+1o+2e", "0e+1o+2e+3o", {}),
    "mult": ("1o+2e", "2x1o+2e+0e", {}),
    "nonorm": ("0e+1o+2e", "0e+1o+2e", {"path_norm": False}),
    "chnorm": ("0e+1o+2e", "0e+1o+2e", {"channel_norm": True, "channel_scale": 0.125}),
    "path": ("0e+1o+2e", "0e+1o+2e", {"path": [(0, 0), (1, 1), (2, 1), (2, 2)]}),
}


def _check(prefix, fields):
    """fields: {name: tensor | list | int | None}; lists are the oracle's (scale lists rounded to fp32 here, the way
    ``torch.tensor(list)`` rounds them in the reference)."""
    none = set(FX[prefix + "/__none__"].tolist())
    for name, v in fields.items():
        key = f"{prefix}/{name}"
        if v is None:
            assert name in none, f"{key}: the reference has a tensor here"
            continue
        if isinstance(v, int):
            assert int(FX[key]) == v, key
            continue
        assert name not in none, f"{key}: the reference has None here"
        t = v if isinstance(v, torch.Tensor) else torch.tensor(v)
        assert str(t.dtype) == str(FX[key + "/dtype"]), (key, t.dtype)
        assert np.array_equal(t.numpy(), FX[key]), key


def _fields(info):
    return info._asdict() if hasattr(info, "_asdict") else {k: v for k, v in info.items()}


@pytest.mark.parametrize("name", list(WIGNER_CASES))
def test_wigner_tables_match_golden(name):
    mine = wigner_d_info(WIGNER_CASES[name])
    ref_z = ref_tables.z_rotation_infos(WIGNER_CASES[name])
    ref_j = ref_tables.j_matrix_info(WIGNER_CASES[name])
    _check(f"wigner/{name}/j_matrix_info", _fields(mine.j_matrix_info))
    _check(f"wigner/{name}/j_matrix_info", _fields(ref_j))
    for k, field in enumerate(("rotate_z_info_fwd", "rotate_z_info_bwd_input", "rotate_z_info_bwd_cs")):
        _check(f"wigner/{name}/{field}", _fields(getattr(mine, field)))
        _check(f"wigner/{name}/{field}", _fields(ref_z[k]))
    assert np.array_equal(mine.sign.numpy(), FX[f"wigner/{name}/sign"])
    assert mine.max_m == int(FX[f"wigner/{name}/max_m"])


@pytest.mark.parametrize("name", list(SO2_CASES))
def test_so2_linear_tables_match_golden(name):
    io, ii, kw = SO2_CASES[name]
    *mine, n = so2_linear_infos(io, ii, **kw)
    *ref, n_ref = ref_tables.so2_linear_infos(io, ii, **kw)
    assert n == n_ref == int(FX[f"so2/{name}/num_weights"])
    for d, a, b in zip(("fwd", "bwd1", "bwd2"), mine, ref):
        _check(f"so2/{name}/{d}", _fields(a))
        _check(f"so2/{name}/{d}", _fields(b))


def test_j_matrix_is_the_harmonics_image_of_the_axis_exchange():
    """J is an involution, orthogonal, and Y(-x, z, y) = J Y(x, y, z) for the harmonics of the oracle; the product's
    float64 J equals the oracle's exact one."""
    v = torch.randn(30, 3, generator=torch.Generator().manual_seed(0), dtype=torch.float64)
    v = v / v.norm(dim=-1, keepdim=True)
    jv = torch.stack([-v[:, 0], v[:, 2], v[:, 1]], dim=-1)
    y, yj = ref_sh.spherical_harmonics(v, 4), ref_sh.spherical_harmonics(jv, 4)
    for l in range(5):
        J = torch.tensor(j_matrix(l))
        exact = torch.tensor([[float(e) for e in row] for row in ref_constants.j_matrix(l)], dtype=torch.float64)
        torch.testing.assert_close(J, exact, atol=1e-14, rtol=0)
        torch.testing.assert_close(J @ J, torch.eye(2 * l + 1, dtype=torch.float64), atol=1e-13, rtol=0)
        s = slice(l * l, (l + 1) ** 2)
        torch.testing.assert_close(yj[:, s], y[:, s] @ J.T, atol=1e-12, rtol=0)
