"""The rotation / SO(2)-linear oracle pinned on the CPU: the sparse rotation is a representation of SO(3) whose
degree-1 block is an ordinary rotation matrix and which transports the harmonics; the SO(2) layer commutes with
rotations about z."""
import math

import torch

from oracle import ref_ops, ref_sh, ref_tables

IRR = "0e+1o+2e+3o"


def _dense_d(alpha, beta, gamma, irr=IRR, max_m=3):
    z, _, _ = ref_tables.z_rotation_infos(irr)
    j = ref_tables.j_matrix_info(irr)
    dim = z["out_size"]
    n = alpha.shape[0]
    eye = torch.eye(dim, dtype=torch.float64).expand(n, dim, dim)
    sc = [ref_ops.cpu_sincos(a, max_m) for a in (alpha, beta, gamma)]
    return ref_ops.cpu_wigner_rotation(eye, *sc, z, j)


def _rot(axis, a):
    c, s = math.cos(a), math.sin(a)
    return torch.tensor({"z": [[c, -s, 0], [s, c, 0], [0, 0, 1]], "y": [[c, 0, s], [0, 1, 0], [-s, 0, c]]}[axis],
                        dtype=torch.float64)


def test_rotation_transports_harmonics_with_zyz_euler_angles():
    g = torch.Generator().manual_seed(0)
    ang = (torch.rand(3, 5, generator=g, dtype=torch.float64) - 0.5) * 2 * math.pi
    D = _dense_d(*ang)
    v = torch.randn(20, 3, generator=g, dtype=torch.float64)
    v = v / v.norm(dim=-1, keepdim=True)
    y = ref_sh.spherical_harmonics(v, 3)
    for k in range(5):
        # degree-1 block in (y, z, x) component order -> ordinary 3x3 rotation
        R = D[k, 1:4, 1:4][[2, 0, 1]][:, [2, 0, 1]]
        expect = _rot("z", float(ang[0, k])) @ _rot("y", float(ang[1, k])) @ _rot("z", float(ang[2, k]))
        torch.testing.assert_close(R, expect, atol=1e-12, rtol=0)
        torch.testing.assert_close(ref_sh.spherical_harmonics(v @ R.T, 3), y @ D[k].T, atol=1e-11, rtol=0)
        torch.testing.assert_close(D[k] @ D[k].T, torch.eye(16, dtype=torch.float64), atol=1e-12, rtol=0)
    # composition: D(a1,b1,c1) D(a2,b2,c2) belongs to R1 R2 (checked on the harmonics)
    R1 = D[0, 1:4, 1:4][[2, 0, 1]][:, [2, 0, 1]]
    R2 = D[1, 1:4, 1:4][[2, 0, 1]][:, [2, 0, 1]]
    torch.testing.assert_close(ref_sh.spherical_harmonics(v @ (R1 @ R2).T, 3), y @ (D[0] @ D[1]).T, atol=1e-11, rtol=0)


def test_so2_linear_commutes_with_rotations_about_z():
    g = torch.Generator().manual_seed(1)
    info, _, _, n_w = ref_tables.so2_linear_infos("0e+1o+2e", "0e+1o+2e+3o")
    z_in, _, _ = ref_tables.z_rotation_infos("0e+1o+2e+3o")
    z_out, _, _ = ref_tables.z_rotation_infos("0e+1o+2e")
    x = torch.randn(6, 16, 4, generator=g, dtype=torch.float64)
    phi = torch.rand(6, generator=g, dtype=torch.float64) * 6
    for w in (torch.randn(n_w, 4, generator=g, dtype=torch.float64),
              torch.randn(n_w, 4, 5, generator=g, dtype=torch.float64)):
        a = ref_ops.cpu_so2_linear(ref_ops.cpu_z_rotation(x, ref_ops.cpu_sincos(phi, 3), z_in), w, info)
        b = ref_ops.cpu_z_rotation(ref_ops.cpu_so2_linear(x, w, info), ref_ops.cpu_sincos(phi, 2), z_out)
        torch.testing.assert_close(a, b, atol=1e-12, rtol=0)
    # m = 0 components only see the m = 0 weights: 0e output = sum over inputs of x[l, m=0] * w / sqrt(count)
    w = torch.randn(n_w, 4, generator=g, dtype=torch.float64)
    out = ref_ops.cpu_so2_linear(x, w, info)
    m0 = [0, 2, 6, 12]                                   # m = 0 component of l = 0..3
    w0 = [0, 1, 2, 3]                                    # the paths into the 0e output carry one weight each
    expect = sum(x[:, m0[i]] * w[w0[i]] for i in range(4)) / 2.0
    torch.testing.assert_close(out[:, 0], expect)
