"""GPU parity of the sparse Wigner rotation, the dense Wigner matrices and SO2Linear against the oracle."""
import math

import pytest
import torch

from helpers import assert_close
from oracle import ref_ops, ref_sh, ref_tables

pytestmark = pytest.mark.gpu

IRR = "0e+1o+2e+3o"


def _f32(d):
    """Scale lists as the reference stores them: fp32 values."""
    d = dict(d)
    d["scale"] = torch.tensor(d["scale"]).double().tolist()
    return d


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_sparse_rotation_and_its_gradients(device, dtype):
    from equitorch_amd.nn import SparseWignerRotation
    from equitorch_amd.nn.functional import sincos
    z = _f32(ref_tables.z_rotation_infos(IRR)[0])
    j = _f32(ref_tables.j_matrix_info(IRR))
    g = torch.Generator().manual_seed(0)
    n, c = 50, 12
    x = torch.randn(n, 16, c, generator=g, dtype=torch.float64).to(dtype).double()
    ang = ((torch.rand(3, n, generator=g, dtype=torch.float64) - 0.5) * 6).to(dtype).double()
    ct = torch.randn(n, 16, c, generator=g, dtype=torch.float64).to(dtype).double()
    xr, ar = x.clone().requires_grad_(True), ang.clone().requires_grad_(True)
    ref = ref_ops.cpu_wigner_rotation(xr, *(ref_ops.cpu_sincos(ar[k], 3) for k in range(3)), z, j)
    rgx, rga = torch.autograd.grad(ref, (xr, ar), ct)
    mod = SparseWignerRotation(IRR).to(device)
    xd, ad = x.to(device, dtype).requires_grad_(True), ang.to(device, dtype).requires_grad_(True)
    out = mod(xd, *(sincos(ad[k], 3) for k in range(3)))
    gx, ga = torch.autograd.grad(out, (xd, ad), ct.to(device, dtype))
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    assert_close(out, ref, tol=tol, what="rotated features")
    assert_close(gx, rgx, tol=tol, what="grad input")
    assert_close(ga, rga, tol=10 * tol, what="grad angles")
    # an angle given as None is skipped
    ref0 = ref_ops.cpu_wigner_rotation(x, None, ref_ops.cpu_sincos(ang[1], 3), None, z, j)
    assert_close(mod(xd, None, sincos(ad[1], 3), None), ref0, tol=tol, what="beta only")


def test_dense_wigner_matrices_and_alignment(device):
    from equitorch_amd.nn import AlignToZWignerD, DenseWignerRotation, WignerD
    g = torch.Generator().manual_seed(1)
    n = 9
    ang = (torch.rand(3, n, generator=g, dtype=torch.float64) - 0.5) * 6
    wd = WignerD(IRR).to(device).double()
    D = wd(alpha=ang[0].to(device), beta=ang[1].to(device), gamma=ang[2].to(device))
    assert D.shape == (n, 16, 16)
    v = torch.randn(15, 3, generator=g, dtype=torch.float64)
    v = v / v.norm(dim=-1, keepdim=True)
    y = ref_sh.spherical_harmonics(v, 3)
    for k in range(n):
        Dk = D[k].cpu()
        R = Dk[1:4, 1:4][[2, 0, 1]][:, [2, 0, 1]]          # degree-1 block, (y, z, x) -> (x, y, z)
        assert_close(ref_sh.spherical_harmonics(v @ R.T, 3), y @ Dk.T, tol=1e-6, what="D transports harmonics")
    single = wd(beta=ang[1, :1].to(device))
    assert single.shape == (16, 16)                         # no batch of more than one: the batch axis is dropped
    # alignment: D(v) Y(v) = Y(z axis) = sqrt(2l+1) on the m = 0 components
    vz = v[:n].to(device)
    Dz = AlignToZWignerD(IRR, normalized=True).to(device).double()(vz)
    target = torch.zeros(16, dtype=torch.float64)
    for l in range(4):
        target[l * l + l] = math.sqrt(2 * l + 1)
    yz = DenseWignerRotation(IRR)(y[:n].to(device).unsqueeze(-1), Dz).squeeze(-1)
    assert_close(yz, target.expand(n, 16), tol=1e-6, what="aligned harmonics")


@pytest.mark.parametrize("mode,per_sample", [("uu", False), ("uu", True), ("uv", False), ("uv", True)])
def test_so2_linear(device, mode, per_sample):
    from equitorch_amd.nn import SO2Linear
    irr_in, irr_out = "0e+1o+2e+3o", "0e+1o+2e"
    info = _f32(ref_tables.so2_linear_infos(irr_out, irr_in)[0])
    n, cin, cout = 31, 8, 8 if mode == "uu" else 6
    mod = SO2Linear(irr_in, irr_out, cin, cout, internal_weights=False, feature_mode=mode).to(device)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(n, 16, cin, generator=g, dtype=torch.float64)
    wshape = (mod.num_weights, cout) if mode == "uu" else (mod.num_weights, cin, cout)
    w = torch.randn(*((n,) if per_sample else ()), *wshape, generator=g, dtype=torch.float64)
    ct = torch.randn(n, 9, cout, generator=g, dtype=torch.float64)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_so2_linear(xr, wr, info, per_sample=per_sample)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    xd, wd = x.to(device).requires_grad_(True), w.to(device).requires_grad_(True)
    out = mod(xd, wd)
    gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device))
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert_close(a, b, tol=1e-11, what=f"SO2Linear {mode} per_sample={per_sample} {name}")


@pytest.mark.parametrize("cin,cout,n", [(32, 48, 300), (64, 64, 33)])
def test_so2_linear_uv_fp32_on_the_matrix_core_kernels(device, cin, cout, n):
    """fp32 with a shared weight: the table of the layer is handed to the table-driven kernels of the fully
    connected product as it is (second operand = the scalar 1); out, grad_x and grad_w against the oracle, and the
    second-order route (create_graph) still differentiates."""
    from equitorch_amd.nn import SO2Linear
    from equitorch_amd.nn.functional import _uv_native
    irr_in, irr_out = "0e+1o+2e+3o", "0e+1o+2e"
    info = _f32(ref_tables.so2_linear_infos(irr_out, irr_in)[0])
    mod = SO2Linear(irr_in, irr_out, cin, cout, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(n, 16, cin, generator=g).double()
    w = (torch.randn(mod.num_weights, cin, cout, generator=g) / cin ** 0.5).double()
    ct = torch.randn(n, 9, cout, generator=g).double()
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_so2_linear(xr, wr, info, per_sample=False)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    xd, wd = x.float().to(device).requires_grad_(True), w.float().to(device).requires_grad_(True)
    calls = []
    orig = _uv_native.apply
    _uv_native.apply = lambda *a, **k: (calls.append(1), orig(*a, **k))[1]
    try:
        out = mod(xd, wd)
        gx, gw = torch.autograd.grad(out, (xd, wd), ct.float().to(device), create_graph=True)
    finally:
        _uv_native.apply = orig
    assert calls, "the layer did not run on the table-driven kernels"
    def second_order(xs, ws, cts):
        return torch.autograd.grad(torch.autograd.grad(ref_ops.cpu_so2_linear(xs, ws, info, per_sample=False), ws, cts,
                                                       create_graph=True)[0].sum(), xs)[0]
    # the same CPU function on float32 tensors: what the reference's own fp32 arithmetic loses
    x32, w32 = x.float().requires_grad_(True), w.float().requires_grad_(True)
    ref32 = ref_ops.cpu_so2_linear(x32, w32, info, per_sample=False)
    r32 = (ref32, *torch.autograd.grad(ref32, (x32, w32), ct.float()))
    for (name, a, b), b32 in zip((("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)), r32):
        # sums over C_in (x paths) products; grad_w also over the batch
        assert_close(a, b, tol=1e-5, what=f"SO2Linear uv fp32 {cin}->{cout} {name}", norm="max", fp32_ref=b32)
    (ggx,) = torch.autograd.grad(gw.sum(), (xd,))          # second order through the differentiable route
    assert_close(ggx, second_order(xr, wr, ct), tol=1e-5, what="SO2Linear uv fp32 d(grad_w)/dx", norm="max",
                 fp32_ref=second_order(x32, w32, ct.float()))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("channels", [64, 10])
def test_fused_rotation_kernel(device, dtype, channels):
    """``cgtp_wigner_rotate`` (forward and, with angles that need no gradient, the transposed launch for the gradient
    of the features) against the oracle and against the five-launch composition: irreps up to l = 6 with a repeated
    and an out-of-order degree, 16-byte and single-element lanes, rows not a multiple of the rows per wavefront,
    every subset of the three angles."""
    from equitorch_amd.nn.functional import sincos, sparse_wigner_rotation
    from equitorch_amd.nn.functional.wigner_d import _composed_rotation
    from equitorch_amd.ops import kernels
    from equitorch_amd.utils import wigner_d_info
    irr = "2e+0e+6e+1o+1o+4e"
    dim = 5 + 1 + 13 + 3 + 3 + 9
    z = _f32(ref_tables.z_rotation_infos(irr)[0])
    j = _f32(ref_tables.j_matrix_info(irr))
    info = wigner_d_info(irr).to(device)
    layout = kernels.rotation_layout(info)
    assert layout.ok and list(layout.degree) == [2, 0, 6, 1, 1, 4] and list(layout.first) == [0, 5, 6, 19, 22, 25]
    assert kernels.wigner_rotate_supported(layout, channels, dtype)
    g = torch.Generator().manual_seed(3)
    n = 77
    x = torch.randn(n, dim, channels, generator=g, dtype=torch.float64).to(dtype).double()
    ang = ((torch.rand(3, n, generator=g, dtype=torch.float64) - 0.5) * 6).to(dtype).double()
    ct = torch.randn(n, dim, channels, generator=g, dtype=torch.float64).to(dtype).double()
    tol = 1e-5 if dtype == torch.float32 else 1e-11
    for use in ((1, 1, 1), (1, 0, 0), (0, 1, 0), (0, 0, 1), (1, 0, 1)):
        xr = x.clone().requires_grad_(True)
        ref = ref_ops.cpu_wigner_rotation(xr, *(ref_ops.cpu_sincos(ang[k], 6) if use[k] else None for k in range(3)), z, j)
        (rgx,) = torch.autograd.grad(ref, xr, ct)
        xd = x.to(device, dtype).requires_grad_(True)
        cs = [sincos(ang[k].to(device, dtype), 6) if use[k] else None for k in range(3)]
        out = sparse_wigner_rotation(xd, *cs, info)
        assert type(out.grad_fn).__name__ == "_FusedRotationBackward"
        (gx,) = torch.autograd.grad(out, xd, ct.to(device, dtype))
        assert_close(out, ref, tol=tol, what=f"rotation {use}")
        assert_close(gx, rgx, tol=tol, what=f"transposed rotation {use}")
        with torch.no_grad():
            comp = _composed_rotation(xd, *cs, info)
        assert_close(out, comp, tol=1e-6 if dtype == torch.float32 else 1e-13, what=f"against the composition {use}")
    # degrees above 6 are outside the fused kernel
    big = wigner_d_info("0e+7o").to(device)
    assert not kernels.wigner_rotate_supported(kernels.rotation_layout(big), channels, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
@pytest.mark.parametrize("irr,channels", [("2e+0e+6e+1o+1o+4e", 64), ("2e+0e+6e+1o+1o+4e", 10), ("0e+1o+2e+1o", 64),
                                          ("3o+4e", 24)])
def test_fused_rotation_gradients_of_the_sincos_tensors(device, dtype, irr, channels):
    """``cgtp_wigner_rotate_backward``: gradients of the features and of the three sincos tensors (leaves here, with
    more columns than the largest degree needs) against the oracle's autograd, for largest degrees 2, 4 and 6 (four,
    four and two channels per lane in fp32) and every subset of angles; a sincos tensor that is given but needs no
    gradient gets none."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn.functional import sparse_wigner_rotation
    from equitorch_amd.utils import wigner_d_info
    dim, max_l = Irreps(irr).dim, max(ir.l for ir in Irreps(irr))
    z = _f32(ref_tables.z_rotation_infos(irr)[0])
    j = _f32(ref_tables.j_matrix_info(irr))
    info = wigner_d_info(irr).to(device)
    g = torch.Generator().manual_seed(4)
    n, extra = 53, 2
    x = torch.randn(n, dim, channels, generator=g, dtype=torch.float64).to(dtype).double()
    ang = (torch.rand(3, n, generator=g, dtype=torch.float64) - 0.5) * 6
    cs = [torch.cat([ref_ops.cpu_sincos(ang[k], max_l), torch.randn(n, extra, generator=g, dtype=torch.float64)], dim=1)
          .to(dtype).double() for k in range(3)]
    ct = torch.randn(n, dim, channels, generator=g, dtype=torch.float64).to(dtype).double()
    tol = 2e-5 if dtype == torch.float32 else 1e-10
    for use in ((1, 1, 1), (0, 1, 1), (1, 0, 0), (0, 0, 1)):
        xr = x.clone().requires_grad_(True)
        cr = [c[:, :1 + 2 * max_l].clone().requires_grad_(True) if u else None for c, u in zip(cs, use)]
        ref = ref_ops.cpu_wigner_rotation(xr, *cr, z, j)
        refs = torch.autograd.grad(ref, [xr] + [c for c in cr if c is not None], ct)
        xd = x.to(device, dtype).requires_grad_(True)
        cd = [c.to(device, dtype).requires_grad_(True) if u else None for c, u in zip(cs, use)]
        out = sparse_wigner_rotation(xd, *cd, info)
        assert type(out.grad_fn).__name__ == "_FusedRotationBackward"
        got = torch.autograd.grad(out, [xd] + [c for c in cd if c is not None], ct.to(device, dtype))
        assert_close(got[0], refs[0], tol=tol, what=f"grad x {use}")
        for a, b in zip(got[1:], refs[1:]):
            # sums over dim x channels products: judged relative to the largest entry
            assert_close(a[:, :1 + 2 * max_l], b, tol=tol * 10, what=f"grad sincos {use}")
            assert float(a[:, 1 + 2 * max_l:].abs().max()) == 0.0
    # only one of two given sincos tensors needs a gradient
    xd = x.to(device, dtype)
    ca = cs[0].to(device, dtype).requires_grad_(True)
    cb = cs[1].to(device, dtype)
    (ga,) = torch.autograd.grad(sparse_wigner_rotation(xd, ca, cb, None, info), ca, ct.to(device, dtype))
    cr = [cs[0][:, :1 + 2 * max_l].clone().requires_grad_(True), cs[1][:, :1 + 2 * max_l]]
    (ra,) = torch.autograd.grad(ref_ops.cpu_wigner_rotation(x, cr[0], cr[1], None, z, j), cr[0], ct)
    assert_close(ga[:, :1 + 2 * max_l], ra, tol=tol * 10, what="grad of alpha alone")


@pytest.mark.parametrize("dtype,cin,cout", [(torch.bfloat16, 16, 24), (torch.float32, 6, 5)])
def test_so2_linear_uv_adapted_operands(device, monkeypatch, dtype, cin, cout):
    """bf16 operands (widened to fp32) and channel counts that are not multiples of 4 (zero channels appended) on the
    table-driven kernels; against the oracle on the rounded inputs."""
    from equitorch_amd.nn import SO2Linear
    from equitorch_amd.ops import kernels
    irr_in, irr_out, n = "0e+1o+2e+3o", "0e+1o+2e", 77
    info = _f32(ref_tables.so2_linear_infos(irr_out, irr_in)[0])
    mod = SO2Linear(irr_in, irr_out, cin, cout, internal_weights=False, feature_mode="uv").to(device)
    g = torch.Generator().manual_seed(6)
    rd = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64).to(dtype).double()
    x, w, ct = rd(n, 16, cin), rd(mod.num_weights, cin, cout) / cin ** 0.5, rd(n, 9, cout)
    w = w.to(dtype).double()
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_so2_linear(xr, wr, info)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    seen = []
    monkeypatch.setattr(kernels, "log_tier", lambda op, tier, detail="": seen.append(tier))
    xd, wd = (t.to(device, dtype).requires_grad_(True) for t in (x, w))
    out = mod(xd, wd)
    assert seen and "table-driven matrix-core" in seen[-1], seen
    gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device, dtype))
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
        assert a.dtype == dtype and a.shape == b.shape
        assert_close(a.double(), b, tol, f"SO2Linear uv {dtype} {cin}->{cout} {name}",
                     norm="element" if dtype == torch.float32 else "max")


@pytest.mark.parametrize("irr_in,irr_out", [("0e", "1o+2e"), ("1o+1e", "2e+0e"), ("0e", "2e+0e"), ("0e", "1o")])
@pytest.mark.parametrize("mode,per_sample", [("uu", False), ("uu", True), ("uv", False), ("uv", True)])
def test_so2_linear_on_tables_the_reference_builder_leaves_incomplete(device, irr_in, irr_out, mode, per_sample):
    """When the first output component has no entry (no input component of its order), the reference's
    ``sparse_product_info`` (``equitorch/utils/_structs.py:105-123``) shifts its segment pointers by a row: entries
    move to the wrong output rows, the last ones are reached by no row, and with ``0e -> 2e+0e`` none is reached at
    all.  The tables here are the reference's bit for bit, so the modules follow them — result and gradients of the
    reference's algorithm on those tables, zero gradient for a weight no row uses (not whatever the allocator
    returned: the buffers are dirtied first), zeros with zero gradients for a table without a reachable entry."""
    from equitorch_amd.irreps import Irreps
    from equitorch_amd.nn import SO2Linear
    info = _f32(ref_tables.so2_linear_infos(irr_out, irr_in)[0])
    n, cin = 17, 33 if mode == "uv" else 8
    cout = 4 if mode == "uv" else cin
    mod = SO2Linear(irr_in, irr_out, cin, cout, internal_weights=False, feature_mode=mode).to(device)
    g = torch.Generator().manual_seed(len(irr_in) + len(irr_out))
    x = torch.randn(n, Irreps(irr_in).dim, cin, generator=g, dtype=torch.float64)
    wshape = (mod.num_weights, cout) if mode == "uu" else (mod.num_weights, cin, cout)
    w = torch.randn(*((n,) if per_sample else ()), *wshape, generator=g, dtype=torch.float64)
    ct = torch.randn(n, Irreps(irr_out).dim, cout, generator=g, dtype=torch.float64)
    xr, wr = x.clone().requires_grad_(True), w.clone().requires_grad_(True)
    ref = ref_ops.cpu_so2_linear(xr, wr, info, per_sample=per_sample)
    rgx, rgw = torch.autograd.grad(ref, (xr, wr), ct)
    for dtype, tol in ((torch.float64, 1e-11), (torch.float32, 1e-5)):
        xd, wd = x.to(device, dtype).requires_grad_(True), w.to(device, dtype).requires_grad_(True)
        dirt = [torch.full_like(t, 1e3) for t in (xd, wd, wd)]
        del dirt
        out = mod(xd, wd)
        gx, gw = torch.autograd.grad(out, (xd, wd), ct.to(device, dtype))
        for name, a, b in (("out", out, ref), ("grad_x", gx, rgx), ("grad_w", gw, rgw)):
            assert_close(a, b, tol=tol, what=f"SO2Linear {irr_in} -> {irr_out} {mode} per_sample={per_sample} {dtype} {name}",
                         norm="max")
