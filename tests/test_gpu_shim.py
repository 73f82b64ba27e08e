"""The PyTorch C++ extension over the C ABI (``equitorch_amd/lib/_cgtp_torch.so``): the fused edge product issued
through its autograd node must give the same bits as the same launches issued through ``ctypes`` — both call
``cgtp_uvu_fwd`` / ``cgtp_uvu_bwd`` with the same argument block."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _sh(lmax):
    return "+".join(f"{l}{'e' if l % 2 == 0 else 'o'}" for l in range(lmax + 1))


def _case(device, lmax, ch, n_nodes, n_edges, dtype, shared_w, vectors, kw, need=(True, True, True)):
    from equitorch_amd import _shim
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu, edge_tensor_product_uu_vectors
    assert _shim.module() is not None, "the extension is not built"
    irr = _sh(lmax)
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu", **kw).to(device)
    d = (lmax + 1) ** 2
    g = torch.Generator().manual_seed(lmax + ch + n_edges)
    src = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst = torch.randint(0, n_nodes, (n_edges,), generator=g)
    dst[dst == 3] = 4                                           # a node without edges
    x = torch.randn(n_nodes, d, ch, generator=g, dtype=dtype)
    y = torch.randn(n_edges, 3 if vectors else d, generator=g, dtype=dtype)
    w = torch.randn(*(() if shared_w else (n_edges,)), mod.num_paths, ch, generator=g, dtype=dtype)
    ct = torch.randn(n_nodes, d, ch, generator=g, dtype=dtype).to(device)
    fn = edge_tensor_product_uu_vectors if vectors else edge_tensor_product_uu
    results = []
    for use_shim in (True, False):
        plan = EdgePlan(src.to(device), dst.to(device), n_nodes)
        saved = _shim._module
        if not use_shim:
            _shim._module = None
        try:
            leaves = [t.to(device).requires_grad_(r) for t, r in zip((x, y, w), need)]
            out = fn(*leaves, plan, mod.tp_info_forward)
            assert ("Cpp" in type(out.grad_fn).__name__) == use_shim, type(out.grad_fn).__name__   # C++ nodes show as CppFunction
            grads = torch.autograd.grad(out, [t for t, r in zip(leaves, need) if r], ct)
        finally:
            _shim._module = saved
        results.append((out, *grads))
    for a, b in zip(*results):
        assert torch.equal(a, b)


@pytest.mark.parametrize("lmax,ch,dtype,shared_w,vectors,kw", [
    (2, 64, torch.float32, False, False, {}),
    (2, 64, torch.float32, True, False, {}),
    (2, 64, torch.float32, False, True, {}),
    (1, 32, torch.float64, False, False, {}),
    (2, 48, torch.float32, False, False, {"path_norm": False}),      # a factor per weight path next to the compiled table
    (3, 20, torch.float32, False, False, {}),
    (6, 32, torch.float32, False, False, {}),                        # block-wise kernels, ranges by position
])
def test_extension_and_ctypes_issue_the_same_launches(device, lmax, ch, dtype, shared_w, vectors, kw):
    _case(device, lmax, ch, 200, 3000, dtype, shared_w, vectors, kw)


def test_gradient_subsets_and_no_grad(device):
    for need in ((True, False, False), (False, True, True), (False, False, True)):
        _case(device, 2, 64, 100, 1500, torch.float32, False, False, {}, need)
    from equitorch_amd.nn import SO3Linear
    from equitorch_amd.nn.functional import EdgePlan, edge_tensor_product_uu
    irr = _sh(2)
    mod = SO3Linear(irr, irr, irr, 64, 64, internal_weights=False, feature_mode="uu").to(device)
    plan = EdgePlan(torch.randint(0, 50, (400,), device=device), torch.randint(0, 50, (400,), device=device), 50)
    with torch.no_grad():
        out = edge_tensor_product_uu(torch.randn(50, 9, 64, device=device), torch.randn(400, 9, device=device),
                                     torch.randn(400, 11, 64, device=device), plan, mod.tp_info_forward)
    assert out.shape == (50, 9, 64) and out.grad_fn is None and torch.isfinite(out).all()


@pytest.mark.parametrize("lmax,ch,dtype,shared_w,kw", [
    (2, 16, torch.float32, True, {}),
    (2, 64, torch.float32, False, {}),
    (3, 32, torch.float64, True, {}),
    (2, 20, torch.float32, True, {"path_norm": False}),
])
def test_row_mode_through_the_extension(device, lmax, ch, dtype, shared_w, kw):
    """``SO3Linear('uu')`` on a batch: first-order results bit-equal to the ``ctypes`` route; a gradient of the
    gradient goes back to Python's differentiable route and agrees with it."""
    from equitorch_amd import _shim
    from equitorch_amd.nn import SO3Linear
    assert _shim.module() is not None
    irr, n, d = _sh(lmax), 700, (lmax + 1) ** 2
    mod = SO3Linear(irr, irr, irr, ch, ch, internal_weights=False, feature_mode="uu", **kw).to(device)
    g = torch.Generator().manual_seed(lmax * 100 + ch)
    x, y = torch.randn(n, d, ch, generator=g, dtype=dtype), torch.randn(n, d, generator=g, dtype=dtype)
    w = torch.randn(*(() if shared_w else (n,)), mod.num_paths, ch, generator=g, dtype=dtype)
    ct = torch.randn(n, d, ch, generator=g, dtype=dtype).to(device)
    first, second = [], []
    for use_shim in (True, False):
        saved = _shim._module
        if not use_shim:
            _shim._module = None
        try:
            xd, yd, wd = (t.to(device).requires_grad_(True) for t in (x, y, w))
            out = mod(xd, yd, wd)
            assert ("Cpp" in type(out.grad_fn).__name__) == use_shim, type(out.grad_fn).__name__
            grads = torch.autograd.grad(out, (xd, yd, wd), ct, retain_graph=True)
            gx, = torch.autograd.grad(out, xd, ct, create_graph=True)
            gg = torch.autograd.grad(gx.square().sum(), (yd, wd))
        finally:
            _shim._module = saved
        first.append((out, *grads))
        second.append(gg)
    for a, b in zip(*first):
        assert torch.equal(a, b)
    for a, b in zip(*second):
        assert torch.allclose(a, b, rtol=1e-5 if dtype == torch.float32 else 1e-12, atol=1e-5 if dtype == torch.float32 else 1e-12)
