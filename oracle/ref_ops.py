"""TEST INFRASTRUCTURE ONLY: CPU numerics of the sparse tensor-product path.

Two independent restatements:

* ``dense_*`` — float64 einsum straight from the dense Clebsch-Gordan blocks (no sparse table involved),
  differentiated by torch autograd.  This is the arbiter for parity.
* ``cpu_*`` — step-for-step restatement of the reference's CPU fallbacks in torch CPU ops
  (``index_select`` both operands to nnz length -> product -> ``* scale`` -> CSR segment-sum), composed as the
  reference's Functions compose them.  ``torch_geometric.utils.segment`` (PyG 2.5.3, absent here; used at
  ``equitorch/ops/batched_sparse_dense_op.py:262,818,1495,1781`` and ``indexed_scale_segment_op.py:167``) is a
  CSR sum along dim 1 and is restated as ``index_add_`` over expanded segment ids.  This is the timed
  "reference CPU path" of the benchmark.

Pinned by: agreement of the two restatements with each other (tests/test_oracle.py, tests/test_oracle_uv.py),
and for the dense one by O(3)-equivariance, the l2=0 scaling identity, the 1x1->0 dot product, the 1x1->1
cross product and ``torch.autograd.gradcheck``; the fully connected members (``dense_u1v``, ``dense_uvw``)
additionally by their reduction to ``x @ W`` at lmax = 0, by the ``l2 = 0`` paths being ``y0 * x[block] @ W[p]``,
by ``dense_uvw`` with a single second-operand channel equal to ``dense_u1v`` and with diagonal weights equal to
``dense_uuu``, and by the structural ``cpu_u1v_* / cpu_1vu_* / cpu_vu1_* / cpu_uvw_*`` chains.  No stored output
vectors exist in the reference for this path.
"""
import torch

from . import ref_constants, ref_tables


# ---- dense float64 oracle -----------------------------------------------------------------------------------
def dense_coupling(irreps_out, irreps1, irreps2, path=None, path_norm=True, channel_norm=False,
                   channel_scale=1.0) -> torch.Tensor:
    """``T[p, M, M1, M2]`` float64 with the path normalisation of ``prepare_so3``
    (``equitorch/utils/_structs.py:177-206``) folded in."""
    io, i1, i2 = ref_tables.parse(irreps_out), ref_tables.parse(irreps1), ref_tables.parse(irreps2)
    if not path:
        path = ref_tables.fully_connected_paths(io, i1, i2)
    so, s1, s2 = ref_tables.segments(io), ref_tables.segments(i1), ref_tables.segments(i2)
    count, cur = {}, None
    for k, _, _ in path:
        count[k] = count[k] + 1 if k == cur else 1
        cur = k
    T = torch.zeros(len(path), so[-1], s1[-1], s2[-1], dtype=torch.float64)
    for p, (k, i, j) in enumerate(path):
        cg = ref_constants.so3_cg(io[k][0], i1[i][0], i2[j][0])
        blk = torch.tensor([[[float(v) for v in r] for r in m] for m in cg], dtype=torch.float64)
        norm = (count[k] ** -0.5 if path_norm else 1.0) * (channel_scale if channel_norm else 1.0)
        T[p, so[k]:so[k + 1], s1[i]:s1[i + 1], s2[j]:s2[j + 1]] = blk * norm
    return T


def dense_u1u(T, x, y, w, dtype=torch.float64):
    """``out[n,M,c] = sum T[p,M,a,b] x[n,a,c] y[n,b] w[(n),p,c]`` in float64 (the arbiter), or in ``dtype``: with
    float32, what plain fp32 arithmetic loses on the same contraction — the yardstick the tests hold a kernel's
    rounding error against where an element-wise relative bound cannot hold."""
    T, x, y, w = T.to(dtype), x.to(dtype), y.to(dtype), w.to(dtype)
    if w.ndim == 2:
        return torch.einsum("pmab,nac,nb,pc->nmc", T, x, y, w)
    return torch.einsum("pmab,nac,nb,npc->nmc", T, x, y, w)


def dense_uuu(T, x, y, w, dtype=torch.float64):
    T, x, y, w = T.to(dtype), x.to(dtype), y.to(dtype), w.to(dtype)
    if w.ndim == 2:
        return torch.einsum("pmab,nac,nbc,pc->nmc", T, x, y, w)
    return torch.einsum("pmab,nac,nbc,npc->nmc", T, x, y, w)


def dense_u1v(T, x, y, w, dtype=torch.float64):
    """``out[n,M,v] = sum T[p,M,a,b] y[n,b] x[n,a,u] w[(n),p,u,v]``."""
    T, x, y, w = T.to(dtype), x.to(dtype), y.to(dtype), w.to(dtype)
    if w.ndim == 3:
        return torch.einsum("pmab,nau,nb,puv->nmv", T, x, y, w)
    return torch.einsum("pmab,nau,nb,npuv->nmv", T, x, y, w)


def dense_uvw(T, x, y, w, dtype=torch.float64):
    T, x, y, w = T.to(dtype), x.to(dtype), y.to(dtype), w.to(dtype)
    if w.ndim == 4:
        return torch.einsum("pmab,nau,nbv,puvw->nmw", T, x, y, w)
    return torch.einsum("pmab,nau,nbv,npuvw->nmw", T, x, y, w)


def dense_grads(fn, T, inputs, cotangent, dtype=torch.float64):
    """``(out, gradients)`` of ``(fn(T, *inputs) * cotangent).sum()`` w.r.t. every input, in float64 (or ``dtype``)."""
    leaves = [t.detach().to(dtype).requires_grad_(True) for t in inputs]
    out = fn(T, *leaves) if dtype == torch.float64 else fn(T, *leaves, dtype=dtype)
    return out.detach(), torch.autograd.grad((out * cotangent.to(dtype)).sum(), leaves)


def scatter_sum(msg, dst, num_nodes):
    """``node[v] = sum_{e: dst[e]=v} msg[e]`` in the dtype of ``msg``."""
    out = torch.zeros((num_nodes,) + msg.shape[1:], dtype=msg.dtype)
    return out.index_add_(0, dst, msg)


# ---- structural restatement of the reference CPU path ------------------------------------------------------
def _tt(v, dtype=None):
    return None if v is None else torch.tensor(v, dtype=dtype)


def tables_to_torch(info: dict, float_dtype=torch.float32) -> dict:
    """Lists of ``oracle.ref_tables`` -> tensors as ``torch.tensor(list)`` makes them in the reference."""
    out = {}
    for k, v in info.items():
        if isinstance(v, dict):
            out[k] = tables_to_torch(v, float_dtype)
        elif isinstance(v, list):
            # coefficient lists ("scale" of the product tables, "scale_MM0" / "scales_ii0" of the channel-mixing tables)
            # are floating point, everything else an index
            out[k] = torch.tensor(v, dtype=float_dtype if k.startswith("scale") else torch.int64)
        else:
            out[k] = v
    return out


def segment_csr(src: torch.Tensor, ptr: torch.Tensor, dim: int) -> torch.Tensor:
    """Sum of ``src`` over ``[ptr[i], ptr[i+1])`` along ``dim`` (what PyG's ``segment(src, ptr[None])`` does)."""
    n_seg = ptr.shape[0] - 1
    ids = torch.repeat_interleave(torch.arange(n_seg), ptr[1:] - ptr[:-1])
    shape = list(src.shape)
    shape[dim] = n_seg
    # entries past the last pointer belong to no segment (the reference's builders can leave some behind,
    # equitorch/utils/_structs.py:105-123); a pointer-driven sum never reads them
    src = src.narrow(dim, int(ptr[0]), int(ptr[-1]) - int(ptr[0]))
    return torch.zeros(shape, dtype=src.dtype).index_add_(dim, ids, src)


def cpu_mul(x, y, info, out_accumulated=False):
    """``indexed_mul_scale_gather_cpu`` (batched_sparse_dense_op.py:234-275)."""
    if info["index1"] is not None:
        x = x.index_select(-2, info["index1"])
    if info["index2"] is not None:
        y = y.index_select(-2, info["index2"])
    inter = x * y
    if info["scale"] is not None:
        inter = inter * info["scale"].unsqueeze(-1)
    if info["seg_out"] is not None:
        inter = segment_csr(inter, info["seg_out"], inter.ndim - 2)
    return inter.sum(0) if out_accumulated else inter


def cpu_vecsca(x, y, info, out_accumulated=False):
    """``indexed_vecsca_scale_gather_cpu`` (:1752-1794): x vector, y scalar."""
    if info["index1"] is not None:
        x = x.index_select(-2, info["index1"])
    if info["index2"] is not None:
        y = y.index_select(-1, info["index2"])
    inter = x * y.unsqueeze(-1)
    if info["scale"] is not None:
        inter = inter * info["scale"].unsqueeze(-1)
    if info["seg_out"] is not None:
        inter = segment_csr(inter, info["seg_out"], inter.ndim - 2)
    return inter.sum(0) if out_accumulated else inter


def cpu_scavec(x, y, info, out_accumulated=False):
    """``indexed_scavec_scale_gather`` (:994-1035): operands and their index columns swapped into vecsca."""
    swapped = dict(info, index1=info["index2"], index2=info["index1"])
    return cpu_vecsca(y, x, swapped, out_accumulated)


def cpu_inner(x, y, info, out_accumulated=False):
    """``indexed_inner_scale_gather_cpu`` (:790-831)."""
    if info["index1"] is not None:
        x = x.index_select(-2, info["index1"])
    if info["index2"] is not None:
        y = y.index_select(-2, info["index2"])
    inter = (x * y).sum(-1)
    if info["scale"] is not None:
        inter = inter * info["scale"]
    if info["seg_out"] is not None:
        inter = segment_csr(inter, info["seg_out"], inter.ndim - 1)
    return inter.sum(0) if out_accumulated else inter


def cpu_outer(x, y, info, out_accumulated=False):
    """``indexed_outer_scale_gather_cpu`` (batched_sparse_dense_op.py:515-556): ``x (.., M1, U)``, ``y (.., M2, V)``
    -> ``(.., M, U, V)``."""
    if info["index1"] is not None:
        x = x.index_select(-2, info["index1"])
    if info["index2"] is not None:
        y = y.index_select(-2, info["index2"])
    inter = x.unsqueeze(-1) * y.unsqueeze(-2)
    if info["scale"] is not None:
        inter = inter * info["scale"].view(-1, 1, 1)
    if info["seg_out"] is not None:
        inter = segment_csr(inter, info["seg_out"], inter.ndim - 3)
    return inter.sum(0) if out_accumulated else inter


def cpu_vecmat(x, y, info, out_accumulated=False):
    """``indexed_vecmat_scale_gather_cpu`` (:1461-1509): ``x (.., M1, U)`` vector, ``y (.., M2, U, V)`` matrix
    -> ``(.., M, V)``."""
    if info["index1"] is not None:
        x = x.index_select(-2, info["index1"])
    if info["index2"] is not None:
        y = y.index_select(-3, info["index2"])
    inter = torch.einsum("...ti,...tij->...tj", x, y)
    if info["scale"] is not None:
        inter = inter * info["scale"].unsqueeze(-1)
    if info["seg_out"] is not None:
        inter = segment_csr(inter, info["seg_out"], inter.ndim - 2)
    return inter.sum(0) if out_accumulated else inter


def cpu_mat_t_vec(x, y, info, out_accumulated=False):
    """``indexed_mat_t_vec_scale_gather`` (:1200-1238): matrix first, vector second; calls vecmat with the operands
    and their index columns exchanged."""
    swapped = dict(info, index1=info["index2"], index2=info["index1"])
    return cpu_vecmat(y, x, swapped, out_accumulated)


def cpu_scale_segment(inp, scale, index, seg):
    """``indexed_scale_segment_cpu`` (indexed_scale_segment_op.py:143-170)."""
    if index is not None:
        inp = inp.index_select(-2, index)
    if scale is not None:
        inp = inp * scale.unsqueeze(-1)
    if seg is not None:
        inp = segment_csr(inp, seg, inp.ndim - 2)
    return inp


def cpu_u1u_forward(x, y, w, tp_fwd):
    """``TensorProductU1UDummy.forward`` (nn/functional/linears.py:24-25) -> (ret, inter)."""
    inter = cpu_vecsca(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_mul(inter, w, tp_fwd["info_M_fwd"]), inter


def cpu_1uu_forward(x, y, w, tp_fwd):
    """``TensorProduct1UUDummy.forward`` (:104-105): x scalar, y vector."""
    inter = cpu_scavec(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_mul(inter, w, tp_fwd["info_M_fwd"])


def cpu_uu1_forward(x, y, w, tp_fwd):
    """``TensorProductUU1Dummy.forward`` (:184-185): both vectors, inner product with the weight."""
    inter = cpu_mul(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_inner(inter, w, tp_fwd["info_M_fwd"])


def cpu_u1u_backward(g, x, y, w, inter, tp_fwd, tp_bwd1, tp_bwd2):
    """First-order part of ``TensorProductU1UDummy.backward`` (:44-83); the ``grad_inter`` terms vanish."""
    gx = cpu_1uu_forward(y, g, w, tp_bwd1)
    gy = cpu_uu1_forward(g, x, w, tp_bwd2)
    gw = cpu_mul(g, inter, tp_fwd["info_M_bwd2"], out_accumulated=(w.ndim == 2))
    return gx, gy, gw


# fully connected family: ``TensorProductU1VDummy`` and siblings (nn/functional/linears.py:254-492) and
# ``TensorProductUVWDummy`` (nn/functional/tensor_products.py:92-172), first-order parts
def cpu_sparse_scale(x, info):
    """``sparse_scale`` (nn/functional/sparse_scale.py:14-46) on a table dict with ``scale / index / seg_out``."""
    return cpu_scale_segment(x, info["scale"], info["index"], info["seg_out"])


def cpu_u1v_forward(x, y, w, tp_fwd):
    """``TensorProductU1VDummy.forward`` (linears.py:257-280): vecsca then vecmat -> (ret, inter)."""
    inter = cpu_vecsca(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_vecmat(inter, w, tp_fwd["info_M_fwd"]), inter


def cpu_1vu_forward(x, y, w, tp_fwd):
    """``TensorProduct1VUDummy.forward`` (:341-344): x channel-less, y carries the input channels."""
    inter = cpu_scavec(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_vecmat(inter, w, tp_fwd["info_M_fwd"]), inter


def cpu_vu1_forward(x, y, w, tp_fwd):
    """``TensorProductVU1Dummy.forward`` (:419-422): weight first (``info_kM1j``), inner product with the second
    operand (``info_kM1M2``), then the coefficient sum (``info_M_kM1M2``)."""
    inter = cpu_vecmat(x, w, tp_fwd["info_kM1j_fwd"])
    inter = cpu_inner(inter, y, tp_fwd["info_kM1M2_fwd"])
    return cpu_sparse_scale(inter.unsqueeze(-1), tp_fwd["info_M_kM1M2_fwd"]).squeeze(-1)


def cpu_u1v_backward(g, x, y, w, inter, tp_fwd, tp_bwd1, tp_bwd2):
    """First-order part of ``TensorProductU1VDummy.backward`` (:282-324)."""
    wt = w.transpose(-1, -2).contiguous()
    gx, _ = cpu_1vu_forward(y, g, wt, tp_bwd1)
    gy = cpu_vu1_forward(g, x, wt, tp_bwd2)
    gw = cpu_outer(g, inter, tp_fwd["info_M_bwd2"], out_accumulated=(w.ndim == 3)).transpose(-1, -2).contiguous()
    return gx, gy, gw


def cpu_uvw_forward(x, y, w, tp_fwd):
    """``TensorProductUVWDummy.forward`` (tensor_products.py:95-101): outer product of the operands' channels, then
    vecmat with the weight flattened over (u, v) -> (ret, inter)."""
    inter = cpu_outer(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_vecmat(inter.flatten(-2), w.flatten(-3, -2), tp_fwd["info_M_fwd"]), inter


def cpu_uvw_backward(g, x, y, w, inter, tp_fwd, tp_bwd1, tp_bwd2):
    """First-order part of ``TensorProductUVWDummy.backward`` (:120-161)."""
    lead = tuple(range(w.ndim - 3))
    gx, _ = cpu_uvw_forward(y, g, w.permute(*lead, -2, -1, -3).contiguous(), tp_bwd1)
    gy, _ = cpu_uvw_forward(g, x, w.permute(*lead, -1, -3, -2).contiguous(), tp_bwd2)
    gw = cpu_outer(g, inter.flatten(-2), tp_fwd["info_M_bwd2"], out_accumulated=(w.ndim == 4))
    gw = gw.transpose(-1, -2).contiguous().unflatten(-2, w.shape[-3:-1])
    return gx, gy, gw


def cpu_uuu_forward(x, y, w, tp_fwd):
    """``TensorProductUUUDummy.forward`` (tensor_products.py:12-18): both operands and the weight per channel."""
    inter = cpu_mul(x, y, tp_fwd["info_Mij_fwd"])
    return cpu_mul(inter, w, tp_fwd["info_M_fwd"]), inter


def cpu_edge_forward(x, sh, w, src, perm, ptr, tp_fwd):
    """``x.index_select(0, src)`` -> u1u -> ``indexed_scale_segment(msg.view(1,E,-1), None, perm, ptr)``."""
    msg, inter = cpu_u1u_forward(x.index_select(0, src), sh, w, tp_fwd)
    e, d, c = msg.shape
    out = cpu_scale_segment(msg.view(1, e, d * c), None, perm, ptr)
    return out.view(-1, d, c), inter


def cpu_edge_backward(ct, x, sh, w, inter, src, dst, tp_fwd, tp_bwd1, tp_bwd2):
    """Transposed direction: gather the cotangent at dst, TP backward per edge, scatter grad_x to src."""
    g = ct.index_select(0, dst)
    gxs, gy, gw = cpu_u1u_backward(g, x.index_select(0, src), sh, w, inter, tp_fwd, tp_bwd1, tp_bwd2)
    gx = torch.zeros_like(x).index_add_(0, src, gxs)
    return gx, gy, gw


# ---- irreps-preserving channel mixing ------------------------------------------------------------------------
def cpu_irreps_linear(x, w, info):
    """``IrrepsLinear.forward`` (equitorch/nn/functional/linears.py:533-546): per table entry the vector-matrix
    product ``scale * x[n, M0] @ W[(n,) path]`` summed over the entries of each output segment
    (``indexed_vecmat_scale_segment``), then scattered to the rows ``M_out`` of a zero ``(N, out_size, C_out)``.
    ``info``: dict from ``ref_tables.irreps_linear_infos``; float64 loops, small cases only."""
    n = x.shape[0]
    seg = torch.zeros(n, len(info["M_out"]), w.shape[-1], dtype=x.dtype)
    ptr = info["M_seg_MM0"]
    for s in range(len(ptr) - 1):
        for t in range(ptr[s], ptr[s + 1]):
            wp = w[info["ii0_MM0"][t]] if w.ndim == 3 else w[:, info["ii0_MM0"][t]]
            vec = x[:, info["M0_MM0"][t], :]
            prod = vec @ wp if w.ndim == 3 else torch.einsum("nu,nuw->nw", vec, wp)
            seg[:, s] = seg[:, s] + info["scale_MM0"][t] * prod
    out = torch.zeros(n, info["out_size"], w.shape[-1], dtype=x.dtype)
    return out.index_add(1, torch.tensor(info["M_out"], dtype=torch.int64), seg)


def cpu_irrep_wise_linear(x, w, info):
    """``IrrepWiseLinear.forward`` (equitorch/nn/functional/linears.py:497-509): ``sparse_vecmat`` with
    ``index2 = irrep_index``: ``out[n, M] = x[n, M] @ W[(n,) irrep_index[M]]``."""
    rows = []
    for M, i in enumerate(info["irrep_index"]):
        rows.append(x[:, M, :] @ w[i] if w.ndim == 3 else torch.einsum("nu,nuw->nw", x[:, M, :], w[:, i]))
    return torch.stack(rows, dim=1)


# ---- gates, norms, RMS normalisation (pure torch float64; autograd gives the gradient oracle) -----------------
def _block_sum(t, seg):
    """``torch_geometric.utils.segment(t, ptr)`` along dim -2, as a slice-and-sum (cf. ``segment_csr`` above)."""
    return torch.stack([t[..., seg[i]:seg[i + 1], :].sum(dim=-2) for i in range(len(seg) - 1)], dim=-2)


def cpu_gating(x, gates, info):
    """``gating`` (equitorch/nn/functional/activations.py:9-35): ``x[n, M, c] * gates[(n,) irrep_index[M], c]``."""
    idx = torch.tensor(info["irrep_index"], dtype=torch.int64)
    return x * gates.index_select(-2, idx)


def cpu_squared_norm(x, info, scaled=True):
    """``SquaredNorm.forward`` (equitorch/nn/functional/norm.py:22-37)."""
    out = _block_sum(x.pow(2), info["irrep_seg"])
    return out * torch.tensor(info["rdims"], dtype=x.dtype).unsqueeze(-1) if scaled else out


def cpu_tensor_dot(x1, x2, info, scaled=True):
    """``TensorDotUU.forward`` (equitorch/nn/functional/tensor_products.py:176-198): the products summed over the
    components of each irrep, times ``dim^-1/2`` when ``scaled``.  Pinned in tests/test_oracle_norms.py by the
    per-block dot product written out with slices and by ``dot(x, x) = squared norm``."""
    out = _block_sum(x1 * x2, info["irrep_seg"])
    return out * torch.tensor(info["rsqrt_dims"], dtype=out.dtype).unsqueeze(-1) if scaled else out


def cpu_norm(x, info, scaled=True):
    """``Norm.forward`` (:80-98); its backward (:100-126) puts a zero gradient at zero blocks."""
    out = torch.sqrt(_block_sum(x.pow(2), info["irrep_seg"]))
    return out * torch.tensor(info["rsqrt_dims"], dtype=x.dtype).unsqueeze(-1) if scaled else out


def cpu_channel_mean_squared_norm(x, info, scaled=True):
    """``ChannelMeanSquaredNorm.forward`` (:139-160)."""
    out = _block_sum(x.pow(2), info["irrep_seg"]).sum(dim=-1) / x.shape[-1]
    return out * torch.tensor(info["rdims"], dtype=x.dtype) if scaled else out


def cpu_batch_mean_squared_norm(x, info, scaled=True):
    """``BatchMeanSquaredNorm.forward`` (:200-224)."""
    out = _block_sum(x.pow(2), info["irrep_seg"]).sum(dim=0) / x.shape[0]
    return out * torch.tensor(info["rdims"], dtype=x.dtype).unsqueeze(-1) if scaled else out


def cpu_batch_rms_norm(x, running, info, weight=None, scaled=True, training=False, momentum=0.1, eps=1e-5):
    """``batch_rms_norm`` (equitorch/nn/functional/normalization.py:10-72) -> (output, updated running statistic)."""
    if training:
        stat = cpu_squared_norm(x, info, scaled).mean(dim=0)
        running = torch.lerp(running, stat.detach(), momentum)
    else:
        stat = running
    scale = torch.rsqrt(stat + eps)
    if weight is not None:
        scale = weight * scale
    return cpu_gating(x, scale, info), running


def cpu_layer_rms_norm(x, info, weight=None, scaled=True, eps=1e-5):
    """``layer_rms_norm`` (:75-118)."""
    rsigma = torch.rsqrt(cpu_channel_mean_squared_norm(x, info, scaled) + eps)
    idx = torch.tensor(info["irrep_index"], dtype=torch.int64)
    out = x * rsigma.index_select(-1, idx).unsqueeze(-1)
    return out if weight is None else cpu_gating(out, weight, info)


# ---- rotations and the SO(2) linear layer --------------------------------------------------------------------
def _product_entries(info):
    """(out, i1, i2, scale) per entry of a ``sparse_product_info`` dict (None index = identity)."""
    n = len(info["scale"])
    i1 = info["index1"] if info["index1"] is not None else list(range(n))
    i2 = info["index2"] if info["index2"] is not None else list(range(n))
    seg = info["seg_out"] if info["seg_out"] is not None else list(range(n + 1))
    out = [m for m in range(len(seg) - 1) for _ in range(seg[m], seg[m + 1])]
    return list(zip(out, i1, i2, info["scale"]))


def cpu_z_rotation(x, cs, info):
    """``sparse_vecsca(x, cs, rotate_z_info_fwd)`` (equitorch/nn/functional/wigner_d.py:34-37):
    ``out[n, M, c] = sum_t scale_t x[n, i1_t, c] cs[n, i2_t]``."""
    rows = [torch.zeros_like(x[:, 0]) for _ in range(info["out_size"])]
    for o, i1, i2, s in _product_entries(info):
        rows[o] = rows[o] + s * x[:, i1] * cs[:, i2, None]
    return torch.stack(rows, dim=1)


def cpu_j(x, info):
    """``sparse_scale(x, j_matrix_info)``: ``out[n, M] = sum_{t in seg M} scale_t x[n, index_t]``."""
    seg, idx, sc = info["seg_out"], info["index"], info["scale"]
    n = len(sc)
    seg = seg if seg is not None else list(range(n + 1))       # the builders store an identity as None
    idx = idx if idx is not None else list(range(n))
    return torch.stack([sum(sc[t] * x[:, idx[t]] for t in range(seg[m], seg[m + 1])) for m in range(len(seg) - 1)],
                       dim=1)


def cpu_wigner_rotation(x, sc_alpha, sc_beta, sc_gamma, z_info, j_info):
    """``sparse_wigner_rotation`` (equitorch/nn/functional/wigner_d.py:14-56): Z(alpha) J Z(beta) J Z(gamma) x."""
    if sc_gamma is not None:
        x = cpu_z_rotation(x, sc_gamma, z_info)
    if sc_beta is not None:
        x = cpu_j(cpu_z_rotation(cpu_j(x, j_info), sc_beta, z_info), j_info)
    if sc_alpha is not None:
        x = cpu_z_rotation(x, sc_alpha, z_info)
    return x


def cpu_sincos(angle, max_m):
    """``sincos`` (equitorch/nn/functional/angular.py): [1, sin a, cos a, sin 2a, cos 2a, ...]."""
    cols = [torch.ones_like(angle)]
    for m in range(1, max_m + 1):
        cols += [torch.sin(m * angle), torch.cos(m * angle)]
    return torch.stack(cols, dim=-1)


def cpu_so2_linear(x, w, info, per_sample=False):
    """``SO2Linear.forward`` (equitorch/nn/linears.py:495-507): ``sparse_mul`` for a channel-wise weight
    ``((N,) num_weights, C)``, ``sparse_vecmat`` for ``((N,) num_weights, C_in, C_out)``."""
    rows = [None] * info["out_size"]
    matrix = w.ndim - int(per_sample) == 3
    for o, i1, i2, s in _product_entries(info):
        wt = w[:, i2] if per_sample else w[i2]
        if not matrix:
            term = s * x[:, i1] * wt
        else:
            term = s * (torch.einsum("nu,nuw->nw", x[:, i1], wt) if per_sample else x[:, i1] @ wt)
        rows[o] = term if rows[o] is None else rows[o] + term
    # a row no entry reaches is zero; a table none of whose entries is reachable gives zeros that still hang on the
    # operands (the reference's kernel returns its zero-filled output and zero gradients)
    blank = 0.0 * (x[:, 0, :1] * (w[:, 0].flatten(1)[:, :1] if per_sample else w[0].reshape(-1)[:1]))
    blank = blank.expand(x.shape[0], w.shape[-1])
    return torch.stack([r if r is not None else blank for r in rows], dim=1)
