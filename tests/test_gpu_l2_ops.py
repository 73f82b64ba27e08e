"""The operator-level drop-in signature, called as the reference's callers call it
(``equitorch/ops/batched_sparse_dense_op.py:277-299`` and siblings):

    indexed_<op>_scale_gather(input1, input2, scale, index1, index2, seg, gather_index, index_out, out,
                              out_accumulated, out_size)

for the seven members, against the oracle's restatement of the reference's CPU functions.  Covered here and nowhere
else: the positional table arguments instead of a ``SparseProductInfo``, ``out=``, an ``out_size`` larger than the
number of segments, operands of different precision (the result takes ``torch.result_type``), the ``(N, M1, 1)``
form of the channel-less operand of ``scavec``, and ``gather_index`` / ``index_out``."""
import itertools

import pytest
import torch

from helpers import assert_close, stable_seed
from oracle import ref_ops, ref_tables

pytestmark = pytest.mark.gpu

# name: (oracle, axes of input1, axes of input2, axes of the result)
OPS = {
    "mul": (ref_ops.cpu_mul, "u", "u", "u"),
    "vecsca": (ref_ops.cpu_vecsca, "u", "", "u"),
    "scavec": (ref_ops.cpu_scavec, "", "u", "u"),
    "inner": (ref_ops.cpu_inner, "u", "u", ""),
    "outer": (ref_ops.cpu_outer, "u", "w", "uw"),
    "vecmat": (ref_ops.cpu_vecmat, "u", "uw", "w"),
    "mat_t_vec": (ref_ops.cpu_mat_t_vec, "uw", "u", "w"),
}
EXT = {"u": 21, "w": 12}
N, D = 37, 15


@pytest.fixture(scope="module")
def table13(device):
    """``info_Mij_fwd`` of Irreps((1, 3)) x Irreps((1, 3)) -> Irreps((1, 3)): the table of the reference's own
    operator sweep (test/test_op/test_sparse_structs.py:668-675), as the oracle builds it and as device tensors."""
    ref = ref_ops.tables_to_torch(ref_tables.tp_infos((1, 3), (1, 3), (1, 3))[0], torch.float64)["info_Mij_fwd"]
    ref = dict(ref, scale=ref["scale"].float().double())      # the reference stores fp32 coefficients
    dev = {k: (None if v is None else (v.float() if v.is_floating_point() else v).to(device))
           for k, v in ref.items() if k in ("scale", "index1", "index2", "seg_out")}
    return ref, dev


def _operand(axes, shared, gen, dtype=torch.float64):
    shape = (() if shared else (N,)) + (D,) + tuple(EXT[a] for a in axes)
    return torch.randn(*shape, generator=gen, dtype=torch.float64).float().to(dtype)


def _call(op, x, y, dev, **kw):
    from equitorch_amd import ops
    fn = getattr(ops, f"indexed_{op}_scale_gather")
    return fn(x, y, dev["scale"], dev["index1"], dev["index2"], dev["seg_out"], **kw)


@pytest.mark.parametrize("op", sorted(OPS))
@pytest.mark.parametrize("shared1,shared2,acc", [s for s in itertools.product([False, True], repeat=3)
                                                 if not (s[0] and s[1])])
def test_positional_signature_against_the_cpu_functions(device, table13, op, shared1, shared2, acc):
    ref, dev = table13
    oracle, ax1, ax2, _ = OPS[op]
    gen = torch.Generator().manual_seed(stable_seed("l2", op, shared1, shared2, acc))
    x, y = _operand(ax1, shared1, gen), _operand(ax2, shared2, gen)
    want = oracle(x, y, ref, out_accumulated=acc)
    got = _call(op, x.float().to(device), y.float().to(device), dev, out_accumulated=acc)
    assert got.dtype == torch.float32 and got.shape == want.shape
    # accumulated results are sums over the 37 rows, the others over at most 13 coefficients: element-wise bound
    assert_close(got, want, 1e-5, f"indexed_{op}_scale_gather shared=({shared1},{shared2}) accumulated={acc}")


@pytest.mark.parametrize("op", sorted(OPS))
@pytest.mark.parametrize("acc", [False, True])
def test_out_argument_and_padded_out_size(device, table13, op, acc):
    """``out=`` receives the result and is what the call returns; with ``out_size`` beyond the number of segments the
    rows past the last segment are zero (the reference allocates ``zeros`` when accumulating and ``empty``
    otherwise, ``batched_sparse_dense_op.py:190-203``: zeros are within both)."""
    ref, dev = table13
    oracle, ax1, ax2, _ = OPS[op]
    gen = torch.Generator().manual_seed(stable_seed("l2 out", op, acc))
    x, y = _operand(ax1, False, gen), _operand(ax2, False, gen)
    want = oracle(x, y, ref, out_accumulated=acc)
    n_seg = ref["seg_out"].shape[0] - 1
    xd, yd = x.float().to(device), y.float().to(device)
    # stored into when per row (any previous content is overwritten), added onto when accumulated
    buf = torch.full(want.shape, 0.0 if acc else float("nan"), dtype=torch.float32, device=device)
    ret = _call(op, xd, yd, dev, out=buf, out_accumulated=acc)
    assert ret is buf
    assert_close(buf, want, 1e-5, f"indexed_{op}_scale_gather out=")
    padded = _call(op, xd, yd, dev, out_accumulated=acc, out_size=n_seg + 3)
    dim = 0 if acc else 1
    assert padded.shape[dim] == n_seg + 3
    assert_close(padded.narrow(dim, 0, n_seg), want, 1e-5, f"indexed_{op}_scale_gather out_size, leading rows")
    assert torch.count_nonzero(padded.narrow(dim, n_seg, 3)) == 0


@pytest.mark.parametrize("op", sorted(OPS))
def test_mixed_precision_operands_promote(device, table13, op):
    """fp32 x fp64 -> fp64 (``torch.result_type``, reference ``:171``), computed in fp64."""
    ref, dev = table13
    oracle, ax1, ax2, _ = OPS[op]
    gen = torch.Generator().manual_seed(stable_seed("l2 mixed", op))
    x, y = _operand(ax1, False, gen), _operand(ax2, False, gen)
    got = _call(op, x.float().to(device), y.to(device), dev)
    assert got.dtype == torch.float64
    assert_close(got, oracle(x, y, ref), 1e-11, f"indexed_{op}_scale_gather fp32 x fp64")


def test_scavec_takes_the_scalar_operand_with_a_unit_channel_axis(device, table13):
    ref, dev = table13
    gen = torch.Generator().manual_seed(stable_seed("l2 scalar form"))
    x, y = _operand("", False, gen), _operand("u", False, gen)
    want = ref_ops.cpu_scavec(x, y, ref)
    got = _call("scavec", x.float().to(device).unsqueeze(-1), y.float().to(device), dev)
    assert_close(got, want, 1e-5, "indexed_scavec_scale_gather (N, M1, 1)")


def test_identity_tables(device, table13):
    """No index, no segment pointer: entry t of the result is ``scale[t] * x[t] * y[t]`` (the reference collapses
    identity tables to None, utils/_indices.py:111-126)."""
    from equitorch_amd import ops
    _, dev = table13
    gen = torch.Generator().manual_seed(stable_seed("l2 identity"))
    x, y = _operand("u", False, gen), _operand("u", False, gen)
    scale = torch.randn(D, generator=gen, dtype=torch.float64).float()
    got = ops.indexed_mul_scale_gather(x.float().to(device), y.float().to(device), scale.to(device))
    assert_close(got, x * y * scale.double()[None, :, None], 1e-5, "indexed_mul_scale_gather, identity table")


@pytest.mark.parametrize("op", sorted(OPS))
@pytest.mark.parametrize("acc", [False, True])
def test_gather_index_and_index_out(device, table13, op, acc):
    """``gather_index`` maps a position inside a segment to the table entry it uses (reference kernel ``:103-106``) and
    ``index_out`` a segment to the output row it is written to (``:138-144``).  Built here from the sweep's table:
    its entries stored in a shuffled order with ``gather_index`` undoing the shuffle, and its segments sent to a
    permutation of the rows of a larger output — the result must be the unshuffled table's, rows permuted, the
    rows no segment names zero."""
    ref, dev = table13
    oracle, ax1, ax2, _ = OPS[op]
    gen = torch.Generator().manual_seed(stable_seed("l2 gather", op, acc))
    x, y = _operand(ax1, False, gen), _operand(ax2, False, gen)
    want = oracle(x, y, ref, out_accumulated=acc)
    nnz, n_seg = ref["scale"].shape[0], ref["seg_out"].shape[0] - 1
    shuffle = torch.randperm(nnz, generator=gen)
    inverse = torch.empty_like(shuffle)
    inverse[shuffle] = torch.arange(nnz)
    stored = {k: dev[k][shuffle.to(device)] for k in ("scale", "index1", "index2")}     # entry shuffle[t] at place t
    rows = torch.randperm(n_seg + 4, generator=gen)[:n_seg]
    from equitorch_amd import ops
    got = getattr(ops, f"indexed_{op}_scale_gather")(
        x.float().to(device), y.float().to(device), stored["scale"], stored["index1"], stored["index2"],
        dev["seg_out"], gather_index=inverse.to(device), index_out=rows.to(device), out_accumulated=acc,
        out_size=n_seg + 4)
    dim = 0 if acc else 1
    assert got.shape[dim] == n_seg + 4
    assert_close(got.index_select(dim, rows.to(device)), want, 1e-5, f"indexed_{op}_scale_gather gather_index/index_out")
    unused = torch.tensor(sorted(set(range(n_seg + 4)) - set(rows.tolist())), device=device)
    assert torch.count_nonzero(got.index_select(dim, unused)) == 0


def test_accumulated_out_argument_is_added_to(device, table13):
    """With ``out_accumulated`` the reference's kernels add onto ``out`` (``kernel_utils.py:139-155``: atomic add);
    without, they store the segments' rows and leave any further row of ``out`` alone."""
    ref, dev = table13
    gen = torch.Generator().manual_seed(stable_seed("l2 out add"))
    x, y = _operand("u", False, gen), _operand("u", False, gen)
    n_seg = ref["seg_out"].shape[0] - 1
    base = torch.randn(n_seg, EXT["u"], generator=gen, dtype=torch.float64).float()
    buf = base.clone().to(device)
    _call("mul", x.float().to(device), y.float().to(device), dev, out=buf, out_accumulated=True)
    assert_close(buf, base.double() + ref_ops.cpu_mul(x, y, ref, out_accumulated=True), 1e-5, "accumulated onto out")
    tall = torch.full((N, n_seg + 2, EXT["u"]), 7.0, device=device)
    _call("mul", x.float().to(device), y.float().to(device), dev, out=tall)
    assert_close(tall[:, :n_seg], ref_ops.cpu_mul(x, y, ref), 1e-5, "stored into the leading rows of out")
    assert bool((tall[:, n_seg:] == 7.0).all())
