"""The gate / norm / RMS-normalisation oracle pinned on the CPU against formulas written out by hand."""
import torch

from oracle import ref_ops, ref_tables


def test_norm_oracle_against_hand_written_blocks():
    info = ref_tables.irreps_info("0e+1o+2e")
    g = torch.Generator().manual_seed(0)
    x = torch.randn(6, 9, 5, generator=g, dtype=torch.float64)
    blocks = [x[:, 0:1], x[:, 1:4], x[:, 4:9]]
    sq = torch.stack([b.pow(2).sum(1) for b in blocks], dim=1)
    dims = torch.tensor([1.0, 3.0, 5.0], dtype=torch.float64)
    torch.testing.assert_close(ref_ops.cpu_squared_norm(x, info, False), sq)
    torch.testing.assert_close(ref_ops.cpu_squared_norm(x, info, True), sq / dims[:, None])
    torch.testing.assert_close(ref_ops.cpu_norm(x, info, False)[:, 1], torch.linalg.vector_norm(x[:, 1:4], dim=1))
    torch.testing.assert_close(ref_ops.cpu_norm(x, info, True), sq.sqrt() / dims.sqrt()[:, None])
    torch.testing.assert_close(ref_ops.cpu_channel_mean_squared_norm(x, info, True), sq.mean(-1) / dims)
    torch.testing.assert_close(ref_ops.cpu_batch_mean_squared_norm(x, info, True), sq.mean(0) / dims[:, None])


def test_gate_and_normalisation_oracle_properties():
    info = ref_tables.irreps_info("0e+1o+2e")
    g = torch.Generator().manual_seed(1)
    x = torch.randn(7, 9, 4, generator=g, dtype=torch.float64)
    gate = torch.randn(7, 3, 4, generator=g, dtype=torch.float64)
    out = ref_ops.cpu_gating(x, gate, info)
    torch.testing.assert_close(out[:, 1:4], x[:, 1:4] * gate[:, 1:2])
    torch.testing.assert_close(out[:, 4:9], x[:, 4:9] * gate[:, 2:3])
    # after layer normalisation every block has channel-mean squared norm 1 (eps -> 0), for any input scale
    y = ref_ops.cpu_layer_rms_norm(3.7 * x, info, eps=0.0)
    torch.testing.assert_close(ref_ops.cpu_channel_mean_squared_norm(y, info, True), torch.ones(7, 3, dtype=torch.float64))
    # after batch normalisation in training mode every (block, channel) has batch-mean squared norm 1
    z, running = ref_ops.cpu_batch_rms_norm(x, torch.ones(3, 4, dtype=torch.float64), info, training=True, eps=0.0,
                                            momentum=0.25)
    torch.testing.assert_close(ref_ops.cpu_batch_mean_squared_norm(z, info, True), torch.ones(3, 4, dtype=torch.float64))
    stat = ref_ops.cpu_batch_mean_squared_norm(x, info, True)
    torch.testing.assert_close(running, 0.75 * torch.ones(3, 4, dtype=torch.float64) + 0.25 * stat)


def test_tensor_dot_oracle_against_hand_written_blocks():
    info = ref_tables.irreps_info("0e+1o+2e")
    g = torch.Generator().manual_seed(2)
    x = torch.randn(6, 9, 5, generator=g, dtype=torch.float64)
    y = torch.randn(6, 9, 5, generator=g, dtype=torch.float64)
    dots = torch.stack([(x[:, a:b] * y[:, a:b]).sum(1) for a, b in ((0, 1), (1, 4), (4, 9))], dim=1)
    dims = torch.tensor([1.0, 3.0, 5.0], dtype=torch.float64)
    torch.testing.assert_close(ref_ops.cpu_tensor_dot(x, y, info, False), dots)
    torch.testing.assert_close(ref_ops.cpu_tensor_dot(x, y, info, True), dots / dims.sqrt()[:, None])
    torch.testing.assert_close(ref_ops.cpu_tensor_dot(x, x, info, False), ref_ops.cpu_squared_norm(x, info, False))
    # the l = 1 block is the Euclidean dot product of the two vectors, whatever the component order
    torch.testing.assert_close(ref_ops.cpu_tensor_dot(x, y, info, False)[:, 1],
                               torch.einsum("nmc,nmc->nc", x[:, 1:4], y[:, 1:4]))
