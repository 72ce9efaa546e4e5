"""GPU parity of the interleaved [E][T][D] layout (the older sparse_embedding_cuda interface)
against the CPU oracle, through the module mirror as in test_sparse_embedding_cuda.py:12-135."""
import numpy as np
import pytest
import torch

from gpu_util import DEV, assert_close, dev

import sparse_embedding_cuda as se
import sparse_embedding_cuda_ops as se_ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("E,T,D,B,L", [(1000, 4, 32, 16, 7), (50, 1, 4, 3, 2), (300, 3, 128, 33, 20),
                                       (64, 5, 12, 9, 4)])
def test_dense_and_offsets_variants_match_oracle(oracle, E, T, D, B, L):
    rs = np.random.RandomState(E + T)
    weights = rs.randn(E, T, D).astype(np.float32)
    dense = (rs.zipf(1.2, size=(B, T, L)) % E).astype(np.int32)
    offsets = np.arange(0, B * T * L + 1, L, dtype=np.int32)
    go = rs.randn(B, T, D).astype(np.float32)
    want = oracle.forward_etd(weights, dense.reshape(-1), offsets)
    w_ref = weights.copy()
    oracle.backward_etd(go, w_ref, dense.reshape(-1), offsets, 0.05)

    cc = se_ops.UniformShardedEmbeddingBags(T, E, D).cuda()
    cc.embedding_weights.data.copy_(dev(weights))
    out = cc(dev(dense))
    assert tuple(out.shape) == (B, T, D)
    assert_close(out.detach().cpu().numpy(), want, 1e-5)
    out.backward(dev(go))
    assert_close(cc.embedding_weights.detach().cpu().numpy(), w_ref, 1e-5)

    # merged offsets [B][T+1] as get_merged_offsets_from_dense builds them (:61-72)
    merged = np.fromfunction(lambda b, t: (b * T + t) * L, (B, T + 1), dtype=np.int32).astype(np.int32)
    cc2 = se_ops.UniformShardedEmbeddingBags(T, E, D).cuda()
    cc2.embedding_weights.data.copy_(dev(weights))
    out2 = cc2(dev(dense.reshape(-1)), dev(merged))
    assert torch.equal(out2, out)
    out2.backward(dev(go))
    assert torch.equal(cc2.embedding_weights, cc.embedding_weights)


def test_ragged_offsets_and_function_level_calls(oracle):
    rs = np.random.RandomState(2)
    E, T, D, B = 200, 3, 64, 11
    weights = rs.randn(E, T, D).astype(np.float32)
    lengths = rs.randint(0, 9, size=B * T)
    flat = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    indices = (rs.zipf(1.3, size=int(flat[-1])) % E).astype(np.int32)
    merged = np.stack([flat[b * T:b * T + T + 1] for b in range(B)]).astype(np.int32)
    go = rs.randn(B, T, D).astype(np.float32)
    w = dev(weights)
    got = se.forward_offsets(w, dev(indices), dev(merged))
    assert_close(got.cpu().numpy(), oracle.forward_etd(weights, indices, flat), 1e-5)
    se.backward_update_offsets(dev(go), w, dev(indices), dev(merged), 0.1)
    w_ref = weights.copy()
    oracle.backward_etd(go, w_ref, indices, flat, 0.1)
    torch.cuda.synchronize()
    assert_close(w.cpu().numpy(), w_ref, 1e-5)
    with pytest.raises(NotImplementedError):
        se.forward_all2all(w, w)


@pytest.mark.parametrize("dtype,tol", [(np.float16, 1e-2), (np.float64, 1e-12), (np.float32, 1e-5)])
def test_half_and_double_tables(oracle, dtype, tol):
    """The reference dispatches these kernels over half, float and double
    (sparse_embedding_cuda_kernel.cu:599-882).  An interleaved table set is one table of E*T rows
    whose row ind*T + t is row `ind` of table t, with the bags numbered b*T + t: the expected
    values come from the table-batched oracle on that single table."""
    rs = np.random.RandomState(6)
    E, T, D, B = 150, 4, 24, 13
    weights = (rs.randn(E, T, D) * 0.1).astype(dtype)
    lengths = rs.randint(0, 7, size=B * T)
    flat = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    indices = (rs.zipf(1.3, size=int(flat[-1])) % E).astype(np.int32)
    merged = np.stack([flat[b * T:b * T + T + 1] for b in range(B)]).astype(np.int32)
    go = rs.randn(B, T, D).astype(dtype)
    table_of_lookup = np.repeat(np.arange(B * T) % T, lengths)
    one_table_rows = (indices * T + table_of_lookup).astype(np.int32)
    one_table = weights.reshape(E * T, D).copy()
    zero = np.zeros(1, np.int32)
    want = oracle.forward(one_table, zero, one_table_rows, flat).reshape(B, T, D)
    w = dev(weights)
    got = se.forward_offsets(w, dev(indices), dev(merged))
    assert got.dtype == w.dtype
    assert_close(got.cpu().numpy(), want, tol)
    se.backward_update_offsets(dev(go), w, dev(indices), dev(merged), 0.1)
    oracle.backward("sgd", go.reshape(B * T, 1, D), one_table, zero, one_table_rows, flat, 0.1)
    torch.cuda.synchronize()
    assert_close(w.cpu().numpy().reshape(E * T, D), one_table, tol)


def test_large_ragged_batch_and_layout_query(oracle):
    """More bags than one scan chunk per table (B > 256), empty bags, tables whose lookups differ a
    lot: the pass that puts the batch into table-major order before the sort (offsets scan in
    chunks of 256 bags, permutation of the indices) is exercised across chunk boundaries."""
    import tbe_native
    rs = np.random.RandomState(12)
    E, T, D, B = 500, 7, 32, 1000
    weights = rs.randn(E, T, D).astype(np.float32)
    lengths = rs.randint(0, 6, size=(B, T))
    lengths[:, 2] = 0                      # a table nobody looks up
    lengths[300:600, 4] += 20              # and a busy stretch of another
    flat = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    indices = (rs.zipf(1.2, size=int(flat[-1])) % E).astype(np.int32)
    merged = np.stack([flat[b * T:b * T + T + 1] for b in range(B)]).astype(np.int32)
    go = rs.randn(B, T, D).astype(np.float32)
    w = dev(weights)
    got = se.forward_offsets(w, dev(indices), dev(merged))
    assert_close(got.cpu().numpy(), oracle.forward_etd(weights, indices, flat), 1e-5)
    se.backward_update_offsets(dev(go), w, dev(indices), dev(merged), 0.1)
    w_ref = weights.copy()
    oracle.backward_etd(go, w_ref, indices, flat, 0.1)
    torch.cuda.synchronize()
    assert_close(w.cpu().numpy(), w_ref, 1e-5)
    lay = tbe_native.backward_interleaved_workspace_layout(indices.size, D, tbe_native.DTYPE_F32, T, B)
    plain = tbe_native.backward_workspace_layout(indices.size, D, tbe_native.DTYPE_F32, T)
    assert lay.grad_rows - lay.keys >= indices.size * 4 + (T * B + 1) * 4 and lay.total_bytes > plain.total_bytes


def test_interleaved_step_in_a_graph():
    """Forward and fused update on the interleaved layout only launch kernels (nothing is rewritten
    or allocated besides the output), so a step can be captured and replayed with new indices."""
    rs = np.random.RandomState(3)
    E, T, D, B, L = 400, 5, 64, 40, 6
    w = dev(rs.randn(E, T, D).astype(np.float32))
    w_eager = w.clone()
    x = dev((rs.zipf(1.3, size=(B, T, L)) % E).astype(np.int32))
    go = dev(rs.randn(B, T, D).astype(np.float32))
    stream = torch.cuda.Stream()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):        # sizes this stream's scratch buffer, fills the offsets cache
        warm = w.clone()
        se.forward_fast_single(warm, x)
        se.backward_update_fast_single(go, warm, x, 0.05)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        out = se.forward_fast_single(w, x)
        se.backward_update_fast_single(go, w, x, 0.05)
    for replay in range(3):
        if replay:
            x.copy_(dev((rs.zipf(1.3, size=(B, T, L)) % E).astype(np.int32)))
        graph.replay()
        want = se.forward_fast_single(w_eager, x.clone())
        se.backward_update_fast_single(go, w_eager, x.clone(), 0.05)
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(w, w_eager)
