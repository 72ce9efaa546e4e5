"""Micro-benchmark CLI with the flags of the reference's sparse_embedding_cuda_benchmark.py (:113-120):
--num-tables 64 --num-embeddings 10000 --embedding-dim 32 --batch-size 128 --bag-size 32 --iters 100
[--fp16], plus --alpha / --seed.

The interleaved [E][T][D] layout of the older extension: forward and fused exact-SGD update on
dense [B][T][L] indices ("Fused") and on flat indices with [B][T+1] offsets ("Fused-Offsets"),
each after one warm-up call, `iters` calls between two events on the current stream
(sparse_embedding_cuda_benchmark.py:11-21).  "BW" is the reference's figure, 4 * B * T * L * D / time
for forward and for backward alike (:77-79, :108-110; the factor is 4 whatever the element size).
The same lookups through the table-major kernels are timed beside it ("Table-major").  The
reference's "Fused-Slow" and per-table nn.EmbeddingBag "Baseline" rows have no counterpart here.
One JSON object per measurement goes to stdout.
"""
import json
import logging
import sys

import click
import numpy as np
import torch

import sparse_embedding_cuda
import sparse_embedding_cuda_ops
import table_batched_embeddings


def time_calls(iters, fn):
    fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1.0e-3 / iters


def report(shape, implementation, method, seconds):
    B, T, L, D = shape["B"], shape["T"], shape["L"], shape["D"]
    bw = 4 * B * T * L * D / seconds / 1.0e9
    logging.info("%s %s, B: %d, E: %d, T: %d, D: %d, L: %d, BW: %.2fGB/s, T: %.0fus", method, implementation, B,
                 shape["E"], T, D, L, bw, seconds * 1e6)
    print(json.dumps(dict(shape, time_per_iter=seconds, implementation=implementation, method=method, BW_GBps=bw)))


def run(B, E, T, L, D, iters, fp16, alpha, seed):
    rs = np.random.RandomState(seed)
    cc = sparse_embedding_cuda_ops.UniformShardedEmbeddingBags(T, E, D, fp16=fp16).cuda()
    logging.info("Embedding parameters: %.2fGParam", cc.embedding_weights.numel() / 1.0e9)
    draws = rs.zipf(alpha, size=(B, T, L)) % E if alpha and alpha > 1.0 else rs.randint(0, E, size=(B, T, L))
    x = torch.from_numpy(draws.astype(np.int32)).cuda()
    shape = dict(B=B, E=E, T=T, D=D, L=L, fp16=fp16, alpha=alpha)
    w = cc.embedding_weights.data
    # merged offsets as get_merged_offsets_from_dense builds them (test_sparse_embedding_cuda.py:61-72)
    flat = x.view(-1)
    merged = (torch.arange(B, device="cuda").view(B, 1) * T + torch.arange(T + 1, device="cuda").view(1, T + 1)) * L
    merged = merged.int().contiguous()
    # the same lookups for the table-major kernels: tables [T][E][D], indices [T][B][L]
    w_tm = w.permute(1, 0, 2).contiguous().view(T * E, D)
    x_tm = x.permute(1, 0, 2).contiguous().view(-1)
    off_tm = torch.arange(0, T * B * L + 1, L, dtype=torch.int32, device="cuda")
    to_tm = (torch.arange(T, device="cuda") * E).int()

    y = sparse_embedding_cuda.forward_fast_single(w, x)
    assert torch.equal(y, sparse_embedding_cuda.forward_offsets(w, flat, merged))
    y_tm = table_batched_embeddings.forward(w_tm, to_tm, x_tm, off_tm, None, L, 1, False)
    torch.testing.assert_close(y, y_tm, rtol=1e-2 if fp16 else 1e-5, atol=1e-2 if fp16 else 1e-5)
    report(shape, "Fused", "forward", time_calls(iters, lambda: sparse_embedding_cuda.forward_fast_single(w, x)))
    report(shape, "Fused-Offsets", "forward",
           time_calls(iters, lambda: sparse_embedding_cuda.forward_offsets(w, flat, merged)))
    report(shape, "Table-major", "forward", time_calls(
        iters, lambda: table_batched_embeddings.forward(w_tm, to_tm, x_tm, off_tm, None, L, 1, False)))

    go = torch.rand_like(y)
    report(shape, "Fused", "backward",
           time_calls(iters, lambda: sparse_embedding_cuda.backward_update_fast_single(go, w, x, 0.05)))
    report(shape, "Fused-Offsets", "backward",
           time_calls(iters, lambda: sparse_embedding_cuda.backward_update_offsets(go, w, flat, merged, 0.05)))
    report(shape, "Table-major", "backward", time_calls(
        iters, lambda: table_batched_embeddings.backward_sgd(go, w_tm, to_tm, x_tm, off_tm, 0.05, L, 1, False)))


@click.command()
@click.option("--num-tables", default=64)
@click.option("--num-embeddings", default=int(1e4))
@click.option("--embedding-dim", default=32)
@click.option("--batch-size", default=128)
@click.option("--bag-size", default=32)
@click.option("--iters", default=100)
@click.option("--remote", is_flag=True, default=False)
@click.option("--fp16", is_flag=True, default=False)
@click.option("--alpha", default=0.0, help="Zipf exponent of the indices (0 = uniform)")
@click.option("--seed", default=42)
def cli(num_tables, num_embeddings, embedding_dim, batch_size, bag_size, iters, remote, fp16, alpha, seed):
    logging.basicConfig(level=logging.INFO, stream=sys.stderr)
    if remote:
        raise click.UsageError("--remote (cluster submission) is not available; run the benchmark locally")
    run(batch_size, num_embeddings, num_tables, bag_size, embedding_dim, iters, fp16, alpha, seed)


if __name__ == "__main__":
    cli()
