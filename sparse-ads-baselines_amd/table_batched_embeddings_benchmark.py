"""Micro-benchmark CLI with the flags of the reference's table_batched_embeddings_benchmark.py
(:360-370): --num-tables 64 --num-embeddings 10000 --embedding-dim 32 --batch-size 128
--bag-size 32 --iters 100 [--fp16] [--managed] [--mixed] [--remote], plus --alpha / --seed / --kernels /
--compiled / --cache-slots.

Each operator is called directly on the extension-module mirror (not through autograd), after
one warm-up call, `iters` times between two events on the current stream
(table_batched_embeddings_benchmark.py:27-37).  "BW" is the reference's figure:
elem * B * T * L * D / time for forward (:240) and twice that for backward (:356).  One JSON
object per measurement goes to stdout.

--cache-slots N (no counterpart in the reference): the tables live in pinned host memory behind an
HBM row cache of N rows (EmbeddingLocation.HOST_CACHED) and the rows printed are the cache's plan
for a batch (sort, slots, row traffic), the forward through it, and plan + update per optimizer
-- a plan serves one update.  Every call sees the same batch, so from the second call on the rows
the cache can hold are resident: with N at least the batch's unique rows this times the kernels'
way through the slots, with fewer the host link as well.
"""
import json
import logging
import sys

import click
import numpy as np
import torch

import table_batched_embeddings
import table_batched_embeddings_ops as ops

# the module whose functions are timed: the Python binding of the C ABI, or the compiled one (--compiled)
EXT = table_batched_embeddings

HBM_PEAK_GBPS = 8000.0


KERNEL_TIMES = False  # --kernels: also log the average duration of every library kernel of an op


def time_calls(iters, fn):
    fn()
    torch.cuda.synchronize()
    if KERNEL_TIMES:
        import tbe_native
        with tbe_native.profile() as prof:
            for _ in range(3):
                fn()
        per_kernel = {}
        for name, ms in prof.launches:
            per_kernel.setdefault(name, []).append(ms)
        logging.info("  kernels (us x launches per call): %s", ", ".join(
            "%s %.1f x%d" % (k, 1e3 * sum(v) / len(v), len(v) // 3) for k, v in per_kernel.items()))
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1.0e-3 / iters


def draw_indices(rs, T, B, L, rows, alpha):
    if alpha and alpha > 1.0:
        cols = [rs.zipf(alpha, size=(B, L)) % rows[t] for t in range(T)]
    else:
        cols = [rs.randint(0, rows[t], size=(B, L)) for t in range(T)]
    merged = np.stack(cols).astype(np.int32)  # [T][B][L], table-major as the kernels expect
    offsets = np.arange(0, T * B * L + 1, L, dtype=np.int32)
    return torch.from_numpy(merged.reshape(-1)).cuda(), torch.from_numpy(offsets).cuda()


def report(name, seconds, bytes_moved, shape):
    record = dict(shape, op=name, time_us=seconds * 1e6, BW_GBps=bytes_moved / seconds / 1e9,
                  frac_of_hbm_peak=bytes_moved / seconds / 1e9 / HBM_PEAK_GBPS)
    logging.info("%s, B: %d, E: %s, T: %d, D: %s, L: %d, BW: %.2fGB/s, T: %.0fus", name, shape["B"], shape["E"],
                 shape["T"], shape["D"], shape["L"], record["BW_GBps"], record["time_us"])
    print(json.dumps(record))


def run_cached(cc, indices, offsets, iters, fwd_bytes, shape):
    """The rows of --cache-slots: plan, forward and plan + update through the module's row cache."""
    cache = cc.row_cache
    first_rows = cc.cache_table_rows()
    lr, eps = 0.05, 0.01
    plan = lambda: cache.prepare(first_rows, indices, offsets)
    plan()
    y0 = cache.forward(first_rows, indices, offsets)
    go = torch.randn_like(y0)
    report("Cached-Plan", time_calls(iters, plan), 0.0, shape)
    report("Cached-Forward", time_calls(iters, lambda: cache.forward(first_rows, indices, offsets)), fwd_bytes, shape)
    for name, kind in (("SGD-EXACT", "sgd"), ("ADAGRAD-nonstochastic-APPROX-NR", "approx_adagrad"),
                       ("ADAGRAD-nonstochastic-EXACT-NR", "adagrad")):
        def step():
            plan()
            cache.backward(kind, go, None, cc.optimizer_state, lr, eps)
        report("Cached-Plan+Backward-" + name, time_calls(iters, step), 2 * fwd_bytes, shape)
    logging.info("cache after the last plan: %s", cache.stats())


def run(B, E, T, L, D, iters, fp16, managed, mixed, alpha, seed, cache_slots=0):
    rs = np.random.RandomState(seed)
    location = ops.EmbeddingLocation.HOST_MAPPED if managed else ops.EmbeddingLocation.DEVICE
    cache_args = {}
    if cache_slots:
        location = ops.EmbeddingLocation.HOST_CACHED
        cache_args = dict(cache_slots=cache_slots, cache_stage_slots=T * B * L)
    elem = 2 if fp16 else 4
    if mixed:
        dims = [int((rs.randint(int(0.5 * D), int(1.5 * D) + 1) + 3) // 4 * 4) for _ in range(T)]
        cc = ops.MixedDimTableBatchedEmbeddingBags([(E, d) for d in dims], optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD,
                                                   learning_rate=0.1, eps=0.1, fp16=fp16, managed=location,
                                                   **cache_args).cuda()
        D_eff = float(np.mean(dims))
    else:
        cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.1,
                                           eps=0.1, fp16=fp16, managed=location, **cache_args).cuda()
        D_eff = D
    logging.info("Embedding parameters: %.2fGParam", cc.embedding_weights.numel() / 1.0e9)
    indices, offsets = draw_indices(rs, T, B, L, [E] * T, alpha)
    unique = np.unique(indices.cpu().numpy().astype(np.int64) + np.repeat(np.arange(T), B * L) * E).size
    logging.info("Duplicate proportion: %.3f", 1.0 - unique / indices.numel())
    shape = dict(B=B, E=E, T=T, D=D_eff, L=L, fp16=fp16, managed=managed, mixed=mixed, alpha=alpha)
    w = cc.embedding_weights.data
    fwd_bytes = elem * B * T * L * D_eff
    if cache_slots:
        shape["cache_slots"] = cache_slots
        return run_cached(cc, indices, offsets, iters, fwd_bytes, shape)

    if mixed:
        fwd = lambda: EXT.forward_mixed_D(
            w, cc.table_offsets, cc.dim_offsets, cc.total_D, indices, offsets, None, L, 1, False)
    else:
        fwd = lambda: EXT.forward(w, cc.table_offsets, indices, offsets, None, L, 1, False)
    y0 = fwd()
    if not mixed:  # the launch knobs of the reference must not change results (:179-206)
        for bt in (1, 2, 4, 8, 16, 32, 64, 128):
            for shmem in (True, False):
                assert torch.equal(EXT.forward(w, cc.table_offsets, indices, offsets, None, L,
                                                                    bt, shmem), y0)
    report("Forward", time_calls(iters, fwd), fwd_bytes, shape)

    go = torch.randn_like(y0)
    lr, eps = 0.05, 0.01
    if mixed:
        sgd = lambda: table_batched_embeddings.backward_sgd_mixed_D(
            go, w, cc.table_offsets, cc.table_dim_offsets, cc.dim_offsets, cc.total_D, indices, offsets,
            cc.optimizer_state, lr)
    else:
        sgd = lambda: EXT.backward_sgd(go, w, cc.table_offsets, indices, offsets, lr, L, 1,
                                                            False)
    report("Backward-SGD-EXACT", time_calls(iters, sgd), 2 * fwd_bytes, shape)

    # the reference's rows (table_batched_embeddings_benchmark.py:266-357): approximate and exact
    # row-wise Adagrad, with stochastic rounding as well when the weights are fp16; the launch knob
    # it sweeps (BT_block_size) does not exist here, so each row is printed once
    def adagrad(exact, stochastic):
        if mixed:
            if exact:
                return lambda: EXT.backward_exact_adagrad_mixed_D(
                    go, w, cc.table_offsets, cc.table_dim_offsets, cc.dim_offsets, cc.total_D, indices, offsets,
                    None, cc.optimizer_state, lr, eps, stochastic, 1)
            return lambda: EXT.backward_approx_adagrad_mixed_D(
                go, w, cc.table_offsets, cc.table_dim_offsets, cc.dim_offsets, cc.total_D, indices, offsets, None,
                cc.optimizer_state, lr, eps, L, stochastic, 1)
        if exact:
            return lambda: EXT.backward_exact_adagrad(
                go, w, cc.table_offsets, indices, offsets, None, cc.optimizer_state, lr, eps, stochastic, 1)
        return lambda: EXT.backward_approx_adagrad(
            go, w, cc.table_offsets, indices, offsets, None, cc.optimizer_state, lr, eps, L, stochastic, 1)

    for exact in (0, 1):
        for stochastic in ((0, 1) if fp16 else (0,)):
            name = "Backward-ADAGRAD-%s-%s-NR" % ("stochastic" if stochastic else "nonstochastic",
                                                  "EXACT" if exact else "APPROX")
            report(name, time_calls(iters, adagrad(exact, bool(stochastic))), 2 * fwd_bytes, shape)


@click.command()
@click.option("--num-tables", default=64)
@click.option("--num-embeddings", default=int(1e4))
@click.option("--embedding-dim", default=32)
@click.option("--batch-size", default=128)
@click.option("--bag-size", default=32)
@click.option("--iters", default=100)
@click.option("--remote", is_flag=True, default=False)
@click.option("--fp16", is_flag=True, default=False)
@click.option("--managed", is_flag=True, default=False)
@click.option("--mixed", is_flag=True, default=False)
@click.option("--kernels", is_flag=True, default=False, help="Log per-kernel times of every op")
@click.option("--alpha", default=0.0, help="Zipf exponent of the indices (0 = uniform)")
@click.option("--seed", default=42)
@click.option("--compiled", is_flag=True, default=False,
              help="Call the kernels through the pybind11 module (table_batched_embeddings_cpp)")
@click.option("--cache-slots", default=0, help="Host-resident tables behind an HBM row cache of this many rows")
def cli(num_tables, num_embeddings, embedding_dim, batch_size, bag_size, iters, remote, fp16, managed, mixed, kernels,
        alpha, seed, compiled, cache_slots):
    global KERNEL_TIMES, EXT
    KERNEL_TIMES = kernels
    if compiled:
        import table_batched_embeddings_cpp
        EXT = table_batched_embeddings_cpp
        ops.use_extension(EXT)
    logging.basicConfig(level=logging.INFO, stream=sys.stderr)
    if remote:
        raise click.UsageError("--remote (cluster submission) is not available; run the benchmark locally")
    if cache_slots and (managed or compiled):
        raise click.UsageError("--cache-slots goes with neither --managed nor --compiled")
    run(batch_size, num_embeddings, num_tables, bag_size, embedding_dim, iters, fp16, managed, mixed, alpha, seed,
        cache_slots)


if __name__ == "__main__":
    cli()
