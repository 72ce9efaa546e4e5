"""GPU parity of tables of different widths behind the HBM row cache (tbe_forward_mixed_cached /
tbe_backward_mixed_cached and the tbe_cache_* calls on a cache that describes such tables).

The reference has neither a cache nor host-cached mixed-D tables; the property that ties the path
back to the reference's semantics is the one the uniform tables' cache is tested by: a run through
the cache equals, bit for bit, the same steps of tbe_forward_mixed / tbe_backward_mixed (checked
against the CPU oracle in test_gpu_mixed_dim.py) on tables that live entirely in device memory --
the arithmetic kernels are the same, only the rows' addresses differ.  The cache's decisions depend
on the keys alone and are checked against the CPU model of its specification."""
import numpy as np
import pytest
import torch

from gpu_util import DEV, dev

import table_batched_embeddings as ext
import table_batched_embeddings_cache as tc
import table_batched_embeddings_ops as ops

pytestmark = pytest.mark.gpu


def _tables_on_device(tables):
    rows, dims = zip(*tables)
    table_dim_offsets = dev(np.concatenate([[0], np.cumsum(rows)]).astype(np.int32))
    table_offsets = dev(np.concatenate([[0], np.cumsum([r * d for r, d in tables])]).astype(np.int64))
    dim_offsets = dev(np.concatenate([[0], np.cumsum(dims)]).astype(np.int32))
    return table_offsets, table_dim_offsets, dim_offsets


def _draw_batch(rs, tables, B, L, zipf):
    T = len(tables)
    lengths = rs.randint(0, L + 1, size=(T, B))
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    per_table = lengths.sum(axis=1)
    indices = np.concatenate([(rs.zipf(zipf, size=int(per_table[t])) % tables[t][0]) for t in range(T)])
    return indices.astype(np.int32), offsets


# narrow, odd vector counts, a table wider than 64 vectors (fp32: 520 / 4 = 130), hot rows in small tables
# (the table of one row: every lookup of its bags on the same row, several hundred per step -- several
# chunks for the exact updates, a workgroup's walk for the approximate update of fp16 rows)
TABLES = [(700, 8), (90, 36), (3000, 64), (40, 520), (5, 128), (1200, 20), (1, 64)]


@pytest.mark.parametrize("mode,dtype", [("sgd", torch.float32), ("adagrad", torch.float32),
                                        ("adagrad_weighted", torch.float16), ("adagrad_weighted", torch.float32),
                                        ("sgd", torch.float16), ("adagrad", torch.float64),
                                        ("approx", torch.float32), ("approx_weighted", torch.float16),
                                        ("approx", torch.float16), ("approx_weighted", torch.float64)])
@pytest.mark.parametrize("num_sets,stage_slots,deferred", [(2, 0, False), (60, 0, False), (2, 8192, False),
                                                          (2, 7, False), (2, 8192, True), (2, 7, True),
                                                          (9, 300, True)])
def test_cached_mixed_training_equals_uncached_bit_exact(mode, dtype, num_sets, stage_slots, deferred):
    """Six forward + backward steps through the cache, then a flush: outputs of every step, the
    final tables, optimizer state and per-sample-weight gradients are bit-identical to the same
    steps on tables in device memory.  Rows of every kind of the update meet every kind of home:
    rows of few occurrences (strips), of up to 256 (one chunk record), of more (several chunks and
    the finishing kernel: B * L lookups on a table of 5 rows) and rows wider than 64 vectors, in a
    slot, a staging row, a landing row or -- with 2 sets and little staging -- the backing table.
    The approximate (per-lookup) Adagrad goes through the strip kernel's per-lookup form and, for
    the rows of more occurrences and the wide rows, the approximate update's own kernels."""
    rs = np.random.RandomState(5)
    B, L = 64, 12
    T = len(TABLES)
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(TABLES)
    total_D = sum(d for _, d in TABLES)
    total_rows = sum(r for r, _ in TABLES)
    numel = sum(r * d for r, d in TABLES)
    start = (torch.rand(numel, device=DEV, dtype=torch.float64) * 0.02 - 0.01).to(dtype)
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=dtype), (numel,))
    cached_w.copy_(start)
    st_dtype = torch.float64 if dtype == torch.float64 else torch.float32
    plain_state = torch.zeros(total_rows, device=DEV, dtype=st_dtype)
    cached_state = torch.zeros(total_rows, device=DEV, dtype=st_dtype)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    cache = tc.RowCache(cached_w, num_sets * 64, "lru", stage_slots, deferred_write_back=deferred, mixed=mixed)
    weighted = mode.endswith("weighted")
    opt = "sgd" if mode == "sgd" else "approx_adagrad" if mode.startswith("approx") else "adagrad"
    served_uncached = served_staged = 0
    for step in range(6):
        indices, offsets = _draw_batch(rs, TABLES, B, L, 1.2)
        idx, off = dev(indices), dev(offsets)
        go = torch.randn(B, total_D, device=DEV, dtype=torch.float64).to(dtype)
        psw = torch.rand(indices.size, device=DEV, dtype=torch.float64).to(dtype) if weighted else None
        want = ext.forward_mixed_D(plain_w, table_offsets, dim_offsets, total_D, idx, off, psw, 200, 1, False)
        if opt == "sgd":
            ext.backward_sgd_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets, total_D, idx, off,
                                     plain_state, 0.05)
            want_g = None
        elif opt == "approx_adagrad":
            want_g = ext.backward_approx_adagrad_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets,
                                                         total_D, idx, off, psw, plain_state, 0.05, 0.1, 200, False, 1)
        else:
            want_g = ext.backward_exact_adagrad_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets,
                                                        total_D, idx, off, psw, plain_state, 0.05, 0.1, False, 1)
        cache.prepare(mixed.table_rows, idx, off)
        got = cache.forward(mixed.table_rows, idx, off, psw)
        got_g = cache.backward(opt, go, psw, cached_state, 0.05, 0.1)
        assert torch.equal(got, want), "forward output differs at step %d" % step
        if weighted:
            assert torch.equal(got_g, want_g)
        served_uncached += cache.stats()["uncached"]
        served_staged += cache.stats()["staged"]
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w)
    assert torch.equal(cached_state, plain_state)
    if num_sets != 9:
        assert (served_uncached > 0) == (num_sets == 2 and stage_slots < 8192)
    assert (served_staged > 0) == (stage_slots > 0)
    ext.free_host_tensor(cached_w)


@pytest.mark.parametrize("order", ["before_forward", "before_backward", "after_backward", "every_other"])
@pytest.mark.parametrize("mode,dtype", [("sgd", torch.float32), ("adagrad_weighted", torch.float16)])
@pytest.mark.parametrize("num_sets,stage_slots", [(2, 8192), (2, 7), (9, 300), (1, 1)])
def test_prefetched_mixed_training_equals_uncached_bit_exact(order, mode, dtype, num_sets, stage_slots):
    """Ten steps with every batch planned ahead (RowCache.prefetch: tbe_cache_plan + tbe_cache_commit),
    in several orders of the calls, then a flush.  An evicted row waits in the landing row of the
    row that replaced it -- a row of another table and another width now and then -- and goes back
    to its table two steps later with its own width."""
    rs = np.random.RandomState(6)
    B, L = 48, 10
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(TABLES)
    total_D = sum(d for _, d in TABLES)
    total_rows = sum(r for r, _ in TABLES)
    numel = sum(r * d for r, d in TABLES)
    start = (torch.rand(numel, device=DEV, dtype=torch.float64) * 0.02 - 0.01).to(dtype)
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=dtype), (numel,))
    cached_w.copy_(start)
    plain_state = torch.zeros(total_rows, device=DEV)
    cached_state = torch.zeros(total_rows, device=DEV)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    cache = tc.RowCache(cached_w, num_sets * 64, "lru", stage_slots, mixed=mixed)
    assert cache.deferred_write_back
    weighted = mode.endswith("weighted")
    opt = "sgd" if mode == "sgd" else "adagrad"
    steps = 10
    batches = []
    for _ in range(steps):
        indices, offsets = _draw_batch(rs, TABLES, B, L, 1.2)
        batches.append((dev(indices), dev(offsets), torch.randn(B, total_D, device=DEV, dtype=torch.float64).to(dtype),
                        torch.rand(indices.size, device=DEV, dtype=torch.float64).to(dtype) if weighted else None))
    planned = 0

    def prefetch_up_to(k):
        nonlocal planned
        while planned <= min(k, steps - 1):
            cache.prefetch(mixed.table_rows, batches[planned][0], batches[planned][1])
            planned += 1

    seen = dict.fromkeys(("staged", "uncached", "from_staging", "late_fetches", "no_landing_row", "written_out",
                          "hits", "written_back"), 0)
    for i, (idx, off, go, psw) in enumerate(batches):
        want = ext.forward_mixed_D(plain_w, table_offsets, dim_offsets, total_D, idx, off, psw, 200, 1, False)
        if opt == "sgd":
            ext.backward_sgd_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets, total_D, idx, off,
                                     plain_state, 0.05)
            want_g = None
        else:
            want_g = ext.backward_exact_adagrad_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets,
                                                        total_D, idx, off, psw, plain_state, 0.05, 0.1, False, 1)
        if order == "before_forward":
            prefetch_up_to(i + 1)
        elif order == "every_other" and i % 2 == 0:
            cache.prefetch(mixed.table_rows, idx, off)
        elif order in ("before_backward", "after_backward") and i == 0:
            prefetch_up_to(0)
        cache.prepare(mixed.table_rows, idx, off)
        got = cache.forward(mixed.table_rows, idx, off, psw)
        if order == "before_backward":
            prefetch_up_to(i + 1)
        got_g = cache.backward(opt, go, psw, cached_state, 0.05, 0.1)
        if order == "after_backward":
            prefetch_up_to(i + 1)
        assert torch.equal(got, want), "forward output differs at step %d" % i
        if weighted:
            assert torch.equal(got_g, want_g), "per-sample-weight gradient differs at step %d" % i
        st = cache.stats()
        for k in seen:
            seen[k] += st[k]
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w)
    assert torch.equal(cached_state, plain_state)
    assert seen["hits"] > 0 and seen["written_back"] > 0 and seen["staged"] > 0
    if stage_slots == 8192:
        assert seen["uncached"] == 0 and seen["no_landing_row"] == 0
        assert seen["from_staging"] > 0 and seen["written_out"] > 0
    if stage_slots in (1, 7) and num_sets <= 2:
        assert seen["uncached"] > 0 and seen["no_landing_row"] > 0
    ext.free_host_tensor(cached_w)


def test_cached_mixed_stochastic_rounding_equals_uncached_bit_exact():
    """fp16 tables with stochastic rounding: a weight's random word goes by its place in the table,
    so the rows come out bit-identical wherever they are updated."""
    import ctypes
    import tbe_native
    rs = np.random.RandomState(9)
    tables = [(900, 64), (150, 24), (6, 128), (30, 520)]
    B, L = 40, 10
    T = len(tables)
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(tables)
    total_D = sum(d for _, d in tables)
    total_rows = sum(r for r, _ in tables)
    numel = sum(r * d for r, d in tables)
    start = (torch.rand(numel, device=DEV) * 0.02 - 0.01).half()
    plain_w, cached_w = start.clone(), start.clone()
    plain_state, cached_state = torch.zeros(total_rows, device=DEV), torch.zeros(total_rows, device=DEV)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    cache = tc.RowCache(cached_w, 2 * 64, "lru", stage_slots=50, mixed=mixed)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    for step in range(4):
        indices, offsets = _draw_batch(rs, tables, B, L, 1.2)
        idx, off = dev(indices), dev(offsets)
        go = torch.randn(B, total_D, device=DEV).half()
        lay = tbe_native.backward_mixed_workspace_layout(indices.size, tbe_native.DTYPE_F16, T)
        ws = torch.empty(lay.total_bytes, dtype=torch.uint8, device=DEV)
        tbe_native.check(tbe_native.load().tbe_backward_mixed(
            tbe_native.OPT_ROWWISE_ADAGRAD, vp(go), vp(plain_w), tbe_native.DTYPE_F16, mixed.vector_width, total_rows,
            0, vp(table_offsets), vp(table_dim_offsets), vp(dim_offsets), total_D, T, vp(idx), indices.size, vp(off),
            B, None, vp(plain_state), 0.05, 0.1, None, 1, 99, 4 * step, vp(ws), ws.numel(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        cache.prepare(mixed.table_rows, idx, off)
        cache.backward("adagrad", go, None, cached_state, 0.05, 0.1, stochastic_rounding=(99, 4 * step))
        st = cache.stats()
        assert st["staged"] > 0 and st["uncached"] > 0 and st["hits"] + st["inserted"] > 0
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w) and torch.equal(cached_state, plain_state)
    rn_w = start.clone()
    ext.backward_exact_adagrad_mixed_D(go, rn_w, table_offsets, table_dim_offsets, dim_offsets, total_D, idx, off,
                                       None, torch.zeros(total_rows, device=DEV), 0.05, 0.1, False, 1)
    assert not torch.equal(rn_w, start)


@pytest.mark.parametrize("policy", ["lru", "lfu"])
def test_cache_decisions_for_mixed_tables_match_the_model(oracle, policy):
    """Slots, evictions and tags depend on the keys alone: with tables of different widths they
    equal the CPU model's as with uniform tables, and a fetched row is the table's row, in the
    front of its cache row."""
    rs = np.random.RandomState(12)
    tables = [(300, 8), (5000, 40), (40, 132)]
    B, L, num_sets = 64, 12, 3
    rows = [r for r, _ in tables]
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(tables)
    first_rows = np.concatenate([[0], np.cumsum(rows)]).astype(np.int64)
    first_elements = np.concatenate([[0], np.cumsum([r * d for r, d in tables])]).astype(np.int64)
    backing = torch.randn(sum(r * d for r, d in tables), device=DEV)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    cache = tc.RowCache(backing, num_sets * 64, policy, 2000, deferred_write_back=False, mixed=mixed)
    model = oracle.CacheModel(num_sets, policy)
    for step in range(5):
        indices, offsets = _draw_batch(rs, tables, B, L, 1.15)
        cache.prepare(mixed.table_rows, dev(indices), dev(offsets))
        table_of_lookup = np.repeat(np.arange(len(tables) * B), np.diff(offsets)) // B
        keys = np.unique(first_rows[table_of_lookup] + indices)
        slots, evicted, stats = model.step(keys)
        got = cache.unique_slots().cpu().numpy()
        staged = got >= num_sets * 64
        np.testing.assert_array_equal(np.where(staged, -1, got), slots)
        np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)
        np.testing.assert_array_equal(cache.last_used.cpu().numpy(), model.last_used)
        np.testing.assert_array_equal(cache.use_count.cpu().numpy(), model.use_count)
        held = cache.rows.cpu()
        everything = backing.cpu()
        for u in rs.choice(keys.size, size=40, replace=False):
            if got[u] < 0:
                continue
            t = int(np.searchsorted(first_rows, keys[u], side="right") - 1)
            D = tables[t][1]
            at = first_elements[t] + (keys[u] - first_rows[t]) * D
            assert torch.equal(held[got[u], :D], everything[at:at + D])
    cache.flush()
    torch.cuda.synchronize()


def test_module_mixed_host_cached_trains_like_device_module():
    """MixedDimTableBatchedEmbeddingBags with managed=HOST_CACHED follows the trajectory of the
    device module, with and without planning batches ahead, and state_dict() sees the cached rows."""
    tables = [(500, 16), (60, 64), (2000, 36), (9, 260)]
    B, L = 32, 6
    torch.manual_seed(0)
    plain = ops.MixedDimTableBatchedEmbeddingBags(tables, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD,
                                                  learning_rate=0.1, eps=0.1).cuda()
    cached = ops.MixedDimTableBatchedEmbeddingBags(tables, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD,
                                                   learning_rate=0.1, eps=0.1,
                                                   managed=ops.EmbeddingLocation.HOST_CACHED, cache_slots=256,
                                                   cache_stage_slots=4096).cuda()
    cached.embedding_weights.data.copy_(plain.embedding_weights.data)
    rs = np.random.RandomState(1)
    batches = []
    for _ in range(6):
        indices, offsets = _draw_batch(rs, tables, B, L, 1.2)
        batches.append((dev(indices), dev(offsets), torch.randn(B, plain.total_D, device=DEV)))
    cached.prefetch(batches[0][0], batches[0][1])
    for i, (idx, off, go) in enumerate(batches):
        if i + 1 < len(batches) and i < 3:   # the first batches are planned ahead, the last ones are not
            cached.prefetch(batches[i + 1][0], batches[i + 1][1])
        a = plain(idx, off)
        a.backward(go)
        b = cached(idx, off)
        b.backward(go)
        assert torch.equal(a, b)
    sd = cached.state_dict()
    torch.cuda.synchronize()
    assert torch.equal(sd["embedding_weights"], plain.embedding_weights.data)
    assert torch.equal(sd["optimizer_state"], plain.optimizer_state)
    for got, want in zip(cached.split_embedding_weights(), plain.split_embedding_weights()):
        assert torch.equal(got, want)
    st = cached.row_cache.stats()
    assert st["hits"] > 0 and st["unique_rows"] == st["hits"] + st["misses"]


def test_mixed_cached_bad_arguments_and_empty_batch():
    tables = [(30, 8), (7, 32)]
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(tables)
    backing = torch.randn(30 * 8 + 7 * 32, device=DEV)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    assert (mixed.T, mixed.total_D, mixed.widest, mixed.total_rows) == (2, 40, 32, 37)
    cache = tc.RowCache(backing, 64, "lru", 16, mixed=mixed)
    assert tuple(cache.rows.shape) == (64 + 3 * 16, 32)
    with pytest.raises(RuntimeError, match="contiguous 1-D"):
        tc.RowCache(backing.view(-1, 8), 64, "lru", 16, mixed=mixed)
    none = torch.zeros(0, dtype=torch.int32, device=DEV)
    off = dev(np.zeros(2 * 4 + 1, np.int32))
    cache.flush()
    cache.prepare(mixed.table_rows, none, off)
    out = cache.forward(mixed.table_rows, none, off)
    assert out.shape == (4, 40) and not out.any()
    assert cache.backward("sgd", torch.zeros(4, 40, device=DEV), None, None, 0.1, 0.0) is None
    idx = dev(np.array([1, 2, 3, 0], np.int32))
    off = dev(np.array([0, 1, 2, 2, 2, 3, 3, 4, 4], np.int32))
    with pytest.raises(RuntimeError, match="first row of each"):
        cache.prepare(dev(np.zeros(3, np.int32)), idx, off)
    cache.prepare(mixed.table_rows, idx, off)
    with pytest.raises(RuntimeError, match="grad_output must be"):
        cache.backward("sgd", torch.zeros(4, 2, 8, device=DEV), None, None, 0.1, 0.0)
    with pytest.raises(ValueError):
        cache.backward("adam", torch.zeros(4, 40, device=DEV), None, torch.zeros(37, device=DEV), 0.1, 0.1)
    cache.backward("approx_adagrad", torch.zeros(4, 40, device=DEV), None, torch.zeros(37, device=DEV), 0.1, 0.1)
    torch.cuda.synchronize()


@pytest.mark.parametrize("mixed", [False, True])
def test_benchmark_cli_times_the_way_through_the_cache(mixed):
    """--cache-slots on the micro-benchmark: host-resident tables (uniform or mixed-D) behind the cache."""
    import json
    import os
    import subprocess
    import sys
    from conftest import PACKAGE
    cmd = [sys.executable, os.path.join(PACKAGE, "table_batched_embeddings_benchmark.py"), "--num-tables", "4",
           "--num-embeddings", "1000", "--embedding-dim", "32", "--batch-size", "64", "--bag-size", "8", "--iters",
           "3", "--cache-slots", "1024"] + (["--mixed"] if mixed else [])
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stderr[-2000:]
    records = [json.loads(line) for line in out.stdout.splitlines() if line.startswith("{")]
    assert [r["op"] for r in records] == [
        "Cached-Plan", "Cached-Forward", "Cached-Plan+Backward-SGD-EXACT",
        "Cached-Plan+Backward-ADAGRAD-nonstochastic-APPROX-NR", "Cached-Plan+Backward-ADAGRAD-nonstochastic-EXACT-NR"]
    assert all(r["time_us"] > 0 and r["cache_slots"] == 1024 and r["mixed"] == mixed for r in records)


def test_cache_fronted_modules_refuse_to_be_moved_or_cast():
    """The cache keeps the addresses of the pinned table (and of the mixed-D offset buffers): .cuda() on
    the device they are on is a no-op and fine, a cast is refused loudly."""
    uniform = ops.TableBatchedEmbeddingBags(2, 50, 16, managed=ops.EmbeddingLocation.HOST_CACHED, cache_slots=64).cuda()
    mixed = ops.MixedDimTableBatchedEmbeddingBags([(50, 16), (20, 8)], managed=ops.EmbeddingLocation.HOST_CACHED,
                                                  cache_slots=64).cuda()
    assert mixed.cuda() is mixed and uniform.cuda() is uniform
    for module in (uniform, mixed):
        with pytest.raises(RuntimeError, match="cannot be moved to another device or cast"):
            module.half()
    plain = ops.MixedDimTableBatchedEmbeddingBags([(50, 16), (20, 8)]).cuda()
    assert plain.half().embedding_weights.dtype == torch.float16   # (tables in device memory cast as ever)


def test_cached_mixed_training_at_the_benchmark_shape_equals_uncached():
    """64 tables of 100 000 rows, widths 64..192, 5.2 M lookups per step (the mixed-D micro-benchmark's
    shape): three steps of exact Adagrad through a cache a sixth the size of a step's unique rows, every
    batch planned ahead, against the same steps on tables in device memory, bit for bit."""
    if torch.cuda.mem_get_info()[0] < 24 << 30:
        pytest.skip("needs 24 GB of free device memory")
    rs = np.random.RandomState(3)
    T, E, B, L = 64, 100000, 4096, 20
    tables = [(E, int((rs.randint(64, 193) + 3) // 4 * 4)) for _ in range(T)]
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(tables)
    total_D = sum(d for _, d in tables)
    numel = sum(r * d for r, d in tables)
    start = torch.rand(numel, device=DEV) * 0.02 - 0.01
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV), (numel,))
    cached_w.copy_(start)
    del start
    plain_state = torch.zeros(T * E, device=DEV)
    cached_state = torch.zeros(T * E, device=DEV)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    cache = tc.RowCache(cached_w, 1 << 19, "lru", 1 << 22, mixed=mixed)
    offsets = dev(np.arange(0, T * B * L + 1, L, dtype=np.int32))
    batches = [torch.from_numpy((rs.zipf(1.05, size=T * B * L) % E).astype(np.int32)).to(DEV) for _ in range(3)]
    go = torch.randn(B, total_D, device=DEV)
    cache.prefetch(mixed.table_rows, batches[0], offsets)
    staged = 0
    for i, idx in enumerate(batches):
        if i + 1 < len(batches):
            cache.prefetch(mixed.table_rows, batches[i + 1], offsets)
        want = ext.forward_mixed_D(plain_w, table_offsets, dim_offsets, total_D, idx, offsets, None, 200, 1, False)
        ext.backward_exact_adagrad_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets, total_D, idx,
                                           offsets, None, plain_state, 0.05, 0.1, False, 1)
        cache.prepare(mixed.table_rows, idx, offsets)
        got = cache.forward(mixed.table_rows, idx, offsets)
        cache.backward("adagrad", go, None, cached_state, 0.05, 0.1)
        assert torch.equal(got, want), "forward output differs at step %d" % i
        st = cache.stats()
        assert st["uncached"] == 0
        staged += st["staged"]
    assert staged > 1 << 20
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w)
    assert torch.equal(cached_state, plain_state)
    ext.free_host_tensor(cached_w)


@pytest.mark.parametrize("seed", range(24))
def test_cached_mixed_training_random_sweep(seed):
    """Seeded random shapes of the cached-equals-uncached property for tables of different widths:
    1..40 tables (the bisection that finds a key's table), tables of a few rows and of thousands,
    widths from one vector to more than 64, dtype, optimizer (approximate Adagrad included), policy,
    cache and staging sizes from "nearly everything misses" to "everything fits", write-back deferred
    or not, batches planned ahead or not, index skew."""
    rs = np.random.RandomState(900 + seed)
    T = int(rs.choice([1, 2, 7, 40]))
    dtype = [torch.float32, torch.float16, torch.float64][seed % 3]
    widths = [4, 8, 12, 32, 64, 100, 128, 260, 520]
    tables = [(int(rs.choice([1, 3, 60, 900, 4000])), int(rs.choice(widths))) for _ in range(T)]
    mode = ["sgd", "adagrad", "adagrad_weighted", "approx", "approx_weighted"][(seed // 3) % 5]
    policy = ["lru", "lfu"][seed % 2]
    num_sets = int(rs.choice([1, 3, 17, 200]))
    stage_slots = int(rs.choice([0, 5, 300, 100000]))
    deferred = bool(rs.randint(2))
    B, L, zipf = int(rs.choice([1, 30, 200])), int(rs.choice([1, 6, 25])), float(rs.choice([1.05, 1.3, 2.0]))
    table_offsets, table_dim_offsets, dim_offsets = _tables_on_device(tables)
    total_D = sum(d for _, d in tables)
    total_rows = sum(r for r, _ in tables)
    numel = sum(r * d for r, d in tables)
    start = (torch.rand(numel, device=DEV, dtype=torch.float64) * 0.02 - 0.01).to(dtype)
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=dtype), (numel,))
    cached_w.copy_(start)
    st_dtype = torch.float64 if dtype == torch.float64 else torch.float32
    plain_state = torch.zeros(total_rows, device=DEV, dtype=st_dtype)
    cached_state = torch.zeros(total_rows, device=DEV, dtype=st_dtype)
    mixed = tc.MixedTables(table_offsets, table_dim_offsets, dim_offsets)
    cache = tc.RowCache(cached_w, num_sets * 64, policy, stage_slots, deferred_write_back=deferred, mixed=mixed)
    ahead = cache.deferred_write_back and seed % 2 == 1
    weighted = mode.endswith("weighted")
    opt = "sgd" if mode == "sgd" else "approx_adagrad" if mode.startswith("approx") else "adagrad"
    batches = []
    for _ in range(5):
        indices, offsets = _draw_batch(rs, tables, B, L, zipf)
        batches.append((dev(indices), dev(offsets), torch.randn(B, total_D, device=DEV, dtype=torch.float64).to(dtype),
                        torch.rand(indices.size, device=DEV, dtype=torch.float64).to(dtype) if weighted else None))
    if ahead:
        cache.prefetch(mixed.table_rows, batches[0][0], batches[0][1])
    for step, (idx, off, go, psw) in enumerate(batches):
        if ahead and step + 1 < len(batches):
            cache.prefetch(mixed.table_rows, batches[step + 1][0], batches[step + 1][1])
        want = ext.forward_mixed_D(plain_w, table_offsets, dim_offsets, total_D, idx, off, psw, 200, 1, False)
        if opt == "sgd":
            ext.backward_sgd_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets, total_D, idx, off,
                                     plain_state, 0.05)
            want_g = None
        elif opt == "approx_adagrad":
            want_g = ext.backward_approx_adagrad_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets,
                                                         total_D, idx, off, psw, plain_state, 0.05, 0.1, 200, False, 1)
        else:
            want_g = ext.backward_exact_adagrad_mixed_D(go, plain_w, table_offsets, table_dim_offsets, dim_offsets,
                                                        total_D, idx, off, psw, plain_state, 0.05, 0.1, False, 1)
        cache.prepare(mixed.table_rows, idx, off)
        got = cache.forward(mixed.table_rows, idx, off, psw)
        got_g = cache.backward(opt, go, psw, cached_state, 0.05, 0.1)
        assert torch.equal(got, want), "forward output differs at step %d" % step
        if weighted and idx.numel():
            assert torch.equal(got_g, want_g)
        resident = cache.resident_keys()
        assert resident.numel() == torch.unique(resident).numel() <= num_sets * 64
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w)
    assert torch.equal(cached_state, plain_state)
    ext.free_host_tensor(cached_w)
