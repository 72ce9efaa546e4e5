"""Planning a batch ahead of its step (RowCache.prefetch / tbe_cache_plan + tbe_cache_commit).

The reference has nothing to compare with (its host-resident tables are read over the bus on
every lookup, table_batched_embeddings_cuda.cu:795-880), so the checks are the ones that tie the
row cache back to the reference's arithmetic: a run that plans every batch one step ahead, on
side streams, while the batch before it computes, gives bit for bit the outputs, the flushed
table and the optimizer state of the same steps on a table held in device memory; and the cache's
decisions (slots, evictions, tags) still equal the CPU model's, because planning ahead moves
work in time and changes no decision."""
import numpy as np
import pytest
import torch

from gpu_util import DEV, dev

import table_batched_embeddings as ext
import table_batched_embeddings_cache as tc
import table_batched_embeddings_ops as ops

pytestmark = pytest.mark.gpu


def _draw_batch(rs, T, rows, B, L, zipf):
    lengths = rs.randint(0, L + 1, size=(T, B))
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    per_table = lengths.sum(axis=1)
    indices = np.concatenate([(rs.zipf(zipf, size=int(per_table[t])) % rows[t]) for t in range(T)]).astype(np.int32)
    return indices, offsets


def _tables(rows, D, dtype):
    total = sum(rows)
    start = (torch.rand(total, D, device=DEV, dtype=torch.float64) * 0.02 - 0.01).to(dtype)
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=dtype), (total, D))
    cached_w.copy_(start)
    st_dtype = torch.float64 if dtype == torch.float64 else torch.float32
    return (start.clone(), cached_w, torch.zeros(total, device=DEV, dtype=st_dtype),
            torch.zeros(total, device=DEV, dtype=st_dtype))


ORDERS = ["before_forward", "before_backward", "after_backward", "every_other"]


@pytest.mark.parametrize("order", ORDERS)
@pytest.mark.parametrize("mode,dtype,D", [("sgd", torch.float32, 128), ("adagrad_weighted", torch.float16, 64),
                                          ("adagrad", torch.float64, 12), ("sgd", torch.float32, 520)])
@pytest.mark.parametrize("num_sets,stage_slots", [(2, 4096), (2, 7), (5, 300), (40, 64), (1, 1)])
def test_prefetched_training_equals_uncached_bit_exact(order, mode, dtype, D, num_sets, stage_slots):
    """Ten steps with every batch planned ahead, in several orders of the calls, then a flush.  With
    4096 staging rows every missing row finds a staging or landing row; with 7 or 1 most do not, so
    rows stay in the backing table for a step and inserted rows enter their slot without a landing
    row; with 40 sets most rows are cached.  Rows that consecutive batches share (Zipf) travel from
    one step's staging area to the next step's slot or staging row."""
    rs = np.random.RandomState(5)
    T, rows, B, L = 3, [700, 90, 3000], 48, 9
    table_offsets = dev(np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    plain_w, cached_w, plain_state, cached_state = _tables(rows, D, dtype)
    cache = tc.RowCache(cached_w, num_sets * 64, "lru", stage_slots)
    assert cache.deferred_write_back
    weighted = mode.endswith("weighted")
    opt = "sgd" if mode == "sgd" else "adagrad"
    steps = 10
    batches = []
    for _ in range(steps):
        indices, offsets = _draw_batch(rs, T, rows, B, L, 1.2)
        batches.append((dev(indices), dev(offsets),
                        torch.randn(B, T, D, device=DEV, dtype=torch.float64).to(dtype),
                        torch.rand(indices.size, device=DEV, dtype=torch.float64).to(dtype) if weighted else None))
    planned = 0  # batches handed to prefetch so far

    def prefetch_up_to(k):
        nonlocal planned
        while planned <= min(k, steps - 1):
            cache.prefetch(table_offsets, batches[planned][0], batches[planned][1])
            planned += 1

    seen = dict.fromkeys(("staged", "uncached", "from_staging", "late_fetches", "no_landing_row", "written_out",
                          "hits", "written_back"), 0)
    for i, (idx, off, go, psw) in enumerate(batches):
        want = ext.forward(plain_w, table_offsets, idx, off, psw, 200, 1, False)
        if opt == "sgd":
            ext.backward_sgd(go, plain_w, table_offsets, idx, off, 0.05, 200, 1, False)
            want_g = None
        else:
            want_g = ext.backward_exact_adagrad(go, plain_w, table_offsets, idx, off, psw, plain_state, 0.05, 0.1,
                                                False, 1)
        if order == "before_forward":
            prefetch_up_to(i + 1)       # this batch was planned one step ago; the next one goes out now,
                                        # so two planned batches exist until the prepare() below
        elif order == "every_other" and i % 2 == 0:
            cache.prefetch(table_offsets, idx, off)   # planned right before use; odd steps are not planned ahead
        elif order in ("before_backward", "after_backward") and i == 0:
            prefetch_up_to(0)
        cache.prepare(table_offsets, idx, off)
        got = cache.forward(table_offsets, idx, off, psw)
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
    # the run went through the paths it is meant to cover
    assert seen["hits"] > 0
    if num_sets <= 5:
        assert seen["written_back"] > 0 and seen["staged"] > 0
    if stage_slots == 4096:
        assert seen["uncached"] == 0 and seen["no_landing_row"] == 0
        assert seen["from_staging"] > 0 and seen["written_out"] > 0
        if order != "every_other":
            assert seen["late_fetches"] > 0       # rows taken over from the staging area of the step before
    if stage_slots in (1, 7) and num_sets <= 2:
        assert seen["uncached"] > 0 and seen["no_landing_row"] > 0
    ext.free_host_tensor(cached_w)


@pytest.mark.parametrize("policy", ["lru", "lfu"])
def test_prefetch_changes_no_decision(oracle, policy):
    """Slots, evictions, counters of every batch and the tags after it equal the CPU model's when
    every batch is planned one step ahead."""
    rs = np.random.RandomState(21)
    T, rows, B, L, D, num_sets, stage_slots = 3, [300, 5000, 40], 64, 12, 32, 3, 2000
    table_offsets = np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32)
    backing = torch.randn(sum(rows), D, device=DEV)
    cache = tc.RowCache(backing, num_sets * 64, policy, stage_slots)
    model = oracle.CacheModel(num_sets, policy)
    batches = [_draw_batch(rs, T, rows, B, L, 1.15) for _ in range(7)]
    on_device = [(dev(i), dev(o)) for i, o in batches]
    to = dev(table_offsets)
    cache.prefetch(to, *on_device[0])
    for step, (indices, offsets) in enumerate(batches):
        keys = np.unique(table_offsets[np.repeat(np.arange(T * B), np.diff(offsets)) // B] + indices)
        slots, evicted, stats = model.step(keys)
        # the tags are this batch's until the next one is planned
        np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)
        np.testing.assert_array_equal(cache.last_used.cpu().numpy(), model.last_used)
        np.testing.assert_array_equal(cache.use_count.cpu().numpy(), model.use_count)
        if step + 1 < len(batches):
            cache.prefetch(to, *on_device[step + 1])
        cache.prepare(to, *on_device[step])
        got = cache.unique_slots().cpu().numpy()
        staged = got >= num_sets * 64
        np.testing.assert_array_equal(cache.unique_keys().cpu().numpy(), keys)
        np.testing.assert_array_equal(np.where(staged, -1, got), slots)
        got_evicted = cache.evicted_keys().cpu().numpy()
        np.testing.assert_array_equal(got_evicted[~staged], evicted[~staged])
        st = cache.stats()
        assert [st[k] for k in ("unique_rows", "hits", "misses", "inserted", "written_back")] == stats[:5].tolist()
        assert st["staged"] + st["uncached"] == stats[5]
        # every row of the batch is where its slot says: cache slot, staging row or backing table
        where = torch.from_numpy(got).to(DEV).long()
        held = cache.rows[where.clamp_min(0)]
        from_table = backing[torch.from_numpy(keys).to(DEV).long()]
        assert torch.equal(torch.where((where >= 0).unsqueeze(1), held, from_table), from_table)
    cache.flush()
    torch.cuda.synchronize()


def test_prefetch_refusals():
    backing = torch.randn(500, 16, device=DEV)
    to = dev(np.zeros(1, np.int32))
    idx = [torch.randint(0, 500, (40,), dtype=torch.int32, device=DEV) for _ in range(4)]
    off = torch.arange(0, 41, 4, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="needs deferred write-back"):
        tc.RowCache(backing, 64).prefetch(to, idx[0], off)
    cache = tc.RowCache(backing, 64, stage_slots=32)
    cache.prefetch(to, idx[0], off)
    with pytest.raises(RuntimeError, match="another batch was prefetched"):
        cache.prepare(to, idx[1], off)
    cache.prefetch(to, idx[1], off)
    with pytest.raises(RuntimeError, match="two batches are already prefetched"):
        cache.prefetch(to, idx[2], off)
    cache.prepare(to, idx[0], off)
    out0 = cache.forward(to, idx[0], off)
    cache.prepare(to, idx[1], off)
    cache.forward(to, idx[1], off)
    assert out0.shape == (10, 1, 16)
    # a flush with a planned batch waiting commits that batch; the batch whose backward is still
    # due loses its slots and is refused
    cache.prefetch(to, idx[2], off)
    cache.flush()
    with pytest.raises(RuntimeError, match="prepared for another batch"):
        cache.backward("sgd", torch.zeros(10, 1, 16, device=DEV), None, None, 0.1, 0.0)
    cache.prepare(to, idx[2], off)
    cache.backward("sgd", torch.zeros(10, 1, 16, device=DEV), None, None, 0.1, 0.0)
    cache.invalidate()
    with pytest.raises(RuntimeError, match="no batch is prepared"):
        cache.forward(to, idx[2], off)
    torch.cuda.synchronize()


def test_module_prefetch_trains_like_device_module():
    """TableBatchedEmbeddingBags.prefetch: the HOST_CACHED module with every batch planned ahead
    follows the trajectory of the plain device module; a checkpoint taken between steps, with a
    planned batch waiting, holds the current rows."""
    T, E, D, B, L = 4, 500, 64, 32, 6
    torch.manual_seed(0)
    kwargs = dict(optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.1, eps=0.1)
    plain = ops.TableBatchedEmbeddingBags(T, E, D, **kwargs).cuda()
    cached = ops.TableBatchedEmbeddingBags(T, E, D, managed=ops.EmbeddingLocation.HOST_CACHED, cache_slots=256,
                                           cache_stage_slots=512, **kwargs).cuda()
    cached.embedding_weights.data.copy_(plain.embedding_weights.data)
    with pytest.raises(RuntimeError, match="behind the row cache"):
        plain.prefetch(None, None)
    rs = np.random.RandomState(1)
    batches = []
    for _ in range(6):
        indices, offsets = _draw_batch(rs, T, [E] * T, B, L, 1.2)
        batches.append((dev(indices), dev(offsets), torch.randn(B, T, D, device=DEV)))
    cached.prefetch(*batches[0][:2])
    for i, (idx, off, go) in enumerate(batches):
        if i + 1 < len(batches):
            cached.prefetch(*batches[i + 1][:2])
        a = plain(idx, off)
        a.backward(go)
        b = cached(idx, off)
        b.backward(go)
        assert torch.equal(a, b)
        if i == 3:
            sd = cached.state_dict()
            torch.cuda.synchronize()
            assert torch.equal(sd["embedding_weights"], plain.embedding_weights.data)
    sd = cached.state_dict()
    torch.cuda.synchronize()
    assert torch.equal(sd["embedding_weights"], plain.embedding_weights.data)
    assert torch.equal(sd["optimizer_state"], plain.optimizer_state)
