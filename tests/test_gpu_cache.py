"""GPU parity of the HBM row cache (tbe_cache_* through the C ABI).

The reference has no cache, so the checker is the CPU model of this repository's own
specification (oracle/lxu_cache_model.c) plus the property that ties the cache back to the
reference's semantics: a run through the cache equals, bit for bit, a run with the tables
fully in HBM, because the arithmetic kernels are the same and only row addresses differ."""
import numpy as np
import pytest
import torch

from conftest import make_problem
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


@pytest.mark.parametrize("policy", ["lru", "lfu"])
@pytest.mark.parametrize("num_sets", [1, 5, 64])
def test_cache_state_matches_model_bit_exact(oracle, policy, num_sets):
    """tags / recency / frequency words, slot of every unique row, evicted keys and counters
    after every step equal the CPU model's."""
    rs = np.random.RandomState(num_sets * 7 + len(policy))
    T, rows, B, L, D = 3, [300, 5000, 40], 64, 12, 32
    table_offsets = np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32)
    backing = torch.randn(sum(rows), D, device=DEV)
    cache = tc.RowCache(backing, num_sets * 64, policy)
    model = oracle.CacheModel(num_sets, policy)
    for step in range(8):
        indices, offsets = _draw_batch(rs, T, rows, B, L, 1.15)
        cache.prepare(dev(table_offsets), dev(indices), dev(offsets))
        keys = np.unique(table_offsets[np.repeat(np.arange(T * B), np.diff(offsets)) // B] + indices)
        slots, evicted, stats = model.step(keys)
        np.testing.assert_array_equal(cache.unique_keys().cpu().numpy(), keys)
        np.testing.assert_array_equal(cache.unique_slots().cpu().numpy(), slots)
        np.testing.assert_array_equal(cache.evicted_keys().cpu().numpy(), evicted)
        np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)
        np.testing.assert_array_equal(cache.last_used.cpu().numpy(), model.last_used)
        np.testing.assert_array_equal(cache.use_count.cpu().numpy(), model.use_count)
        np.testing.assert_array_equal(cache.resident_keys().cpu().numpy(), model.resident())
        got_stats = list(cache.stats().values())
        assert got_stats[:6] == stats.tolist() and not any(got_stats[6:])  # nothing is staged without a staging area
        # per-lookup slots agree with per-unique slots
        all_keys = table_offsets[np.repeat(np.arange(T * B), np.diff(offsets)) // B] + indices
        np.testing.assert_array_equal(cache.lookup_slots.cpu().numpy(), slots[np.searchsorted(keys, all_keys)])


@pytest.mark.parametrize("num_sets,stage_slots", [(1, 0), (1, 50000), (3, 1000)])
def test_many_misses_per_set(oracle, num_sets, stage_slots):
    """Hundreds of thousands of missing rows on one to three sets (a cache far too small for the
    batch): the work per set is one pass over its misses, and slots, evictions, tags and counters
    still equal the model's; staged rows get consecutive staging rows in ascending key order."""
    rs = np.random.RandomState(num_sets + stage_slots)
    rows, B, L, D = 400000, 4096, 40, 4
    table_offsets = np.zeros(1, np.int32)
    backing = torch.zeros(rows, D, device=DEV)
    cache = tc.RowCache(backing, num_sets * 64, "lru", stage_slots, deferred_write_back=stage_slots > 0)
    model = oracle.CacheModel(num_sets, "lru")
    for step in range(3):
        indices = rs.randint(0, rows, size=B * L).astype(np.int32)
        offsets = np.arange(0, B * L + 1, L, dtype=np.int32)
        cache.prepare(dev(table_offsets), dev(indices), dev(offsets))
        keys = np.unique(indices)
        assert keys.size > 100000
        slots, evicted, stats = model.step(keys)
        got_slots = cache.unique_slots().cpu().numpy()
        staged = got_slots >= num_sets * 64
        np.testing.assert_array_equal(np.where(staged, -1, got_slots), slots)
        np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)
        np.testing.assert_array_equal(cache.last_used.cpu().numpy(), model.last_used)
        st = cache.stats()
        assert st["staged"] == min(stage_slots, int((slots < 0).sum())) == int(staged.sum())
        assert st["uncached"] == int((slots < 0).sum()) - st["staged"]
        assert [st[k] for k in ("unique_rows", "hits", "misses", "inserted", "written_back")] == stats.tolist()[:5]
        if st["staged"]:
            # one staging row each, all different, inside this step's area
            rows_used = np.sort(got_slots[staged])
            assert np.unique(rows_used).size == rows_used.size
            area = cache.stage_area_base()
            assert area == num_sets * 64 + (cache.sequence % 3) * stage_slots
            assert rows_used[0] >= area and rows_used[-1] < area + stage_slots


@pytest.mark.parametrize("mode,dtype,D", [("sgd", torch.float32, 128), ("adagrad", torch.float32, 64),
                                          ("adagrad_weighted", torch.float16, 64), ("sgd", torch.float32, 520),
                                          ("sgd", torch.float64, 12), ("approx", torch.float32, 128),
                                          ("approx_weighted", torch.float16, 64), ("approx", torch.float16, 32),
                                          ("approx_weighted", torch.float32, 520), ("approx", torch.float64, 12)])
@pytest.mark.parametrize("num_sets,stage_slots,deferred", [(2, 0, False), (40, 0, False), (2, 4096, False),
                                                          (2, 7, False), (2, 4096, True), (2, 7, True),
                                                          (5, 300, True)])
def test_cached_training_equals_uncached_bit_exact(mode, dtype, D, num_sets, stage_slots, deferred):
    """Several forward + backward steps through the cache, then a flush: outputs of every step,
    the final table, optimizer state and per-sample-weight gradients are bit-identical to the
    same steps on a table that lives entirely in device memory.  With 2 sets most rows are
    served straight from the backing table; with 40 most are cached.  With a staging area the rows
    that find no slot are staged in HBM for the step and copied back after the update (all of
    them with 4096 staging rows, some with 7) -- or, with deferred write-back, kept until the next
    step, which fetches the rows it needs again from there and writes the others back.
    The approximate (per-lookup) Adagrad goes through its own kernels -- tiles of short rows, chunk
    sums or a wavefront's walk for the rows of many occurrences, the kernel for rows wider than a
    wavefront -- each of which has to find a row where it lives."""
    rs = np.random.RandomState(3)
    T, rows, B, L = 3, [700, 90, 3000], 48, 9
    table_offsets = dev(np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    total = sum(rows)
    start = (torch.rand(total, D, device=DEV, dtype=torch.float64) * 0.02 - 0.01).to(dtype)
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=dtype), (total, D))
    cached_w.copy_(start)
    st_dtype = torch.float64 if dtype == torch.float64 else torch.float32
    plain_state = torch.zeros(total, device=DEV, dtype=st_dtype)
    cached_state = torch.zeros(total, device=DEV, dtype=st_dtype)
    cache = tc.RowCache(cached_w, num_sets * 64, "lru", stage_slots, deferred_write_back=deferred)
    weighted = mode.endswith("weighted")
    opt = "sgd" if mode == "sgd" else "approx_adagrad" if mode.startswith("approx") else "adagrad"
    served_uncached = served_staged = 0
    for step in range(6):
        indices, offsets = _draw_batch(rs, T, rows, B, L, 1.2)
        idx, off = dev(indices), dev(offsets)
        go = torch.randn(B, T, D, device=DEV, dtype=torch.float64).to(dtype)
        psw = torch.rand(indices.size, device=DEV, dtype=torch.float64).to(dtype) if weighted else None
        want = ext.forward(plain_w, table_offsets, idx, off, psw, 200, 1, False)
        if opt == "sgd":
            ext.backward_sgd(go, plain_w, table_offsets, idx, off, 0.05, 200, 1, False)
            want_g = None
        elif opt == "approx_adagrad":
            want_g = ext.backward_approx_adagrad(go, plain_w, table_offsets, idx, off, psw, plain_state, 0.05, 0.1,
                                                 200, False, 1)
        else:
            want_g = ext.backward_exact_adagrad(go, plain_w, table_offsets, idx, off, psw, plain_state, 0.05, 0.1,
                                                False, 1)
        cache.prepare(table_offsets, idx, off)
        got = cache.forward(table_offsets, idx, off, psw)
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
    if num_sets != 5:
        assert (served_uncached > 0) == (num_sets == 2 and stage_slots < 4096)
    assert (served_staged > 0) == (stage_slots > 0)
    ext.free_host_tensor(cached_w)


@pytest.mark.parametrize("stage_slots", [4096, 7])
def test_deferred_write_back_with_irregular_steps(stage_slots):
    """Deferred write-back rotates its staging areas by the plan's sequence number, not by the step
    number that stamps the recency words.  Step numbers that skip, an empty batch and a flush in
    the middle of the run must leave nothing behind: outputs, flushed table and state stay
    bit-identical to the run on device memory, and after every flush the host table itself is
    complete."""
    rs = np.random.RandomState(11)
    T, rows, B, L, D = 3, [700, 90, 3000], 48, 9, 64
    table_offsets = dev(np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    total = sum(rows)
    start = torch.rand(total, D, device=DEV) * 0.02 - 0.01
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV), (total, D))
    cached_w.copy_(start)
    plain_state = torch.zeros(total, device=DEV)
    cached_state = torch.zeros(total, device=DEV)
    cache = tc.RowCache(cached_w, 2 * 64, "lru", stage_slots, deferred_write_back=True)
    empty = (np.zeros(0, dtype=np.int32), np.zeros(T * B + 1, dtype=np.int32))
    staged = 0
    for step, skip in enumerate([0, 1, 0, 2, 1, 0, 3, 0]):
        cache.step += skip  # the next prepare uses step + 1
        if step == 5:
            indices, offsets = empty
        else:
            indices, offsets = _draw_batch(rs, T, rows, B, L, 1.2)
        idx, off = dev(indices), dev(offsets)
        cache.prepare(table_offsets, idx, off)
        got = cache.forward(table_offsets, idx, off, None)
        if indices.size == 0:
            assert not got.any()
        else:
            go = torch.randn(B, T, D, device=DEV)
            want = ext.forward(plain_w, table_offsets, idx, off, None, 200, 1, False)
            ext.backward_exact_adagrad(go, plain_w, table_offsets, idx, off, None, plain_state, 0.05, 0.1, False, 1)
            cache.backward("adagrad", go, None, cached_state, 0.05, 0.1)
            assert torch.equal(got, want), "forward output differs at step %d" % step
            staged += cache.stats()["staged"]
        if step in (3, 5):
            cache.flush()
            torch.cuda.synchronize()
            assert torch.equal(cached_w, plain_w), "host table incomplete after the flush at step %d" % step
    cache.flush()
    torch.cuda.synchronize()
    assert staged > 0
    assert torch.equal(cached_w, plain_w)
    assert torch.equal(cached_state, plain_state)
    ext.free_host_tensor(cached_w)


@pytest.mark.parametrize("seed", range(16))
def test_cached_training_random_sweep(seed):
    """Seeded random shapes of the cached-equals-uncached property: table counts and sizes, row
    widths (narrow, odd vector counts, wider than 64 vectors), dtype, optimizer, policy, cache
    and staging sizes from "nearly everything misses" to "everything fits", index skew."""
    rs = np.random.RandomState(700 + seed)
    T = int(rs.choice([1, 2, 5]))
    rows = [int(rs.choice([3, 60, 900, 6000])) for _ in range(T)]
    D = int(rs.choice([4, 12, 32, 64, 128, 260]))
    dtype = [torch.float32, torch.float16, torch.float64][seed % 3]
    mode = ["sgd", "adagrad", "adagrad_weighted"][(seed // 3) % 3]
    policy = ["lru", "lfu"][seed % 2]
    num_sets = int(rs.choice([1, 3, 17, 200]))
    stage_slots = int(rs.choice([0, 5, 300, 100000]))
    B, L, zipf = int(rs.choice([1, 30, 200])), int(rs.choice([1, 6, 25])), float(rs.choice([1.05, 1.3, 2.0]))
    table_offsets = dev(np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    total = sum(rows)
    start = (torch.rand(total, D, device=DEV, dtype=torch.float64) * 0.02 - 0.01).to(dtype)
    plain_w = start.clone()
    cached_w = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=dtype), (total, D))
    cached_w.copy_(start)
    st_dtype = torch.float64 if dtype == torch.float64 else torch.float32
    plain_state = torch.zeros(total, device=DEV, dtype=st_dtype)
    cached_state = torch.zeros(total, device=DEV, dtype=st_dtype)
    cache = tc.RowCache(cached_w, num_sets * 64, policy, stage_slots)
    weighted = mode.endswith("weighted")
    opt = "sgd" if mode == "sgd" else "adagrad"
    for step in range(5):
        indices, offsets = _draw_batch(rs, T, rows, B, L, zipf)
        idx, off = dev(indices), dev(offsets)
        go = torch.randn(B, T, D, device=DEV, dtype=torch.float64).to(dtype)
        psw = torch.rand(indices.size, device=DEV, dtype=torch.float64).to(dtype) if weighted else None
        want = ext.forward(plain_w, table_offsets, idx, off, psw, 200, 1, False)
        if opt == "sgd":
            ext.backward_sgd(go, plain_w, table_offsets, idx, off, 0.05, 200, 1, False)
            want_g = None
        else:
            want_g = ext.backward_exact_adagrad(go, plain_w, table_offsets, idx, off, psw, plain_state, 0.05, 0.1,
                                                False, 1)
        cache.prepare(table_offsets, idx, off)
        got = cache.forward(table_offsets, idx, off, psw)
        got_g = cache.backward(opt, go, psw, cached_state, 0.05, 0.1)
        assert torch.equal(got, want), "forward output differs at step %d" % step
        if weighted and indices.size:
            assert torch.equal(got_g, want_g)
        resident = cache.resident_keys()
        assert resident.numel() == torch.unique(resident).numel() <= num_sets * 64
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w)
    assert torch.equal(cached_state, plain_state)
    ext.free_host_tensor(cached_w)


@pytest.mark.parametrize("deferred", [False, True])
@pytest.mark.parametrize("stage_slots", [100000, 9])
def test_staging_leaves_cache_state_as_the_model_says(oracle, stage_slots, deferred):
    """A staged row is an uncached row of the model: tags, recency and frequency words are
    unchanged by staging; rows the model leaves uncached get distinct staging rows behind the
    slots (index = misses of the earlier sets + rank among the set's staged rows) until the
    staging area is full, the rest stay uncached.  With deferred write-back the steps stage into
    three areas in turn, and a row staged again is fetched from the staging row it had."""
    rs = np.random.RandomState(11)
    T, rows, B, L, D, num_sets = 3, [300, 5000, 40], 64, 12, 32, 2
    table_offsets = np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32)
    backing = torch.randn(sum(rows), D, device=DEV)
    cache = tc.RowCache(backing, num_sets * 64, "lru", stage_slots, deferred_write_back=deferred)
    model = oracle.CacheModel(num_sets, "lru")
    saw_uncached = False
    from_staging = 0
    for step in range(5):
        indices, offsets = _draw_batch(rs, T, rows, B, L, 1.15)
        cache.prepare(dev(table_offsets), dev(indices), dev(offsets))
        keys = np.unique(table_offsets[np.repeat(np.arange(T * B), np.diff(offsets)) // B] + indices)
        slots, evicted, stats = model.step(keys)
        got = cache.unique_slots().cpu().numpy()
        staged = got >= num_sets * 64
        np.testing.assert_array_equal(np.where(staged, -1, got), slots)
        area = cache.stage_area_base()   # first row of this step's area
        assert area == num_sets * 64 + (stage_slots * (cache.sequence % 3) if deferred else 0)
        assert np.unique(got[staged]).size == staged.sum()
        assert (got[staged] >= area).all() and (got[staged] < area + stage_slots).all()
        got_evicted = cache.evicted_keys().cpu().numpy()
        np.testing.assert_array_equal(got_evicted[~staged], evicted[~staged])
        assert (got_evicted[staged] == -1).all()
        np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)
        np.testing.assert_array_equal(cache.last_used.cpu().numpy(), model.last_used)
        np.testing.assert_array_equal(cache.use_count.cpu().numpy(), model.use_count)
        st = cache.stats()
        assert st["staged"] == staged.sum() and st["staged"] + st["uncached"] == stats[5]
        # the staging row holds a copy of the backing row after prepare()
        rows_now = cache.rows[torch.from_numpy(got[staged]).to(DEV).long()]
        assert torch.equal(rows_now, backing[torch.from_numpy(keys[staged]).to(DEV).long()])
        saw_uncached |= st["uncached"] > 0
        from_staging += st["from_staging"]
    assert saw_uncached == (stage_slots == 9)
    assert (from_staging > 0) == deferred
    cache.flush()
    torch.cuda.synchronize()


def test_cached_stochastic_rounding_equals_uncached_bit_exact():
    """fp16 weights with stochastic rounding: the random word of a weight is keyed by its place
    in the table, so the rows come out bit-identical whether they are updated in a cache slot, a
    staging row or the backing table."""
    import ctypes
    import tbe_native
    rs = np.random.RandomState(8)
    T, rows, B, L, D = 2, [900, 150], 40, 8, 64
    table_offsets = dev(np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    total = sum(rows)
    start = (torch.rand(total, D, device=DEV) * 0.02 - 0.01).half()
    plain_w, cached_w = start.clone(), start.clone()
    plain_state, cached_state = torch.zeros(total, device=DEV), torch.zeros(total, device=DEV)
    cache = tc.RowCache(cached_w, 2 * 64, "lru", stage_slots=50)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    for step in range(4):
        indices, offsets = _draw_batch(rs, T, rows, B, L, 1.2)
        idx, off = dev(indices), dev(offsets)
        go = torch.randn(B, T, D, device=DEV).half()
        lay = tbe_native.backward_workspace_layout(indices.size, D, tbe_native.DTYPE_F16, T)
        ws = torch.empty(lay.total_bytes, dtype=torch.uint8, device=DEV)
        tbe_native.check(tbe_native.load().tbe_backward_exact_adagrad_stochastic(
            vp(go), vp(plain_w), tbe_native.DTYPE_F16, total, 0, D, vp(table_offsets), T, vp(idx), indices.size,
            vp(off), B, None, vp(plain_state), 0.05, 0.1, None, 99, 4 * step, vp(ws), ws.numel(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        cache.prepare(table_offsets, idx, off)
        cache.backward("adagrad", go, None, cached_state, 0.05, 0.1, stochastic_rounding=(99, 4 * step))
        st = cache.stats()
        assert st["staged"] > 0 and st["uncached"] > 0 and st["hits"] + st["inserted"] > 0
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w) and torch.equal(cached_state, plain_state)
    # and the rounding is really stochastic: round-to-nearest gives other bits
    rn_w = start.clone()
    ext.backward_exact_adagrad(go, rn_w, table_offsets, idx, off, None, torch.zeros(total, device=DEV), 0.05, 0.1,
                               False, 1)
    assert not torch.equal(rn_w, start)


def test_cached_approx_adagrad_with_stochastic_rounding_equals_uncached_bit_exact():
    """The approximate Adagrad with stochastic rounding behind the cache (hot rows take the walk
    that draws a random word per element and occurrence): bit-identical to the uncached update."""
    import ctypes
    import tbe_native
    rs = np.random.RandomState(9)
    T, rows, B, L, D = 2, [900, 40], 64, 8, 64
    table_offsets = dev(np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    total = sum(rows)
    start = (torch.rand(total, D, device=DEV) * 0.02 - 0.01).half()
    plain_w, cached_w = start.clone(), start.clone()
    plain_state, cached_state = torch.zeros(total, device=DEV), torch.zeros(total, device=DEV)
    cache = tc.RowCache(cached_w, 2 * 64, "lru", stage_slots=50)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    longest = 0
    for step in range(4):
        indices, offsets = _draw_batch(rs, T, rows, B, L, 1.2)
        longest = max(longest, int(np.bincount(indices[offsets[B]:]).max()))
        idx, off = dev(indices), dev(offsets)
        go = torch.randn(B, T, D, device=DEV).half()
        lay = tbe_native.backward_workspace_layout(indices.size, D, tbe_native.DTYPE_F16, T)
        ws = torch.empty(lay.total_bytes, dtype=torch.uint8, device=DEV)
        tbe_native.check(tbe_native.load().tbe_backward_approx_adagrad(
            vp(go), vp(plain_w), tbe_native.DTYPE_F16, total, 0, D, vp(table_offsets), T, vp(idx), indices.size,
            vp(off), B, None, vp(plain_state), 0.05, 0.1, None, 1, 99, 4 * step, vp(ws), ws.numel(),
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
        cache.prepare(table_offsets, idx, off)
        cache.backward("approx_adagrad", go, None, cached_state, 0.05, 0.1, stochastic_rounding=(99, 4 * step))
        st = cache.stats()
        assert st["staged"] > 0 and st["uncached"] > 0 and st["hits"] + st["inserted"] > 0
    assert longest > 16, "no row long enough for the wavefront's walk"
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(cached_w, plain_w) and torch.equal(cached_state, plain_state)


def test_flush_before_any_step_and_empty_batch():
    backing = torch.randn(100, 16, device=DEV)
    before = backing.clone()
    cache = tc.RowCache(backing, 64)
    cache.flush()
    torch.cuda.synchronize()
    assert torch.equal(backing, before)
    to = dev(np.zeros(1, np.int32))
    cache.prepare(to, torch.zeros(0, dtype=torch.int32, device=DEV), dev(np.zeros(5, np.int32)))
    out = cache.forward(to, torch.zeros(0, dtype=torch.int32, device=DEV), dev(np.zeros(5, np.int32)))
    assert out.shape == (4, 1, 16) and not out.any()
    assert cache.stats()["unique_rows"] == 0


def test_module_host_cached_trains_like_device_module():
    """The drop-in module with managed=HOST_CACHED follows the same trajectory as the plain
    device module, and state_dict() sees the rows the cache holds."""
    T, E, D, B, L = 4, 500, 64, 32, 6
    torch.manual_seed(0)
    plain = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.1,
                                          eps=0.1).cuda()
    cached = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD,
                                           learning_rate=0.1, eps=0.1, managed=ops.EmbeddingLocation.HOST_CACHED,
                                           cache_slots=256).cuda()
    cached.embedding_weights.data.copy_(plain.embedding_weights.data)
    assert set(cached.state_dict()) == {"embedding_weights", "table_offsets", "optimizer_state"}
    rs = np.random.RandomState(1)
    for _ in range(5):
        p = make_problem(rs.randint(1 << 30), T, E, D, B, L, np.float32, zipf=1.2)
        idx, off, go = dev(p["indices"]), dev(p["offsets"]), dev(p["grad_output"])
        a = plain(idx, off)
        a.backward(go)
        b = cached(idx, off)
        b.backward(go)
        assert torch.equal(a, b)
    sd = cached.state_dict()
    torch.cuda.synchronize()
    assert torch.equal(sd["embedding_weights"], plain.embedding_weights.data)
    assert torch.equal(sd["optimizer_state"], plain.optimizer_state)
    hit_rate = cached.row_cache.stats()
    assert hit_rate["hits"] > 0 and hit_rate["unique_rows"] == hit_rate["hits"] + hit_rate["misses"]


def test_host_tensors_behave_like_device_tensors():
    """new_managed_tensor / new_host_mapped_tensor (table_batched_embeddings_cuda.cu:864-880):
    tagged as GPU tensors, usable by torch ops and by the kernels."""
    proto = torch.empty(1, device=DEV)
    for make in (ext.new_host_mapped_tensor, ext.new_managed_tensor):
        t = make(proto, (300, 32))
        assert t.is_cuda and t.dtype == torch.float32 and tuple(t.shape) == (300, 32)
        t.normal_()
        ref = t.clone()
        to = dev(np.zeros(1, np.int32))
        idx = torch.randint(0, 300, (20 * 5,), dtype=torch.int32, device=DEV)
        off = torch.arange(0, 101, 5, dtype=torch.int32, device=DEV)
        assert torch.equal(ext.forward(t, to, idx, off, None, 200, 1, False),
                           ext.forward(ref, to, idx, off, None, 200, 1, False))
        go = torch.randn(20, 1, 32, device=DEV)
        ext.backward_sgd(go, t, to, idx, off, 0.1, 200, 1, False)
        ext.backward_sgd(go, ref, to, idx, off, 0.1, 200, 1, False)
        torch.cuda.synchronize()
        assert torch.equal(t, ref)
        ext.free_host_tensor(t)
    half = ext.new_host_mapped_tensor(torch.empty(1, device=DEV, dtype=torch.float16), (8, 4))
    assert half.dtype == torch.float16
    ext.free_host_tensor(half)
