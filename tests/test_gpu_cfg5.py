"""The DLRM-style workload of configuration 5 (tables in pinned host memory behind the HBM row
cache; log-uniform row counts, clip(Poisson(30), 1, 100) bag lengths, per-table permuted
Zipf(1.1) indices re-drawn every step, exact SGD) as a tested configuration.

The reference's only counterpart is EmbeddingLocation.HOST_MAPPED
(table_batched_embeddings_ops.py:159-167, table_batched_embeddings_cuda.cu:797-812): the same
arithmetic on a host-resident table with no cache.  So the checks are (1) at reduced row counts,
every step against the oracle -- pooled output and updated table within 1e-5, cache state bit for
bit against the CPU model of the cache specification -- with the staging area twice the cache as
the benchmark uses it; (2) at full size, the property that ties the cache back to the reference:
the same batches on the same table held entirely in HBM without a cache give bit-identical
outputs and, after a flush, a bit-identical table, and the resident row set equals the model's."""
import numpy as np
import pytest
import torch

import bench
import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda:0")


def _module(w):
    m = ops.TableBatchedEmbeddingBags(w["T"], w["E"], w["D"], optimizer=ops.Optimizer.SGD, learning_rate=w["lr"],
                                      managed=ops.EmbeddingLocation.HOST_CACHED, cache_slots=w["cache_slots"],
                                      cache_stage_slots=w["stage_slots"]).cuda()
    m.embedding_weights.data.mul_(0.01)
    return m


def _unique_keys(table_offsets, indices, offsets, T, B):
    lengths = (offsets[1:] - offsets[:-1]).long()
    table_of_position = torch.repeat_interleave(torch.arange(T, device=DEV), lengths.view(T, B).sum(1))
    return torch.unique(table_offsets.long()[table_of_position] + indices.long())


def _check_cache_against_model(cache, model, keys, num_slots):
    """Slots, evictions, tags, recency / frequency words and counters of the step that was just
    prepared equal the model's.  A row the model leaves uncached is either staged (slot in the
    staging area) or uncached on the device."""
    slots, evicted, stats = model.step(keys)
    got_slots = cache.unique_slots().cpu().numpy()
    np.testing.assert_array_equal(cache.unique_keys().cpu().numpy(), keys)
    cached = slots >= 0
    np.testing.assert_array_equal(got_slots[cached], slots[cached])
    assert ((got_slots[~cached] == -1) | (got_slots[~cached] >= num_slots)).all()
    staged = got_slots >= num_slots
    assert np.unique(got_slots[staged]).size == staged.sum(), "two rows share a staging row"
    got_evicted = cache.evicted_keys().cpu().numpy()
    np.testing.assert_array_equal(got_evicted[~staged], evicted[~staged])
    assert (got_evicted[staged] == -1).all()  # a staged row is fetched into its staging row, nothing is evicted
    np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)
    np.testing.assert_array_equal(cache.last_used.cpu().numpy(), model.last_used)
    np.testing.assert_array_equal(cache.use_count.cpu().numpy(), model.use_count)
    np.testing.assert_array_equal(cache.resident_keys().cpu().numpy(), model.resident())
    st = cache.stats()
    assert [st[k] for k in ("unique_rows", "hits", "misses", "inserted", "written_back")] == stats[:5].tolist()
    assert st["uncached"] + st["staged"] == stats[5] and st["staged"] == staged.sum()
    return st


@pytest.mark.parametrize("prefetch", [False, True])
def test_cfg5_scaled_down_every_step_against_oracle_and_cache_model(oracle, prefetch):
    """12 steps of the configuration-5 generator at reduced sizes: 26 tables of 100 ... 100 k rows,
    512 bags per table, a 4096-slot LRU cache with a staging area twice its size.  With `prefetch`
    every batch is planned while the batch before it is between its forward and its backward, and
    the flush after every step finds that planned batch waiting."""
    w = bench.make_cfg5_workload(seed=0, B=512, row_range=(1e2, 1e5), cache_slots=1 << 12, stage_slots=1 << 13)
    T, B, D = w["T"], w["B"], w["D"]
    assert w["stage_slots"] == 2 * w["cache_slots"]
    module = _module(w)
    cache = module.row_cache
    model = oracle.CacheModel(w["cache_slots"] // 64, "lru")
    table_offsets = module.table_offsets.cpu().numpy()
    gen = torch.Generator(device=DEV).manual_seed(1)
    w_ref = module.embedding_weights.detach().cpu().numpy().copy()
    seen_staged = seen_hits = seen_written_back = 0
    batches = [bench.draw_cfg5_batch(torch, w, step, DEV) for step in range(12)]
    if prefetch:
        module.prefetch(*batches[0])
    for step in range(12):
        indices, offsets = batches[step]
        lengths = (offsets[1:] - offsets[:-1])
        assert int(lengths.min()) >= 1 and int(lengths.max()) <= 100
        grad_output = torch.randn(B, T, D, device=DEV, generator=gen)
        out = module(indices, offsets)
        keys = _unique_keys(module.table_offsets, indices, offsets, T, B).cpu().numpy().astype(np.int32)
        st = _check_cache_against_model(cache, model, keys, w["cache_slots"])
        seen_staged += st["staged"]
        seen_hits += st["hits"]
        seen_written_back += st["written_back"]
        idx_np, off_np, go_np = indices.cpu().numpy(), offsets.cpu().numpy(), grad_output.cpu().numpy()
        want = oracle.forward(w_ref, table_offsets, idx_np, off_np)
        scale = np.abs(want).max()
        np.testing.assert_allclose(out.detach().cpu().numpy(), want, rtol=1e-5, atol=1e-5 * scale,
                                   err_msg="pooled output, step %d" % step)
        if prefetch and step + 1 < 12:
            module.prefetch(*batches[step + 1])
        out.backward(grad_output)
        oracle.backward("sgd", go_np, w_ref, table_offsets, idx_np, off_np, w["lr"])
        module.flush_cache()
        got = module.embedding_weights.detach().cpu().numpy()
        np.testing.assert_allclose(got, w_ref, rtol=1e-5, atol=1e-5 * np.abs(w_ref).max(),
                                   err_msg="table after step %d" % step)
        w_ref = got.copy()  # every step is compared on its own: no drift between the two sides
    # the workload exercises every path of the cache: hits, evictions with write-back, staging
    assert seen_hits > 0 and seen_written_back > 0 and seen_staged > 0


def test_cached_module_refuses_a_backward_whose_plan_was_replaced():
    """Two forwards before a backward: the first graph's backward would run on the second batch's
    plan and slots, so it raises; the second one's runs.  A forward under no_grad in between is
    the same case."""
    w = bench.make_cfg5_workload(seed=2, T=3, B=64, row_range=(1e2, 1e3), cache_slots=128, stage_slots=256)
    module = _module(w)
    i0, o0 = bench.draw_cfg5_batch(torch, w, 0, DEV)
    i1, o1 = bench.draw_cfg5_batch(torch, w, 1, DEV)
    go = torch.randn(w["B"], w["T"], w["D"], device=DEV)
    first = module(i0, o0)
    second = module(i1, o1)
    with pytest.raises(RuntimeError, match="prepared for another batch"):
        first.backward(go)
    second.backward(go)
    third = module(i0, o0)
    with torch.no_grad():
        module(i1, o1)
    with pytest.raises(RuntimeError, match="prepared for another batch"):
        third.backward(go)
    out = module(i0, o0)
    with pytest.raises(RuntimeError, match="grad_output must be"):
        module.row_cache.backward("sgd", go[:, :2], None, None, 0.01, 0.0, plan_id=module.row_cache.plan_id)
    out.backward(go)


def test_cached_module_serves_a_loaded_checkpoint_not_its_stale_rows():
    """train -> load_state_dict -> forward: the rows that were resident before the load must not
    shadow the loaded table, and must not be written over it later."""
    w = bench.make_cfg5_workload(seed=3, T=4, B=128, row_range=(1e2, 2e3), cache_slots=1 << 10, stage_slots=1 << 11)
    T, B, D = w["T"], w["B"], w["D"]
    module = _module(w)
    go = torch.randn(B, T, D, device=DEV)
    for step in range(3):
        indices, offsets = bench.draw_cfg5_batch(torch, w, step, DEV)
        module(indices, offsets).backward(go)
    assert int((module.row_cache.tags >= 0).sum()) > 0
    checkpoint = {k: v.clone() for k, v in module.state_dict().items()}
    checkpoint["embedding_weights"] = torch.full_like(checkpoint["embedding_weights"], 0.5)
    module.load_state_dict(checkpoint)
    assert int((module.row_cache.tags >= 0).sum()) == 0
    indices, offsets = bench.draw_cfg5_batch(torch, w, 7, DEV)
    out = module(indices, offsets)
    lengths = (offsets[1:] - offsets[:-1]).view(T, B).t().float()          # [B][T] rows per bag
    torch.testing.assert_close(out, (0.5 * lengths).unsqueeze(-1).expand(B, T, D), rtol=1e-6, atol=0)
    out.backward(torch.zeros_like(go))                                     # an update that changes nothing
    module.flush_cache()
    assert bool((module.embedding_weights.detach() == 0.5).all())


def test_host_tensor_is_released_with_its_storage():
    """new_host_mapped_tensor / new_managed_tensor: the allocation goes when the last tensor on
    its storage goes (the reference attaches deleters, table_batched_embeddings_cuda.cu:795-835);
    free_host_tensor releases it early, once."""
    released = []
    observer = released.append
    ext.release_observers.append(observer)
    try:
        proto = torch.empty(1, device=DEV)
        for make in (ext.new_host_mapped_tensor, ext.new_managed_tensor):
            t = make(proto, (1000, 8))
            address = t.data_ptr()
            before = len(released)  # (an address may come back: count releases instead of looking for it)
            t.fill_(3.0)
            view = t[10:20]
            param = torch.nn.Parameter(t)
            del t
            assert len(released) == before and float(view.sum()) == 240.0   # views keep the storage alive
            del view
            assert len(released) == before
            del param
            assert len(released) == before + 1 and released[-1] == address
        t = ext.new_host_mapped_tensor(proto, (16, 4))
        address = t.data_ptr()
        ext.free_host_tensor(t)
        assert released[-1] == address and released.count(address) == 1
        with pytest.raises(RuntimeError, match="not allocated by this module"):
            ext.free_host_tensor(t)
        del t                                                               # no second release
        assert released.count(address) == 1
        module = _module(bench.make_cfg5_workload(seed=4, T=2, B=8, row_range=(1e2, 2e2), cache_slots=64,
                                                  stage_slots=64))
        address = module.embedding_weights.data_ptr()
        del module
        import gc
        gc.collect()
        assert released[-1] == address, "dropping a HOST_CACHED module must release its pinned table"
    finally:
        ext.release_observers.remove(observer)


@pytest.mark.timeout(900)
def test_cfg5_full_size_cached_run_equals_uncached_run_bit_for_bit(oracle):
    """Configuration 5 at its full size (69.6 M rows = 35.6 GB in pinned host memory, 2^22-slot
    LRU cache + 3 x 2^23 staging rows, 65 536 bags per table, ~51 M lookups per step), 5 steps: two
    planned inside the step, three planned one step ahead (RowCache.prefetch).  The table also fits
    in HBM, so the same batches run on a plain device copy without a cache: outputs of every step
    and the flushed table are bit-identical, and the set of resident rows after every batch's plan
    equals the CPU model's."""
    free, _ = torch.cuda.mem_get_info()
    w = bench.make_cfg5_workload(seed=0)
    table_bytes = sum(w["E"]) * w["D"] * 4
    if free < table_bytes + (30 << 30):
        pytest.skip("needs %.0f GB of free HBM" % ((table_bytes + (30 << 30)) / 1e9))
    T, B, D = w["T"], w["B"], w["D"]
    print("cfg5 full size: allocating %.1f GB pinned + the same in HBM" % (table_bytes / 1e9), flush=True)
    module = _module(w)
    cache = module.row_cache
    plain = module.embedding_weights.detach().clone()
    assert plain.data_ptr() != module.embedding_weights.data_ptr()
    model = oracle.CacheModel(w["cache_slots"] // 64, "lru")
    gen = torch.Generator(device=DEV).manual_seed(5)
    grad_output = torch.randn(B, T, D, device=DEV, generator=gen)
    steps, plain_steps = 5, 2
    batches = [bench.draw_cfg5_batch(torch, w, step, DEV) for step in range(steps)]
    keys_of = lambda b: _unique_keys(module.table_offsets, b[0], b[1], T, B).cpu().numpy().astype(np.int32)

    def check_model(step):
        """the cache's decisions for batch `step` are made: tags and resident rows equal the model's"""
        model.step(keys_of(batches[step]))
        np.testing.assert_array_equal(cache.resident_keys().cpu().numpy(), model.resident())
        np.testing.assert_array_equal(cache.tags.cpu().numpy(), model.tags)

    for step in range(steps):
        indices, offsets = batches[step]
        print("cfg5 full size: step %d, %d lookups%s" % (step, indices.numel(),
                                                         "" if step < plain_steps else ", planned ahead"), flush=True)
        if step >= plain_steps and step + 1 < steps:
            # from the third step on every batch is planned one step ahead, before this step's forward
            module.prefetch(*batches[step + 1])
        out = module(indices, offsets)
        if step < plain_steps:
            check_model(step)
            if step + 1 == plain_steps:
                module.prefetch(*batches[step + 1])
                check_model(step + 1)
        elif step + 1 < steps:
            check_model(step + 1)
        want = ext.forward(plain, module.table_offsets, indices, offsets, None, 200, 1, False)
        assert torch.equal(out.detach(), want), "pooled output differs at step %d" % step
        st = cache.stats()
        assert st["unique_rows"] == keys_of(batches[step]).size and st["staged"] > 0
        # a staging row is numbered by the misses of the sets before it, so the area holds every
        # unplaced row once a step misses fewer rows than it has: from the second step on
        assert st["uncached"] == 0 or (step == 0 and st["misses"] > w["stage_slots"])
        assert st["no_landing_row"] == 0 or step == 0
        out.backward(grad_output)
        ext.backward_sgd(grad_output, plain, module.table_offsets, indices, offsets, w["lr"], 200, 1, False)
        del out, want
    module.flush_cache()
    torch.cuda.synchronize()
    assert torch.equal(module.embedding_weights.detach(), plain), "flushed table differs from the uncached run"
