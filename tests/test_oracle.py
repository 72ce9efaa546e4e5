"""Pins the CPU oracle (oracle/tbe_oracle.c) before anything is compared with it.

The reference holds no golden vectors for this path (every reference test draws random
data and compares with torch.nn.EmbeddingBag at run time), so the oracle is pinned by:
  * committed fixtures produced with the reference test-suite's own oracle -- per-table
    torch.nn.EmbeddingBag + the Python optimizer (tests/golden/make_golden.py);
  * library routines: numpy's stable argsort, numpy.unique, numpy.float16 conversion;
  * closed forms and special cases (single-lookup bags copy rows, unit weights equal the
    unweighted sum, a row hit once by Adagrad has state |g|^2, untouched rows keep their
    bits, linearity of the SGD update in the gradient);
  * brute force on tiny inputs.
Each check is chosen so that a dropped term, a transposed [B][T] / [T][B] index, a wrong
sort bit range or a multiplier built from the old state fails it.
"""
import numpy as np
import pytest

from conftest import GOLDEN_CASES, load_golden, make_problem


def table_offsets_of(g):
    return (np.arange(g["T"]) * g["E"]).astype(np.int32)


# ------------------------------------------------------------------ fixtures
@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_forward_matches_embeddingbag_fixture(oracle, name):
    g = load_golden(name)
    out = oracle.forward(g["weights"], table_offsets_of(g), g["indices"], g["offsets"], g.get("per_sample_weights"))
    assert out.shape == (g["B"], g["T"], g["D"])
    tol = 2e-3 if g["weights"].dtype == np.float16 else 1e-5
    scale = np.abs(g["expected_output"]).max()
    np.testing.assert_allclose(out.astype(np.float64), g["expected_output"], rtol=tol, atol=tol * scale)


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_backward_matches_embeddingbag_fixture(oracle, name):
    g = load_golden(name)
    w = g["weights"].copy()
    state = np.zeros(w.shape[0], np.float64 if w.dtype == np.float64 else np.float32)
    r = oracle.backward(g["optimizer"], g["grad_output"], w, table_offsets_of(g), g["indices"], g["offsets"],
                        g["lr"], g["eps"], state, g.get("per_sample_weights"))
    half = w.dtype == np.float16
    tol = 1e-2 if half else 1e-5
    scale = np.abs(g["expected_weights"]).max()
    np.testing.assert_allclose(w.astype(np.float64), g["expected_weights"], rtol=tol, atol=tol * scale)
    if g["optimizer"] == "adagrad":
        np.testing.assert_allclose(state.astype(np.float64), g["expected_state"], rtol=1e-3 if half else 1e-5,
                                   atol=1e-30)
    if "expected_grad_psw" in g:
        gs = np.abs(g["expected_grad_psw"]).max()
        np.testing.assert_allclose(r["grad_psw"].astype(np.float64), g["expected_grad_psw"], rtol=tol,
                                   atol=tol * gs)


def test_live_embeddingbag_agrees(oracle):
    """Same comparison against torch.nn.EmbeddingBag computed now (guards a stale fixture)."""
    torch = pytest.importorskip("torch")
    p = make_problem(11, T=3, E=40, D=24, B=21, L=7, dtype=np.float32, weighted=True, zipf=1.3)
    out = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"], p["per_sample_weights"])
    for t in range(p["T"]):
        lo, hi = p["offsets"][t * p["B"]], p["offsets"][(t + 1) * p["B"]]
        w = torch.from_numpy(p["weights"][t * 40:(t + 1) * 40].copy())
        y = torch.nn.functional.embedding_bag(
            torch.from_numpy(p["indices"][lo:hi].astype(np.int64)), w,
            torch.from_numpy((p["offsets"][t * p["B"]:(t + 1) * p["B"]] - lo).astype(np.int64)), mode="sum",
            per_sample_weights=torch.from_numpy(p["per_sample_weights"][lo:hi].copy()))
        np.testing.assert_allclose(out[:, t, :], y.numpy(), rtol=1e-5, atol=1e-8)


# ------------------------------------------------------------- fp16 rounding
def test_half_conversions_match_numpy(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    as_float = bits.view(np.float16).astype(np.float32)
    for b in range(0, 65536, 1):
        f = oracle.half_to_float(b)
        if np.isnan(as_float[b]):
            assert np.isnan(f)
        else:
            assert f == as_float[b] and np.signbit(f) == np.signbit(as_float[b])
    rs = np.random.RandomState(0)
    vals = np.concatenate([rs.randn(20000).astype(np.float32) * 10.0 ** rs.randint(-9, 6, size=20000),
                           np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e-8, 5.96e-8, 2.98e-8, 2.9802322e-8,
                                     6.1e-5, 6.09e-5, np.inf, -np.inf], dtype=np.float32),
                           # exact ties between neighbouring halves
                           ((bits[:0x7bff].view(np.float16).astype(np.float64) +
                             (bits[:0x7bff] + 1).astype(np.uint16).view(np.float16).astype(np.float64)) / 2)
                           .astype(np.float32)]).astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.float_to_half(v) for v in vals], dtype=np.uint16)
    np.testing.assert_array_equal(got, want)


# ------------------------------------------------------- integer stages, bit-exact
@pytest.mark.parametrize("seed,n,hi,end_bit", [(0, 0, 10, 4), (1, 1, 10, 4), (2, 5000, 7, 3), (3, 70000, 1 << 23, 23),
                                               (4, 4097, 300, 9), (5, 33333, 1 << 17, 25)])
def test_sort_is_stable_argsort(oracle, seed, n, hi, end_bit):
    rs = np.random.RandomState(seed)
    keys = rs.randint(0, hi, size=n).astype(np.int32)
    ks, vs = oracle.sort_pairs(keys, None, end_bit)
    order = np.argsort(keys, kind="stable")
    np.testing.assert_array_equal(ks, keys[order])
    np.testing.assert_array_equal(vs, order.astype(np.int32))


def test_sort_ignores_bits_above_end_bit(oracle):
    # CUB's contract: only bits [0, end_bit) take part; equal low bits keep input order
    keys = np.array([0x105, 0x003, 0x205, 0x103, 0x001], np.int32)
    ks, vs = oracle.sort_pairs(keys, None, 8)
    np.testing.assert_array_equal(vs, [4, 1, 3, 0, 2])
    np.testing.assert_array_equal(ks, keys[[4, 1, 3, 0, 2]])


def test_sort_brute_force_tiny(oracle):
    rs = np.random.RandomState(7)
    for _ in range(50):
        n = rs.randint(0, 12)
        keys = rs.randint(0, 4, size=n).astype(np.int32)
        vals = rs.randint(0, 1000, size=n).astype(np.int32)
        ks, vs = oracle.sort_pairs(keys, vals, 2)
        want = sorted(zip(keys.tolist(), range(n)), key=lambda kv: kv[0])  # python's sort is stable
        assert ks.tolist() == [k for k, _ in want]
        assert vs.tolist() == [int(vals[i]) for _, i in want]


@pytest.mark.parametrize("seed,n,hi", [(0, 0, 5), (1, 1, 5), (2, 1000, 3), (3, 50000, 40000), (4, 777, 1)])
def test_segments_match_numpy_unique(oracle, seed, n, hi):
    keys = np.sort(np.random.RandomState(seed).randint(0, hi, size=n)).astype(np.int32)
    starts = oracle.segments(keys)
    uniq, first = np.unique(keys, return_index=True)
    np.testing.assert_array_equal(starts[:-1], first.astype(np.int32))
    assert starts[-1] == n and starts.size == uniq.size + 1


def test_linearize_closed_form(oracle):
    p = make_problem(3, T=4, E=0, D=4, B=9, L=6, dtype=np.float32, rows=[5, 17, 3, 40])
    keys, b_t, idx = oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])
    bag = np.repeat(np.arange(p["T"] * p["B"]), np.diff(p["offsets"]))
    np.testing.assert_array_equal(b_t, bag)
    np.testing.assert_array_equal(idx, np.arange(p["n"]))
    np.testing.assert_array_equal(keys, p["table_offsets"][bag // p["B"]] + p["indices"])


def test_construct_offsets_closed_form(oracle):
    # the check of test_table_batched_embeddings.py:97-105
    rs = np.random.RandomState(5)
    T, B = 7, 13
    lengths = rs.randint(1, 20, size=(T, B))
    starts = np.concatenate([np.zeros((T, 1), int), np.cumsum(lengths, axis=1)[:, :-1]], axis=1).astype(np.int32)
    totals = lengths.sum(axis=1).astype(np.int32)
    out = oracle.construct_offsets(starts, totals)
    assert out[0] == 0
    np.testing.assert_array_equal(out[1:], lengths.reshape(-1))
    np.testing.assert_array_equal(np.cumsum(out), np.concatenate([[0], np.cumsum(lengths.reshape(-1))]))


# ------------------------------------------------------------- special cases
def test_single_lookup_bags_copy_rows_bit_exact(oracle):
    p = make_problem(1, T=3, E=25, D=12, B=10, L=1, dtype=np.float32, ragged=False)
    out = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"])
    for t in range(3):
        for b in range(10):
            row = p["table_offsets"][t] + p["indices"][t * 10 + b]
            assert out[b, t].tobytes() == p["weights"][row].tobytes()  # [B][T] order, not [T][B]


def test_empty_bags_give_zeros_and_unit_weights_equal_unweighted(oracle):
    p = make_problem(2, T=2, E=30, D=8, B=50, L=3, dtype=np.float32)
    out = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"])
    empty = np.diff(p["offsets"]) == 0
    assert empty.any()
    for bag in np.nonzero(empty)[0]:
        assert not out[bag % 50, bag // 50].any()
    ones = np.ones(p["n"], np.float32)
    out_w = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"], ones)
    assert out_w.tobytes() == out.tobytes()


def test_sgd_untouched_rows_keep_bits_and_update_is_linear(oracle):
    p = make_problem(4, T=2, E=200, D=16, B=12, L=5, dtype=np.float64, zipf=1.1)
    w1, w2, w12 = p["weights"].copy(), p["weights"].copy(), p["weights"].copy()
    g1 = p["grad_output"]
    g2 = np.random.RandomState(9).randn(*g1.shape)
    for w, g in ((w1, g1), (w2, g2), (w12, g1 + g2)):
        oracle.backward("sgd", g, w, p["table_offsets"], p["indices"], p["offsets"], 0.25)
    keys = oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])[0]
    untouched = np.setdiff1d(np.arange(400), keys)
    assert untouched.size and w1[untouched].tobytes() == p["weights"][untouched].tobytes()
    np.testing.assert_allclose((w1 - p["weights"]) + (w2 - p["weights"]), w12 - p["weights"], rtol=1e-12, atol=1e-15)
    # closed form: w - lr * scatter-add of gradient rows
    G = np.zeros_like(p["weights"])
    bag = np.repeat(np.arange(24), np.diff(p["offsets"]))
    np.add.at(G, keys, g1[bag % 12, bag // 12])
    np.testing.assert_allclose(w1, p["weights"] - 0.25 * G, rtol=1e-12, atol=1e-15)


def test_adagrad_single_hit_closed_form_and_second_step_uses_new_state(oracle):
    # one table, one bag, one lookup: state = |g|^2, w -= lr / (|g| + eps) * g
    w = np.full((3, 4), 0.5, np.float64)
    g = np.array([[[3.0, 0.0, 4.0, 0.0]]])
    state = np.zeros(3)
    args = (np.array([0], np.int32), np.array([1], np.int32), np.array([0, 1], np.int32))
    oracle.backward("adagrad", g, w, *args, lr=0.5, eps=0.2, optimizer_state=state)
    assert state.tolist() == [0.0, 25.0, 0.0]
    np.testing.assert_allclose(w[1], 0.5 - 0.5 / (5.0 + float(np.float32(0.2))) * g[0, 0], rtol=1e-15)
    assert (w[0] == 0.5).all() and (w[2] == 0.5).all()
    # second step: multiplier is built from old + new (tbe.cu:453-454), i.e. sqrt(50), not sqrt(25)
    before = w[1].copy()
    oracle.backward("adagrad", g, w, *args, lr=0.5, eps=0.2, optimizer_state=state)
    assert state[1] == 50.0
    np.testing.assert_allclose(w[1], before - 0.5 / (np.sqrt(50.0) + float(np.float32(0.2))) * g[0, 0],
                               rtol=1e-15)


def test_grad_psw_is_dot_with_weights_before_update(oracle):
    p = make_problem(6, T=2, E=10, D=8, B=6, L=4, dtype=np.float64, weighted=True, zipf=1.5)
    w = p["weights"].copy()
    state = np.zeros(20)
    r = oracle.backward("adagrad", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.3, 0.1,
                        state, p["per_sample_weights"])
    keys = oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])[0]
    bag = np.repeat(np.arange(12), np.diff(p["offsets"]))
    want = np.einsum("nd,nd->n", p["weights"][keys], p["grad_output"][bag % 6, bag // 6])
    np.testing.assert_allclose(r["grad_psw"], want, rtol=1e-12, atol=1e-18)
    # duplicates make rows change during the pass; the result must still use the old rows
    assert np.unique(keys).size < keys.size


def test_backward_intermediates_are_sort_and_unique_of_keys(oracle):
    p = make_problem(8, T=3, E=0, D=4, B=20, L=6, dtype=np.float32, zipf=1.2, rows=[7, 300, 41])
    w = p["weights"].copy()
    r = oracle.backward("sgd", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.1)
    keys = oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])[0]
    order = np.argsort(keys, kind="stable")
    np.testing.assert_array_equal(r["keys_sorted"], keys[order])
    np.testing.assert_array_equal(r["positions_sorted"], order)
    np.testing.assert_array_equal(r["segment_starts"][:-1], np.unique(keys[order], return_index=True)[1])


# ------------------------------------------------------------------ row cache model
# The reference has no cache; these pin oracle/lxu_cache_model.c to this repository's own
# specification (include/tbe_hip.h, above tbe_cache_t).  Parity with the reference is unpinned.
def _brute_force_cache_step(state, num_sets, policy, step, keys, set_of):
    """Direct transcription of the specification with Python lists."""
    tags, used, count = state
    slots, evicted = [-1] * len(keys), [-2] * len(keys)
    for u, key in enumerate(keys):                      # phase 1: hits
        base = set_of(key, num_sets) * 64
        for w in range(64):
            if tags[base + w] == key:
                slots[u] = base + w
                used[base + w] = step
                count[base + w] += 1
    for u, key in enumerate(keys):                      # phase 2: inserts, ascending key order
        if slots[u] >= 0:
            continue
        base = set_of(key, num_sets) * 64
        free = [(count[base + w] if policy == "lfu" else used[base + w], w) for w in range(64)
                if used[base + w] < step]
        if not free:
            continue
        _, w = min(free)
        evicted[u] = tags[base + w] if tags[base + w] >= 0 else -1
        tags[base + w], used[base + w], count[base + w] = key, step, 1
        slots[u] = base + w
    return slots, evicted


@pytest.mark.parametrize("policy", ["lru", "lfu"])
@pytest.mark.parametrize("num_sets,universe", [(1, 150), (3, 400), (8, 600)])
def test_cache_model_matches_brute_force(oracle, policy, num_sets, universe):
    rs = np.random.RandomState(num_sets)
    model = oracle.CacheModel(num_sets, policy)
    state = ([-1] * (64 * num_sets), [0] * (64 * num_sets), [0] * (64 * num_sets))
    for step in range(1, 9):
        keys = np.unique((rs.zipf(1.3, size=rs.randint(1, 300)) % universe).astype(np.int32))
        slots, evicted, stats = model.step(keys)
        want_slots, want_evicted = _brute_force_cache_step(state, num_sets, policy, step, keys.tolist(),
                                                           oracle.cache_set_of)
        assert slots.tolist() == want_slots and evicted.tolist() == want_evicted
        assert model.tags.tolist() == state[0] and model.last_used.tolist() == state[1]
        assert model.use_count.tolist() == state[2]
        # invariants
        resident = model.tags[model.tags >= 0]
        assert np.unique(resident).size == resident.size <= 64 * num_sets
        assert stats[0] == keys.size and stats[1] + stats[2] == keys.size
        assert stats[3] + stats[5] == stats[2] and stats[4] == (evicted >= 0).sum()
        assert ((slots >= 0) | (evicted == -2)).all()
        assert np.isin(keys[slots >= 0], resident).all()          # used this step => still resident
        assert (model.tags[slots[slots >= 0]] == keys[slots >= 0]).all()


def test_cache_hash_spreads_and_is_in_range(oracle):
    sets = np.array([oracle.cache_set_of(k, 1000) for k in range(20000)])
    assert sets.min() >= 0 and sets.max() < 1000
    assert np.bincount(sets, minlength=1000).max() < 60       # 20 expected per set
    assert oracle.cache_set_of(12345, 1) == 0


def test_cache_lru_and_lfu_pick_different_victims(oracle):
    # one set: fill it with 64 keys, use key A often and long ago, key B once and recently
    for policy, expect_gone in (("lru", 0), ("lfu", 1)):
        m = oracle.CacheModel(1, policy)
        m.step(np.arange(64, dtype=np.int32))                     # step 1: all inserted
        for _ in range(3):
            m.step(np.array([0], np.int32))                       # steps 2-4: key 0 used 3 more times
        m.step(np.arange(1, 64, dtype=np.int32))                  # step 5: everything but key 0
        m.step(np.arange(2, 64, dtype=np.int32))                  # step 6: everything but keys 0, 1
        m.step(np.arange(2, 64, dtype=np.int32))                  # step 7: same (their counts pass key 0's)
        slots, evicted, _ = m.step(np.array([1000], np.int32))    # step 8: one new key needs a victim
        # LRU evicts key 0 (last used in step 4, key 1 in step 5); LFU evicts key 1 (2 uses < key 0's 4)
        assert evicted.tolist() == [expect_gone]
        assert 1000 in m.resident() and expect_gone not in m.resident()


def test_cache_rows_used_in_a_step_are_never_evicted_in_it(oracle):
    m = oracle.CacheModel(1, "lru")
    m.step(np.arange(64, dtype=np.int32))
    slots, evicted, stats = m.step(np.arange(0, 100, dtype=np.int32))   # 64 hits, 36 misses, no free way
    assert stats.tolist() == [100, 64, 36, 0, 0, 36]
    assert (slots[64:] == -1).all() and (evicted == -2).all()
    assert m.resident().tolist() == list(range(64))


# ------------------------------------------------------------ per-table dimension
@pytest.mark.parametrize("weighted", [False, True])
def test_mixed_dim_matches_embeddingbag(oracle, weighted):
    """The check of test_table_batched_embeddings.py:395-521: one torch.nn.EmbeddingBag per
    table with its own (rows, dim); forward, Adagrad state and weights."""
    torch = pytest.importorskip("torch")
    from conftest import make_mixed_problem
    embeddings = [(30, 8), (7, 32), (100, 4), (16, 12)]
    p = make_mixed_problem(21, embeddings, B=11, L=6, dtype=np.float32, weighted=weighted, zipf=1.3)
    out = oracle.forward_mixed(p["weights"], p["table_offsets"], p["dim_offsets"], p["indices"], p["offsets"],
                               p["per_sample_weights"])
    w = p["weights"].copy()
    state = np.zeros(sum(p["rows"]), np.float32)
    lr, eps = 0.5, 0.2
    gpsw = oracle.backward_mixed("adagrad", p["grad_output"], w, p["table_offsets"], p["table_dim_offsets"],
                                 p["dim_offsets"], p["indices"], p["offsets"], lr, eps, state,
                                 p["per_sample_weights"])
    for t, (E, D) in enumerate(embeddings):
        lo, hi = p["offsets"][t * p["B"]], p["offsets"][(t + 1) * p["B"]]
        bag = torch.nn.EmbeddingBag(E, D, mode="sum", sparse=True)
        w_t = p["weights"][p["table_offsets"][t]:p["table_offsets"][t + 1]].reshape(E, D)
        bag.weight.data.copy_(torch.from_numpy(w_t))
        kw = {}
        if weighted:
            psw_t = torch.from_numpy(p["per_sample_weights"][lo:hi].copy()).requires_grad_(True)
            kw["per_sample_weights"] = psw_t
        y = bag(torch.from_numpy(p["indices"][lo:hi].astype(np.int64)),
                torch.from_numpy((p["offsets"][t * p["B"]:(t + 1) * p["B"]] - lo).astype(np.int64)), **kw)
        d0, d1 = p["dim_offsets"][t], p["dim_offsets"][t + 1]
        np.testing.assert_allclose(out[:, d0:d1], y.detach().numpy(), rtol=1e-5, atol=1e-8)
        y.backward(torch.from_numpy(p["grad_output"][:, d0:d1].copy()))
        grad = bag.weight.grad.to_dense()
        st = grad.pow(2).sum(1)
        r0, r1 = p["table_dim_offsets"][t], p["table_dim_offsets"][t + 1]
        np.testing.assert_allclose(state[r0:r1], st.numpy(), rtol=1e-5, atol=1e-12)
        want_w = torch.addcdiv(bag.weight.detach(), grad, (st.sqrt() + eps).view(E, 1), value=-lr)
        got_w = w[p["table_offsets"][t]:p["table_offsets"][t + 1]].reshape(E, D)
        np.testing.assert_allclose(got_w, want_w.numpy(), rtol=1e-5, atol=1e-7)
        if weighted:
            np.testing.assert_allclose(gpsw[lo:hi], psw_t.grad.numpy(), rtol=1e-5, atol=1e-8)


def test_mixed_dim_with_equal_dims_equals_uniform_path(oracle):
    from conftest import make_mixed_problem
    p = make_mixed_problem(22, [(40, 16)] * 3, B=9, L=5, dtype=np.float64)
    out = oracle.forward_mixed(p["weights"], p["table_offsets"], p["dim_offsets"], p["indices"], p["offsets"])
    uni = oracle.forward(p["weights"].reshape(120, 16), p["table_dim_offsets"][:-1], p["indices"], p["offsets"])
    assert out.tobytes() == np.ascontiguousarray(uni.reshape(9, 48)).tobytes()
    w1, w2 = p["weights"].copy(), p["weights"].copy().reshape(120, 16)
    oracle.backward_mixed("sgd", p["grad_output"], w1, p["table_offsets"], p["table_dim_offsets"], p["dim_offsets"],
                          p["indices"], p["offsets"], 0.1)
    oracle.backward("sgd", p["grad_output"].reshape(9, 3, 16), w2, p["table_dim_offsets"][:-1], p["indices"],
                    p["offsets"], 0.1)
    assert w1.tobytes() == w2.tobytes()


# -------------------------------------------------------- stochastic rounding
def test_philox_known_answers(oracle):
    """Known-answer vectors of Philox4x32-10 from the Random123 distribution (kat_vectors)."""
    assert oracle.philox4x32_10([0, 0, 0, 0], [0, 0]) == [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]
    assert oracle.philox4x32_10([0xffffffff] * 4, [0xffffffff] * 2) == [0x408f276d, 0x41c83b0e, 0xa20bc7c6,
                                                                         0x6d5451fd]
    assert oracle.philox4x32_10([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0]) == \
        [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]


def test_stochastic_round_rule(oracle):
    """stochastic_rounding_vector (tbe.cu:569-576): add the top 13 random bits to the fp32
    pattern, truncate toward zero.  Values representable in fp16 never move; others land on one
    of their two fp16 neighbours with probability proportional to proximity (unbiased)."""
    half = lambda bits: float(np.array([bits], np.uint16).view(np.float16)[0])
    for x in (0.0, 1.0, -2.5, 0.000123, 65504.0, 6.1035e-05):
        exact = float(np.float16(x))
        for r in (0, 1 << 19, 0xffffffff, 0x80000000):
            assert half(oracle.stochastic_round(exact, r)) == exact
    x = 1.0 + 0.3 * 2.0 ** -10                                    # 30 % of the way from 1.0 to its successor
    lo, hi = 1.0, 1.0 + 2.0 ** -10
    rs = np.random.RandomState(0)
    draws = np.array([half(oracle.stochastic_round(x, int(r))) for r in rs.randint(0, 2 ** 32, size=20000,
                                                                                      dtype=np.uint64)])
    assert set(np.unique(draws)) == {lo, hi}
    assert abs(draws.mean() - np.float32(x)) < 3e-6             # unbiased: 0.3 +- 0.01 of the draws go up
    assert abs((draws == hi).mean() - 0.3) < 0.01
    assert half(oracle.stochastic_round(x, 0)) == lo and half(oracle.stochastic_round(x, 0xffffffff)) == hi
    # negative values move away from zero with the same rule
    assert half(oracle.stochastic_round(-x, 0)) == -lo and half(oracle.stochastic_round(-x, 0xffffffff)) == -hi


def test_conversion_toward_zero_against_numpy(oracle):
    """With a zero random word the rule is the plain fp32 -> fp16 conversion toward zero.  numpy
    converts to nearest; where that landed beyond the value, the neighbour toward zero is the
    answer.  Two million bit patterns over all exponents, plus the fp16 subnormal range, the
    largest finite values and the first values that overflow."""
    rs = np.random.RandomState(5)
    bits = np.concatenate([
        rs.randint(0, 2 ** 32, size=2_000_000, dtype=np.uint64).astype(np.uint32),
        np.arange(0x33000000, 0x38900000, 977, dtype=np.uint32),          # 2^-25 ... 2^-14 and a bit beyond
        np.arange(0x477fd000, 0x47801000, dtype=np.uint32),               # around 65504 ... 65536
        np.array([0, 0x80000000, 0x7f7fffff, 0xff7fffff, 0x7f800000, 0xff800000, 1, 0x80000001], np.uint32)])
    x = bits.view(np.float32)
    keep = ~np.isnan(x)
    x = x[keep]
    got = oracle.stochastic_round_many(x, np.zeros(x.size, np.uint32)).view(np.float16)
    with np.errstate(over="ignore"):
        near = x.astype(np.float16)
    beyond = np.abs(near.astype(np.float64)) > np.abs(x.astype(np.float64))
    want = np.where(beyond, np.nextafter(near, np.float16(0)), near)
    assert want.view(np.uint16).tobytes() == got.view(np.uint16).tobytes()


def test_stochastic_backward_is_within_one_ulp_and_reproducible(oracle):
    p = make_problem(31, T=2, E=40, D=16, B=30, L=6, dtype=np.float16, zipf=1.3)
    runs = []
    for stream in ((7, 0), (7, 0), (7, 4), None):
        w = p["weights"].copy()
        st = np.zeros(80, np.float32)
        oracle.backward("adagrad", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st,
                        stochastic_rounding=stream)
        runs.append(w)
    same_a, same_b, other, nearest = runs
    assert same_a.tobytes() == same_b.tobytes()                  # same (seed, offset) -> same bits
    assert same_a.tobytes() != other.tobytes()                   # another offset -> another draw
    ulp = np.abs(np.spacing(nearest.astype(np.float16))).astype(np.float32)
    assert (np.abs(same_a.astype(np.float32) - nearest.astype(np.float32)) <= ulp).all()
    untouched = np.setdiff1d(np.arange(80), oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])[0])
    assert same_a[untouched].tobytes() == p["weights"][untouched].tobytes()


# ------------------------------------------------------ interleaved [E][T][D] tables
def test_interleaved_layout_matches_embeddingbag(oracle):
    """The check of test_sparse_embedding_cuda.py:12-135: per table torch.nn.EmbeddingBag on
    weights[:, t, :], forward and w - lr * grad (with repeated rows, exact)."""
    torch = pytest.importorskip("torch")
    rs = np.random.RandomState(33)
    E, T, D, B, L = 50, 3, 8, 9, 5
    weights = rs.randn(E, T, D).astype(np.float32)
    lengths = rs.randint(0, L + 1, size=B * T)
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    indices = (rs.zipf(1.3, size=int(offsets[-1])) % E).astype(np.int32)
    go = rs.randn(B, T, D).astype(np.float32)
    out = oracle.forward_etd(weights, indices, offsets)
    w = weights.copy()
    oracle.backward_etd(go, w, indices, offsets, 0.05)
    for t in range(T):
        bag = torch.nn.EmbeddingBag(E, D, mode="sum", sparse=True)
        bag.weight.data.copy_(torch.from_numpy(weights[:, t, :].copy()))
        sel = [np.arange(offsets[b * T + t], offsets[b * T + t + 1]) for b in range(B)]
        idx_t = torch.from_numpy(indices[np.concatenate(sel)].astype(np.int64))
        off_t = torch.from_numpy(np.concatenate([[0], np.cumsum([len(s) for s in sel])[:-1]]).astype(np.int64))
        y = bag(idx_t, off_t)
        np.testing.assert_allclose(out[:, t, :], y.detach().numpy(), rtol=1e-5, atol=1e-6)
        y.backward(torch.from_numpy(go[:, t, :].copy()))
        want = bag.weight.detach() - bag.weight.grad.to_dense() * 0.05
        np.testing.assert_allclose(w[:, t, :], want.numpy(), rtol=1e-5, atol=1e-6)


# ------------------------------------------------- approximate row-wise Adagrad
# oracle_backward_approx restates batched_embedding_backward_adagrad_approx_kernel_1
# (tbe.cu:648-704) one lookup at a time.  Pinned by: hand-computed cases that tell the state used
# by the multiplier (after the lookup's own addition), the per-lookup weighting and the row a
# weighted lookup sees (already moved by earlier lookups) apart from their plausible mistakes; the
# reference test-suite's own oracle (torch.nn.EmbeddingBag + Python Adagrad,
# test_table_batched_embeddings.py:296-318) on indices drawn without replacement, the only case
# that test covers; a closed form for k identical hits; equality with the exact update when no
# row repeats; the mixed-D addressing against the uniform one.
def _one_row_problem(grads, lengths, D=4):
    """One table with one row; bag b has lengths[b] lookups of it and output gradient grads[b]."""
    B = len(grads)
    offsets = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    indices = np.zeros(int(offsets[-1]), np.int32)
    go = np.asarray(grads, np.float32).reshape(B, 1, D)
    return indices, offsets, go


def test_approx_adagrad_two_bags_by_hand(oracle):
    indices, offsets, go = _one_row_problem([[1, 2, 2, 0], [0, 3, 4, 0]], [1, 1])
    w = np.ones((1, 4), np.float32)
    state = np.array([7.0], np.float32)
    oracle.backward_approx(go, w, np.zeros(1, np.int32), indices, offsets, 0.5, 0.0, state)
    # lookup 0: state 7 + 9 = 16, multiplier 0.5 / 4; lookup 1: state 16 + 25 = 41, multiplier 0.5 / sqrt(41)
    w1 = 1.0 - 0.125 * np.array([1, 2, 2, 0])
    w2 = w1 - 0.5 / np.sqrt(41.0) * np.array([0, 3, 4, 0])
    assert state[0] == 41.0
    np.testing.assert_allclose(w[0], w2, rtol=1e-6)
    # the exact update would have summed the gradients first: G = [1, 5, 6, 0], state 7 + 62
    assert abs(state[0] - 69.0) > 1


def test_approx_adagrad_weighted_by_hand(oracle):
    indices, offsets, go = _one_row_problem([[1, 2, 2, 0], [0, 3, 4, 0]], [1, 1])
    w = np.ones((1, 4), np.float32)
    state = np.array([7.0], np.float32)
    psw = np.array([2.0, 0.5], np.float32)
    gpsw = oracle.backward_approx(go, w, np.zeros(1, np.int32), indices, offsets, 0.5, 0.0, state, psw)
    s1 = 7.0 + 9.0 * 4.0
    m1 = 2.0 * 0.5 / np.sqrt(s1)
    w1 = 1.0 - m1 * np.array([1, 2, 2, 0])
    s2 = s1 + 25.0 * 0.25
    m2 = 0.5 * 0.5 / np.sqrt(s2)
    w2 = w1 - m2 * np.array([0, 3, 4, 0])
    np.testing.assert_allclose(state[0], s2, rtol=1e-6)
    np.testing.assert_allclose(w[0], w2, rtol=1e-6)
    # the first lookup sees the untouched row, the second the row the first one left behind
    np.testing.assert_allclose(gpsw, [5.0, 3 * w1[1] + 4 * w1[2]], rtol=1e-6)
    assert abs(gpsw[1] - 7.0) > 0.1  # ... not the row as it was before the call


def test_approx_adagrad_repeat_inside_a_bag_and_k_identical_hits(oracle):
    # one bag, the same row twice: state 7 -> 16 -> 25, multipliers lr/4 and lr/5
    indices, offsets, go = _one_row_problem([[1, 2, 2, 0]], [2])
    w = np.ones((1, 4), np.float32)
    state = np.array([7.0], np.float32)
    oracle.backward_approx(go, w, np.zeros(1, np.int32), indices, offsets, 0.5, 0.0, state)
    assert state[0] == 25.0
    np.testing.assert_allclose(w[0], 1.0 - 0.5 * (1 / 4 + 1 / 5) * np.array([1, 2, 2, 0]), rtol=1e-6)
    # k bags with the same gradient g, state from 0, eps 0: state = k |g|^2 and
    # w = w0 - lr * g / |g| * sum_{j=1..k} 1 / sqrt(j)
    k, g = 37, np.array([0.5, -1.0, 2.0, 0.25])
    indices, offsets, go = _one_row_problem([g] * k, [1] * k)
    w = np.full((1, 4), 0.3, np.float64)
    state = np.zeros(1, np.float64)
    oracle.backward_approx(go.astype(np.float64), w, np.zeros(1, np.int32), indices, offsets, 0.1, 0.0, state)
    norm = np.sqrt((g * g).sum())
    np.testing.assert_allclose(state[0], k * norm ** 2, rtol=1e-12)
    lr = float(np.float32(0.1))  # the learning rate is a float on the interface
    np.testing.assert_allclose(w[0], 0.3 - lr * g / norm * (1.0 / np.sqrt(np.arange(1, k + 1))).sum(), rtol=1e-12)


@pytest.mark.parametrize("weighted", [False, True])
def test_approx_adagrad_matches_embedding_bag_without_replacement(oracle, weighted):
    """The reference's own check of its approximate kernel (test_table_batched_embeddings.py:
    244-318): indices drawn without replacement, per-table torch.nn.EmbeddingBag gradient,
    state = grad^2 summed per row, weights = addcdiv(w, -lr, grad, sqrt(state) + eps)."""
    import torch
    rs = np.random.RandomState(21)
    T, E, D, B, L, lr, eps = 3, 400, 16, 12, 5, 0.5, 0.2
    weights = rs.uniform(-1, 1, size=(T * E, D)).astype(np.float32)
    indices = np.concatenate([rs.choice(E, size=B * L, replace=False) for _ in range(T)]).astype(np.int32)
    offsets = np.arange(0, T * B * L + 1, L, dtype=np.int32)
    go = rs.randn(B, T, D).astype(np.float32)
    psw = rs.uniform(0.2, 1.5, size=T * B * L).astype(np.float32) if weighted else None
    table_offsets = (np.arange(T) * E).astype(np.int32)
    want_w, want_s = weights.copy(), np.zeros(T * E, np.float32)
    for t in range(T):
        bag = torch.nn.EmbeddingBag(E, D, mode="sum", sparse=True)
        bag.weight.data.copy_(torch.from_numpy(weights[t * E:(t + 1) * E]))
        idx = torch.from_numpy(indices[t * B * L:(t + 1) * B * L].astype(np.int64))
        off = torch.arange(0, B * L, L)
        kw = {"per_sample_weights": torch.from_numpy(psw[t * B * L:(t + 1) * B * L])} if weighted else {}
        bag(idx, off, **kw).backward(torch.from_numpy(go[:, t, :].copy()))
        dense = bag.weight.grad.to_dense()
        st = dense.pow(2).sum(1)
        want_s[t * E:(t + 1) * E] = st.numpy()
        want_w[t * E:(t + 1) * E] = torch.addcdiv(bag.weight.data, dense, (st.sqrt() + eps).view(-1, 1),
                                                  value=-lr).numpy()
    w, s = weights.copy(), np.zeros(T * E, np.float32)
    oracle.backward_approx(go, w, table_offsets, indices, offsets, lr, eps, s, psw)
    np.testing.assert_allclose(s, want_s, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(w, want_w, rtol=1e-5, atol=1e-6)
    # and the exact update agrees when no row repeats (bit for bit when unweighted)
    w2, s2 = weights.copy(), np.zeros(T * E, np.float32)
    oracle.backward("adagrad", go, w2, table_offsets, indices, offsets, lr, eps, s2, psw)
    if weighted:
        np.testing.assert_allclose(w, w2, rtol=1e-5, atol=1e-6)
    else:
        assert w.tobytes() == w2.tobytes() and s.tobytes() == s2.tobytes()


def test_approx_adagrad_mixed_addressing_equals_uniform(oracle):
    rs = np.random.RandomState(22)
    T, E, D, B, L = 3, 50, 8, 20, 4
    p = make_problem(23, T, E, D, B, L, np.float32, weighted=True, zipf=1.2)
    w, s = p["weights"].copy(), np.zeros(T * E, np.float32)
    g1 = oracle.backward_approx(p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.1, 0.01, s,
                                p["per_sample_weights"])
    wm, sm = p["weights"].reshape(-1).copy(), np.zeros(T * E, np.float32)
    g2 = oracle.backward_approx_mixed(
        p["grad_output"].reshape(B, T * D), wm, np.arange(T + 1) * E * D, np.arange(T + 1) * E, np.arange(T + 1) * D,
        p["indices"], p["offsets"], 0.1, 0.01, sm, p["per_sample_weights"])
    assert wm.tobytes() == w.tobytes() and sm.tobytes() == s.tobytes() and g1.tobytes() == g2.tobytes()
    assert (np.diff(p["offsets"]) > 1).any() and np.unique(p["indices"]).size < p["n"]  # rows do repeat here
