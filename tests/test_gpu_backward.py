"""GPU parity of the backward pipeline (linearize -> radix sort -> segments -> fused
update) through the C ABI.  Integer stages are compared bit for bit with the oracle
(sorted keys, stable positions, segment boundaries, U); updated weights / optimizer state /
per-sample-weight gradients within the north star's tolerances: fp32 1e-5 relative,
fp16 1e-2, fp64 1e-7 (the learning rate is a float on both sides, the sums differ in order)."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import GOLDEN_CASES, load_golden, make_problem
from gpu_util import DEV, assert_close, dev, gpu_backward, gpu_forward

import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops
import tbe_native

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float16): 1e-2, np.dtype(np.float64): 1e-7}


def _sync():
    torch.cuda.synchronize()


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _vp(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None and t.numel() else 0)


# ------------------------------------------------------- stages, bit-exact
@pytest.mark.parametrize("n,hi,end_bit", [(0, 10, 4), (1, 10, 4), (63, 2, 1), (64, 300, 9), (4095, 1 << 8, 8),
                                          (4096, 1 << 16, 16), (4097, 1 << 23, 23), (100000, 7, 3),
                                          (250001, 1 << 25, 25), (70000, 1 << 30, 31), (5000, 1000, 0),
                                          (33333, 1 << 17, 17), (50001, 1 << 19, 19), (81920, 1 << 20, 20),
                                          (120000, 1 << 27, 27), (60000, 1 << 29, 29), (9000, 1 << 10, 10),
                                          # either side of the switch from quarter-size to full-size tiles
                                          (524288, 1 << 18, 18), (524289, 1 << 18, 18), (1200000, 1 << 28, 28),
                                          (700000, 1 << 30, 31), (900000, 1 << 20, 20), (1023, 1 << 9, 9),
                                          (1025, 1 << 20, 20)])
def test_sort_pairs_is_stable_and_bit_exact(oracle, n, hi, end_bit):
    rs = np.random.RandomState(n % 97)
    keys = rs.randint(0, hi, size=n).astype(np.int32)
    if n > 100:
        keys[rs.randint(0, n, size=n // 3)] = keys[0]  # a hot key
    lib = tbe_native.load()
    k_in = dev(keys)
    k_out = torch.full((max(n, 1),), -1, dtype=torch.int32, device=DEV)
    v_out = torch.full((max(n, 1),), -1, dtype=torch.int32, device=DEV)
    ws = torch.empty(lib.tbe_sort_workspace_bytes(n), dtype=torch.uint8, device=DEV)
    tbe_native.check(lib.tbe_sort_pairs(_vp(k_in), _vp(None), _vp(k_out), _vp(v_out), n, end_bit, _vp(ws),
                                        ws.numel(), _stream()))
    _sync()
    want_k, want_v = oracle.sort_pairs(keys, None, end_bit)
    np.testing.assert_array_equal(k_out.cpu().numpy()[:n], want_k)
    np.testing.assert_array_equal(v_out.cpu().numpy()[:n], want_v)
    assert torch.equal(k_in.cpu(), torch.from_numpy(keys))  # input untouched
    if end_bit >= 31 or hi <= (1 << end_bit):
        np.testing.assert_array_equal(want_v, np.argsort(keys, kind="stable"))


def test_sort_pairs_carries_arbitrary_values(oracle):
    rs = np.random.RandomState(3)
    n = 30000
    keys = rs.randint(0, 1 << 12, size=n).astype(np.int32)
    vals = rs.randint(-2 ** 31, 2 ** 31 - 1, size=n).astype(np.int32)
    lib = tbe_native.load()
    k_in, v_in = dev(keys), dev(vals)
    k_out, v_out = (torch.empty(n, dtype=torch.int32, device=DEV) for _ in range(2))
    ws = torch.empty(lib.tbe_sort_workspace_bytes(n), dtype=torch.uint8, device=DEV)
    tbe_native.check(lib.tbe_sort_pairs(_vp(k_in), _vp(v_in), _vp(k_out), _vp(v_out), n, 12, _vp(ws),
                                        ws.numel(), _stream()))
    _sync()
    want_k, want_v = oracle.sort_pairs(keys, vals, 12)
    np.testing.assert_array_equal(k_out.cpu().numpy(), want_k)
    np.testing.assert_array_equal(v_out.cpu().numpy(), want_v)


def test_sort_pairs_in_a_workspace_sized_for_a_larger_batch(oracle):
    """One workspace, sized once for the largest batch, serves smaller ones on either tile size."""
    lib = tbe_native.load()
    largest = 600000
    ws = torch.empty(lib.tbe_sort_workspace_bytes(largest), dtype=torch.uint8, device=DEV)
    for n in (largest, 524288, 300000, 77):
        keys = np.random.RandomState(n % 101).randint(0, 1 << 21, size=n).astype(np.int32)
        k_in = dev(keys)
        k_out, v_out = (torch.full((n,), -1, dtype=torch.int32, device=DEV) for _ in range(2))
        tbe_native.check(lib.tbe_sort_pairs(_vp(k_in), _vp(None), _vp(k_out), _vp(v_out), n, 21, _vp(ws),
                                            ws.numel(), _stream()))
        _sync()
        want_k, want_v = oracle.sort_pairs(keys, None, 21)
        np.testing.assert_array_equal(k_out.cpu().numpy(), want_k)
        np.testing.assert_array_equal(v_out.cpu().numpy(), want_v)


@pytest.mark.parametrize("n,hi", [(0, 5), (1, 5), (2047, 3), (2048, 100000), (2049, 1), (300000, 120000),
                                  (8388608, 2000000), (8400000, 3000000)])  # 4096 tiles, and one tile count beyond
def test_find_segments_bit_exact(oracle, n, hi):
    keys = np.sort(np.random.RandomState(n % 89).randint(0, hi, size=n)).astype(np.int32)
    lib = tbe_native.load()
    starts = torch.full((n + 1,), -7, dtype=torch.int32, device=DEV)
    count = torch.full((4,), -7, dtype=torch.int32, device=DEV)
    ws = torch.empty(lib.tbe_segments_workspace_bytes(n), dtype=torch.uint8, device=DEV)
    k_in = dev(keys)
    tbe_native.check(lib.tbe_find_segments(_vp(k_in), n, _vp(starts), _vp(count), _vp(ws), ws.numel(),
                                           _stream()))
    _sync()
    want = oracle.segments(keys)
    U = int(count[0])
    assert U == want.size - 1
    np.testing.assert_array_equal(starts.cpu().numpy()[:U + 1], want)


def test_linearize_and_construct_offsets_bit_exact(oracle):
    p = make_problem(3, T=5, E=0, D=4, B=37, L=11, dtype=np.float32, rows=[5, 17, 3, 40, 1000])
    lib = tbe_native.load()
    keys, grows = (torch.empty(p["n"], dtype=torch.int32, device=DEV) for _ in range(2))
    d_to, d_idx, d_off = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    tbe_native.check(lib.tbe_linearize(_vp(d_to), 5, _vp(d_idx), p["n"], _vp(d_off), 37, _vp(keys), _vp(grows),
                                       _stream()))
    _sync()
    want_keys, b_t, _ = oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])
    np.testing.assert_array_equal(keys.cpu().numpy(), want_keys)
    np.testing.assert_array_equal(grows.cpu().numpy(), (b_t % 37) * 5 + b_t // 37)
    # construct_offsets, the check of test_table_batched_embeddings.py:97-105
    lengths = np.diff(p["offsets"]).reshape(5, 37)
    starts = np.concatenate([np.zeros((5, 1), int), np.cumsum(lengths, axis=1)[:, :-1]], axis=1).astype(np.int32)
    totals = lengths.sum(axis=1).astype(np.int32)
    got = ext.construct_offsets(dev(starts), dev(totals))
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.construct_offsets(starts, totals))
    np.testing.assert_array_equal(torch.cumsum(got, 0).cpu().numpy(), p["offsets"])


def _plan_views(p, max_table_rows):
    """tbe_plan_batch through the C ABI; returns (keys_sorted, positions_sorted, segment_starts)."""
    n, T = p["n"], p["T"]
    total_rows = int(sum(p["rows"]))
    lay = tbe_native.backward_workspace_layout(n, 4, tbe_native.DTYPE_F32, T)
    ws = torch.zeros(lay.total_bytes, dtype=torch.uint8, device=DEV)
    to, idx, off = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    tbe_native.check(tbe_native.load().tbe_plan_batch(_vp(to), T, _vp(idx), n, _vp(off), p["B"], total_rows,
                                                      max_table_rows, 4, tbe_native.DTYPE_F32, _vp(ws), ws.numel(),
                                                      _stream()))
    _sync()
    view = lambda o, c: ws[o:o + 4 * c].view(torch.int32).cpu().numpy()
    U = int(view(lay.num_unique, 1)[0])
    return view(lay.keys_sorted, n), view(lay.positions_sorted, n), view(lay.segment_starts, U + 1)


@pytest.mark.parametrize("case", ["ragged_rows", "empty_tables", "many_small_tables", "multi_tile_tables", "one_table",
                                  "eight_tables_of_thirty_tiles", "one_large_table_among_nine",
                                  "ten_bit_digits", "eight_tables_of_forty_small_tiles",
                                  "one_larger_table_among_nine", "ten_bit_digits_full_tiles",
                                  "two_tables_of_hundreds_of_tiles", "more_tables_than_are_sorted_apart"])
def test_per_table_sort_equals_sort_of_linearized_keys(oracle, case):
    """The plan sorts every table's indices on their own (fewer key bits); keys_sorted,
    positions_sorted and segment_starts must equal the stable sort of table_offsets[t] + index
    (table_batched_embeddings_cuda.cu:1495, 1639-1655) bit for bit, whatever bound of the
    largest table the caller gives."""
    if case == "ragged_rows":
        p = make_problem(11, T=5, E=0, D=4, B=300, L=9, dtype=np.float32, rows=[3, 70000, 1, 513, 1024])
    elif case == "empty_tables":
        p = make_problem(12, T=6, E=0, D=4, B=64, L=30, dtype=np.float32, rows=[100, 5, 3000, 7, 9, 200])
        lengths = np.diff(p["offsets"]).reshape(6, 64)
        lengths[[0, 2, 5]] = 0  # tables 0, 2 and 5 get no lookup at all
        keep = np.repeat(lengths.reshape(-1) > 0, np.diff(p["offsets"]))
        p["indices"] = p["indices"][keep]
        p["offsets"] = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
        p["n"] = int(p["offsets"][-1])
    elif case == "many_small_tables":
        p = make_problem(13, T=700, E=37, D=4, B=3, L=4, dtype=np.float32)
    elif case == "eight_tables_of_thirty_tiles":
        # many tables, every one of at most 48 sort tiles: the per-table count scan runs inside the
        # scatter kernel
        p = make_problem(16, T=8, E=0, D=4, B=3000, L=40, dtype=np.float32, ragged=False, zipf=1.1,
                         rows=[70000, 300, 1 << 17, 5, 90000, 1000, 131071, 2])
    elif case == "eight_tables_of_forty_small_tiles":
        # the same through the quarter-size tiles of a batch of at most 2^19 lookups
        p = make_problem(19, T=8, E=0, D=4, B=1000, L=40, dtype=np.float32, ragged=False, zipf=1.1,
                         rows=[70000, 300, 1 << 17, 5, 90000, 1000, 131071, 2])
    elif case in ("one_large_table_among_nine", "one_larger_table_among_nine"):
        # one table of more tiles than the scatter kernel scans itself, among small ones: the scan
        # kernel with a workgroup per table runs (quarter-size tiles; full-size tiles for the larger)
        rs = np.random.RandomState(17)
        T, B = 9, 3200
        rows = [4000, 100, 50000, 1 << 17, 7, 900, 30000, 12, 65536]
        lengths = np.full((T, B), 2)
        lengths[3] = 80 if case == "one_large_table_among_nine" else 200
        offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
        indices = np.concatenate([rs.zipf(1.2, size=int(lengths[t].sum())) % rows[t] for t in range(T)])
        p = dict(T=T, B=B, rows=rows, n=int(offsets[-1]), offsets=offsets, indices=indices.astype(np.int32),
                 table_offsets=np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    elif case == "more_tables_than_are_sorted_apart":
        # beyond 2048 tables the linearized keys are sorted in one piece
        p = make_problem(24, T=2500, E=41, D=4, B=5, L=6, dtype=np.float32)
    elif case == "two_tables_of_hundreds_of_tiles":
        # 300 and 200 tiles in two of ten tables: their later tiles add up whole groups of 64 tiles
        # from the group totals, and the groups do not start where the tables do
        rs = np.random.RandomState(23)
        T, B = 10, 4100
        rows = [4000, 100, 1 << 19, 50000, 7, 900, 30000, 700001, 12, 65536]
        lengths = np.full((T, B), 3)
        lengths[2] = 300
        lengths[7] = 200
        offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
        indices = np.concatenate([rs.zipf(1.15, size=int(lengths[t].sum())) % rows[t] for t in range(T)])
        p = dict(T=T, B=B, rows=rows, n=int(offsets[-1]), offsets=offsets, indices=indices.astype(np.int32),
                 table_offsets=np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32))
    elif case in ("ten_bit_digits", "ten_bit_digits_full_tiles"):
        p = make_problem(18, T=8, E=0, D=4, B=2000 if case == "ten_bit_digits" else 4000, L=30, dtype=np.float32,
                         zipf=1.05,
                         rows=[1 << 20, 1000000, 999999, 1 << 19, 3, 1 << 20, 70, 524289])
    elif case == "multi_tile_tables":
        p = make_problem(14, T=3, E=0, D=4, B=1500, L=12, dtype=np.float32, zipf=1.1, rows=[1 << 17, 100, 300000])
    else:
        p = make_problem(15, T=1, E=5000, D=4, B=4000, L=5, dtype=np.float32, zipf=1.3)
    keys, _, _ = oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])
    want_k, want_v = oracle.sort_pairs(keys, None, 32)
    want_starts = oracle.segments(want_k)
    for bound in (0, max(p["rows"]), int(sum(p["rows"]))):
        ks, ps, ss = _plan_views(p, bound)
        np.testing.assert_array_equal(ks, want_k)
        np.testing.assert_array_equal(ps, want_v)
        np.testing.assert_array_equal(ss, want_starts)


# --------------------------------------------------- fused backward vs oracle
SHAPES = [(2, 1000, 32, 64, 4), (3, 50, 128, 33, 20), (1, 7, 4, 5, 3), (2, 100, 12, 17, 9), (2, 30, 520, 9, 5),
          (4, 20, 64, 700, 40), (2, 100, 256, 50, 70), (1, 3, 8, 400, 9), (2, 64, 16, 31, 6),
          (2100, 20, 8, 3, 4)]  # (the last: more tables than are sorted apart)


def _run_both(oracle, p, optimizer, lr, eps):
    w = p["weights"].copy()
    st = np.zeros(w.shape[0], np.float64 if w.dtype == np.float64 else np.float32)
    ref = oracle.backward(optimizer, p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], lr, eps,
                          st, p.get("per_sample_weights"))
    got = gpu_backward(p, optimizer, lr, eps)
    return w, st, ref, got


def _check(p, w, st, ref, got, optimizer):
    tol = TOL[p["weights"].dtype]
    v = got["views"]
    if p["n"]:
        np.testing.assert_array_equal(v["keys_sorted"], ref["keys_sorted"])
        np.testing.assert_array_equal(v["positions_sorted"], ref["positions_sorted"])
        np.testing.assert_array_equal(v["segment_starts"], ref["segment_starts"])
        assert v["num_unique"] == ref["segment_starts"].size - 1
    assert_close(got["weights"], w, tol, "weights")
    # rows no lookup touches must keep their bits
    touched = np.zeros(w.shape[0], bool)
    touched[ref["keys_sorted"]] = True
    assert got["weights"][~touched].tobytes() == p["weights"][~touched].tobytes()
    if optimizer == "adagrad":
        assert_close(got["state"], st, 1e-3 if p["weights"].dtype == np.float16 else max(tol, 1e-6), "state")
        assert not got["state"][~touched].any()
    if ref["grad_psw"] is not None:
        assert_close(got["grad_psw"], ref["grad_psw"], tol, "grad_psw")


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
@pytest.mark.parametrize("mode", ["sgd", "adagrad", "adagrad_weighted"])
@pytest.mark.parametrize("shape", SHAPES)
def test_backward_matches_oracle(oracle, shape, mode, dtype):
    T, E, D, B, L = shape
    p = make_problem(hash(shape) % 1000 + 1, T, E, D, B, L, dtype, ragged=True, weighted=mode.endswith("weighted"),
                     zipf=1.2)
    optimizer = "sgd" if mode == "sgd" else "adagrad"
    w, st, ref, got = _run_both(oracle, p, optimizer, 0.05, 0.1)
    _check(p, w, st, ref, got, optimizer)


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_backward_matches_embeddingbag_fixture(name):
    g = load_golden(name)
    g["table_offsets"] = (np.arange(g["T"]) * g["E"]).astype(np.int32)
    g["n"] = g["indices"].size
    got = gpu_backward(g, g["optimizer"], g["lr"], g["eps"])
    tol = TOL[g["weights"].dtype]
    assert_close(got["weights"], g["expected_weights"], tol)
    if g["optimizer"] == "adagrad":
        assert_close(got["state"], g["expected_state"], 1e-3 if g["weights"].dtype == np.float16 else 1e-5)
    if "expected_grad_psw" in g:
        assert_close(got["grad_psw"], g["expected_grad_psw"], tol)


SHORT_SEGMENT = 128  # kShortSegment of csrc/tbe_stages.h: longer segments leave the short-row kernel


@pytest.mark.parametrize("dtype,D,occurrences", [(np.float32, 128, SHORT_SEGMENT + 1), (np.float16, 64, SHORT_SEGMENT + 1),
                                                 (np.float32, 16, 257)])
def test_queues_hold_the_most_chunk_records_a_batch_can_produce(oracle, dtype, D, occurrences):
    """Every row occurs 129 times (the most segments that leave the short-row kernel: one chunk
    record per 129 lookups) or 257 times (two chunks and a partial-row record each): the eight
    queues together receive exactly the number of records the arithmetic predicts, and nothing
    around them is overwritten (the update still matches the oracle)."""
    rs = np.random.RandomState(11)
    T, B, L = 3, 1700, 12
    n = T * B * L
    per_table = B * L
    rows = per_table // occurrences + 1
    p = make_problem(12, T, rows, D, B, L, dtype, ragged=False, weighted=False)
    for t in range(T):
        ids = np.repeat(np.arange(rows, dtype=np.int32), occurrences)[:per_table]
        p["indices"][t * per_table:(t + 1) * per_table] = rs.permutation(ids)
    w, st, ref, got = _run_both(oracle, p, "sgd", 0.01, 0.1)
    lengths = np.diff(ref["segment_starts"])
    assert (lengths == occurrences).sum() >= T * (rows - 1)
    # (one 128-byte line of counters per XCD from word 64 on: [0] chunk records queued, [1] segments of several chunks)
    counters = got["views"]["counters"]
    assert counters[64:320:32].sum() == np.ceil(lengths[lengths > SHORT_SEGMENT] / 256).sum()
    assert counters[65:320:32].sum() == (lengths > 256).sum()
    _check(p, w, st, ref, got, "sgd")


@pytest.mark.parametrize("dtype,D", [(np.float32, 128), (np.float16, 64), (np.float32, 12), (np.float64, 8)])
@pytest.mark.parametrize("mode", ["sgd", "adagrad_weighted"])
def test_hot_rows_take_the_chunked_path(oracle, dtype, D, mode):
    """Segments far longer than one lane group handles: one row receives ~70 % of 60 k lookups,
    others land on both sides of the 128- and 256-occurrence thresholds."""
    rs = np.random.RandomState(5)
    T, E, B, L = 2, 50, 3000, 10
    p = make_problem(9, T, E, D, B, L, dtype, ragged=False, weighted=mode.endswith("weighted"))
    n = p["n"]
    hot = rs.rand(n) < 0.7
    p["indices"][hot] = 7
    p["indices"][~hot] = rs.choice([1, 2, 3, 40, 41], size=(~hot).sum(), p=[0.5, 0.3, 0.19, 0.006, 0.004])
    optimizer = "sgd" if mode == "sgd" else "adagrad"
    w, st, ref, got = _run_both(oracle, p, optimizer, 0.001, 0.1)
    lengths = np.diff(ref["segment_starts"])
    assert lengths.max() > 15000 and (lengths <= 256).any() and ((lengths > 256) & (lengths < 2000)).any()
    # rows with more than 256 occurrences are reduced in several chunks, rows with more than 128 by
    # whole wavefronts: from word 64 on, every XCD has a 128-byte line of counters, [0] the chunk records
    # its workgroups queued, [1] their rows of several chunks
    assert got["views"]["counters"][65:320:32].sum() == (lengths > 256).sum()
    assert got["views"]["counters"][64:320:32].sum() == np.ceil(lengths[lengths > SHORT_SEGMENT] / 256).sum()
    np.testing.assert_array_equal(got["views"]["positions_sorted"], ref["positions_sorted"])
    np.testing.assert_array_equal(got["views"]["segment_starts"], ref["segment_starts"])
    # The truth is the update computed in fp64 from the same inputs.  The HIP path has to be within
    # the stated tolerance of IT (fp32: 1e-5 relative), and no further from it than the oracle's
    # serial fp32 sum is (the oracle adds ~42 k terms one by one, the kernels in trees of chunks).
    tol = TOL[np.dtype(dtype)]
    w64, st64 = _fp64_update(p, optimizer, 0.001, 0.1)
    assert_close(got["weights"], w64, tol, "HIP weights vs fp64")
    err_gpu = np.abs(got["weights"].astype(np.float64) - w64).max()
    err_oracle = np.abs(w.astype(np.float64) - w64).max()
    floor = np.abs(w64).max() * np.finfo(np.dtype(dtype)).eps  # one rounding of the stored weight
    if dtype != np.float64:  # for fp64 inputs the fp64 sum is the oracle's own arithmetic, not the truth
        assert err_gpu <= 2 * err_oracle + floor, (err_gpu, err_oracle)
    # oracle vs HIP: the looser secondary check (both carry their own fp32 rounding)
    loose = {np.dtype(np.float32): 2e-4, np.dtype(np.float16): 1e-2, np.dtype(np.float64): 1e-7}[np.dtype(dtype)]
    assert_close(got["weights"], w, loose)
    if optimizer == "adagrad":
        assert_close(got["state"], st64, 1e-5 if dtype != np.float64 else 1e-12, "HIP state vs fp64")
        assert_close(got["state"], st, 1e-3)
        assert_close(got["grad_psw"], ref["grad_psw"], TOL[np.dtype(dtype)])


def _fp64_update(p, optimizer, lr, eps):
    """The exact update in fp64 numpy (test_table_batched_embeddings.py:190-193, 296-318):
    G[r] = sum over the occurrences of row r of (psw *) grad_output[b, t]; SGD w -= lr * G;
    row-wise Adagrad state = sum_d G^2 (from zero), w -= lr / (sqrt(state) + eps) * G."""
    T, B = p["T"], p["B"]
    bag = np.repeat(np.arange(T * B), np.diff(p["offsets"]))
    t, b = bag // B, bag % B
    rows = p["table_offsets"][t].astype(np.int64) + p["indices"]
    g = p["grad_output"].astype(np.float64)[b, t, :]
    if p.get("per_sample_weights") is not None:
        g = g * p["per_sample_weights"].astype(np.float64)[:, None]
    G = np.zeros(p["weights"].shape, np.float64)
    np.add.at(G, rows, g)
    w = p["weights"].astype(np.float64)
    lr = float(np.float32(lr))
    if optimizer == "sgd":
        return w - lr * G, None
    state = (G * G).sum(axis=1)
    mult = np.where(state > 0, lr / (np.sqrt(state) + float(np.float32(eps))), 0.0)
    return w - mult[:, None] * G, state


def test_two_backward_runs_are_bit_identical():
    p = make_problem(12, T=3, E=40, D=128, B=2000, L=12, dtype=np.float32, weighted=True, zipf=1.1)
    a = gpu_backward(p, "adagrad", 0.05, 0.1)
    b = gpu_backward(p, "adagrad", 0.05, 0.1)
    for k in ("weights", "state", "grad_psw"):
        assert a[k].tobytes() == b[k].tobytes()


def test_zero_gradient_and_empty_input_leave_weights_untouched():
    p = make_problem(13, T=2, E=100, D=64, B=50, L=6, dtype=np.float32)
    p["grad_output"][:] = 0
    assert gpu_backward(p, "sgd", 0.5)["weights"].tobytes() == p["weights"].tobytes()
    p0 = make_problem(14, T=2, E=100, D=64, B=5, L=0, dtype=np.float32)
    assert gpu_backward(p0, "sgd", 0.5)["weights"].tobytes() == p0["weights"].tobytes()


def test_second_adagrad_step_accumulates_state(oracle):
    p = make_problem(15, T=2, E=30, D=32, B=40, L=5, dtype=np.float32, zipf=1.3)
    w = p["weights"].copy()
    st = np.zeros(60, np.float32)
    for _ in range(2):
        oracle.backward("adagrad", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st)
    first = gpu_backward(p, "adagrad", 0.05, 0.1)
    p2 = dict(p, weights=first["weights"])
    second = gpu_backward(p2, "adagrad", 0.05, 0.1, state=first["state"])
    assert_close(second["state"], st, 1e-5)
    assert_close(second["weights"], w, 1e-5)


# ------------------------------------------------------------- module API
def test_module_backward_sgd_like_the_reference_test(oracle):
    """test_table_batched_embeddings.py:163-216 through the drop-in module, but with repeated
    rows (the reference needs sampling without replacement)."""
    T, E, D, B, L = 3, 200, 64, 32, 8
    p = make_problem(16, T, E, D, B, L, np.float32, ragged=False, zipf=1.2)
    cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.SGD, learning_rate=0.05).cuda()
    cc.embedding_weights.data.copy_(dev(p["weights"]))
    out = cc(dev(p["indices"]), dev(p["offsets"]))
    out.backward(dev(p["grad_output"]))
    w = p["weights"].copy()
    oracle.backward("sgd", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.05)
    assert_close(cc.embedding_weights.detach().cpu().numpy(), w, 1e-5)
    g = cc.embedding_weights.grad
    assert g is None or (g.is_sparse and g._nnz() == 0 and g.dtype == torch.float32)


@pytest.mark.parametrize("fp16", [False, True])
@pytest.mark.parametrize("optimizer", [ops.Optimizer.EXACT_ROWWISE_ADAGRAD, ops.Optimizer.APPROX_ROWWISE_ADAGRAD])
def test_module_backward_adagrad_like_the_reference_test(oracle, optimizer, fp16):
    # test_table_batched_embeddings.py:219-318: lr=0.5, eps=0.2; exact => E=100 with replacement
    exact = optimizer == ops.Optimizer.EXACT_ROWWISE_ADAGRAD
    T, E, D, B, L = 4, (100 if exact else 10000), 32, 64, 6
    dtype = np.float16 if fp16 else np.float32
    rs = np.random.RandomState(17)
    p = make_problem(17, T, E, D, B, L, dtype, ragged=False)
    if not exact:  # the approximate optimizer is only specified when no row repeats (:244)
        p["indices"] = np.concatenate([rs.choice(E, size=B * L, replace=False) for _ in range(T)]).astype(np.int32)
    cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=optimizer, learning_rate=0.5, eps=0.2, fp16=fp16).cuda()
    cc.embedding_weights.data.copy_(dev(p["weights"]))
    cc(dev(p["indices"]), dev(p["offsets"])).backward(dev(p["grad_output"]))
    w = p["weights"].copy()
    st = np.zeros(T * E, np.float32)
    oracle.backward("adagrad", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.5, 0.2, st)
    assert_close(cc.optimizer_state.cpu().numpy(), st, 1e-3 if fp16 else 1e-5)
    assert_close(cc.embedding_weights.detach().cpu().numpy(), w, 1e-2 if fp16 else 1e-5)


def test_gradcheck_on_per_sample_weights_in_double():
    # test_table_batched_embeddings.py:320-340: lr = 0, module in double, gradcheck on per_sample_weights
    T, E, D, B, L = 2, 50, 8, 5, 3
    p = make_problem(18, T, E, D, B, L, np.float64, ragged=False, weighted=True)
    cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.0,
                                       eps=0.2).cuda().double()
    cc.embedding_weights.requires_grad = False
    psw = dev(p["per_sample_weights"]).requires_grad_(True)
    assert torch.autograd.gradcheck(cc, (dev(p["indices"]), dev(p["offsets"]), psw))


def test_full_size_backward_properties():
    """The shape of bench.py --config 3 (T=64, E=1e5, D=128 fp32, B=4096, L=20, Zipf(1.05) indices,
    exact SGD lr=0.01).  Size-independent properties instead of the oracle:
    sortedness + permutation + stability of the sort, key/position consistency, strict
    segment boundaries, the column checksum of the update (linearity), untouched rows
    bit-identical, and the first table against the oracle."""
    from oracle import tbe_oracle
    T, E, D, B, L = 64, 100000, 128, 4096, 20
    rs = np.random.RandomState(0)
    idx_np = (rs.zipf(1.05, size=T * B * L) % E).astype(np.int32)
    gen = torch.Generator(device=DEV).manual_seed(0)
    W = torch.empty(T * E, D, device=DEV).uniform_(-0.01, 0.01, generator=gen)
    W0 = W.clone()
    go = torch.randn(B, T, D, device=DEV, generator=gen)
    idx = torch.from_numpy(idx_np).to(DEV)
    offsets = torch.arange(0, T * B * L + 1, L, dtype=torch.int32, device=DEV)
    table_offsets = torch.arange(T, dtype=torch.int32, device=DEV) * E
    ext.backward_sgd(go, W, table_offsets, idx, offsets, 0.01, 200, 1, False)
    _sync()
    n = T * B * L
    lay = tbe_native.backward_workspace_layout(n, D, tbe_native.DTYPE_F32, T)
    ws = ext.backward_workspace(torch.device(DEV))
    view = lambda off, cnt: ws[off:off + 4 * cnt].view(torch.int32)
    ks, ps = view(lay.keys_sorted, n), view(lay.positions_sorted, n)
    U = int(view(lay.num_unique, 1)[0])
    ss = view(lay.segment_starts, U + 1).long()
    want_keys = idx.long() + torch.arange(T, device=DEV).repeat_interleave(B * L) * E
    assert bool((ks[1:] >= ks[:-1]).all())                                   # sorted
    assert torch.equal(torch.sort(ps.long())[0], torch.arange(n, device=DEV))  # permutation
    assert torch.equal(want_keys[ps.long()], ks.long())                                   # pairs stayed together
    same = ks[1:] == ks[:-1]
    assert bool((ps[1:][same] > ps[:-1][same]).all())                         # stable
    assert U == int(torch.unique(want_keys).numel())
    assert int(ss[0]) == 0 and int(ss[-1]) == n and bool((ss[1:] > ss[:-1]).all())
    assert bool((ks[ss[1:-1]] != ks[ss[1:-1] - 1]).all())                     # every start is a head
    heads = torch.ones(n, dtype=torch.bool, device=DEV)
    heads[1:] = ks[1:] != ks[:-1]
    assert int(heads.sum()) == U
    # linearity checksum: sum over rows of (W0 - W) == lr * sum_p go[grad_row(p)]
    counts = torch.bincount(torch.arange(T * B, device=DEV).repeat_interleave(L), minlength=T * B)
    bag_weight = counts.view(T, B).t().contiguous().double()                  # [B][T] lookups per bag
    want_col = 0.01 * (go.double() * bag_weight.unsqueeze(-1)).sum((0, 1))
    got_col = (W0.double() - W.double()).sum(0)
    assert_close(got_col.cpu().numpy(), want_col.cpu().numpy(), 1e-5)
    touched = torch.zeros(T * E, dtype=torch.bool, device=DEV)
    touched[want_keys] = True
    assert torch.equal(W[~touched], W0[~touched])
    # first table against the oracle (81 920 lookups)
    w_ref = W0[:E].cpu().numpy().copy()
    tbe_oracle.backward("sgd", go[:, :1, :].contiguous().cpu().numpy(), w_ref, np.zeros(1, np.int32), idx_np[:B * L],
                        offsets[:B + 1].cpu().numpy(), 0.01)
    assert_close(W[:E].cpu().numpy(), w_ref, 1e-5)


def test_full_size_weighted_adagrad_fp16_properties():
    """The shape of bench.py --config 4 (T=32, E=1e6, D=64 fp16 weights, fp32 state from 0, B=8192, bag
    lengths uniform in [0, 40] with empty bags, per-sample weights ~U(0,1), Zipf(1.2) indices,
    exact row-wise Adagrad lr=0.01 eps=1e-8): sort / segment properties, untouched rows and state
    bit-identical, and the first table (weights, state, per-sample-weight gradients) against the
    oracle."""
    from oracle import tbe_oracle
    T, E, D, B = 32, 1000000, 64, 8192
    rs = np.random.RandomState(4)
    lengths = rs.randint(0, 41, size=T * B)
    off_np = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    n = int(off_np[-1])
    idx_np = (rs.zipf(1.2, size=n) % E).astype(np.int32)
    gen = torch.Generator(device=DEV).manual_seed(4)
    W = torch.empty(T * E, D, device=DEV).uniform_(-0.01, 0.01, generator=gen).half()
    W0 = W.clone()
    state = torch.zeros(T * E, device=DEV)
    go = torch.randn(B, T, D, device=DEV, generator=gen).half()
    psw = torch.rand(n, device=DEV, generator=gen).half()
    idx, offsets = torch.from_numpy(idx_np).to(DEV), torch.from_numpy(off_np).to(DEV)
    table_offsets = torch.arange(T, dtype=torch.int32, device=DEV) * E
    grad_psw = ext.backward_exact_adagrad(go, W, table_offsets, idx, offsets, psw, state, 0.01, 1e-8, False, 1)
    _sync()
    lay = tbe_native.backward_workspace_layout(n, D, tbe_native.DTYPE_F16, T)
    ws = ext.backward_workspace(torch.device(DEV))
    view = lambda off, cnt: ws[off:off + 4 * cnt].view(torch.int32)
    ks, ps = view(lay.keys_sorted, n), view(lay.positions_sorted, n)
    U = int(view(lay.num_unique, 1)[0])
    ss = view(lay.segment_starts, U + 1).long()
    table_of_position = torch.repeat_interleave(torch.arange(T, device=DEV),
                                                torch.from_numpy(lengths.reshape(T, B).sum(1)).to(DEV))
    want_keys = idx.long() + table_of_position * E
    assert bool((ks[1:] >= ks[:-1]).all())
    assert torch.equal(torch.sort(ps.long())[0], torch.arange(n, device=DEV))
    assert torch.equal(want_keys[ps.long()], ks.long())
    same = ks[1:] == ks[:-1]
    assert bool((ps[1:][same] > ps[:-1][same]).all())
    assert U == int(torch.unique(want_keys).numel())
    assert int(ss[0]) == 0 and int(ss[-1]) == n and bool((ss[1:] > ss[:-1]).all())
    seg_len = ss[1:] - ss[:-1]
    assert int(seg_len.max()) > 20000            # the hot rows of Zipf(1.2): thousands of chunks
    touched = torch.zeros(T * E, dtype=torch.bool, device=DEV)
    touched[want_keys] = True
    assert torch.equal(W[~touched], W0[~touched]) and not bool(state[~touched].any())
    assert bool((state[touched] >= 0).all()) and bool(torch.isfinite(W.float()).all())
    # first table against the oracle
    n0 = int(off_np[B])
    w_ref = W0[:E].cpu().numpy().copy()
    st_ref = np.zeros(E, np.float32)
    ref = tbe_oracle.backward("adagrad", go[:, :1, :].contiguous().cpu().numpy(), w_ref, np.zeros(1, np.int32),
                              idx_np[:n0], off_np[:B + 1], 0.01, 1e-8, st_ref, psw[:n0].cpu().numpy())
    assert_close(W[:E].cpu().numpy(), w_ref, 1e-2)
    assert_close(state[:E].cpu().numpy(), st_ref, 1e-3)
    assert_close(grad_psw[:n0].cpu().numpy(), ref["grad_psw"], 1e-2)


@pytest.mark.parametrize("mode", ["sgd", "adagrad_weighted"])
def test_plan_ahead_equals_single_call_backward(mode):
    """tbe_plan_batch on a side stream + tbe_backward_planned give bit-identical results to the
    one-call backward, directly and through the module with LookupFunction.plan_ahead."""
    p = make_problem(60, T=3, E=500, D=64, B=200, L=12, dtype=np.float32, weighted=mode.endswith("weighted"),
                     zipf=1.15)
    optimizer = "sgd" if mode == "sgd" else "adagrad"
    want = gpu_backward(p, optimizer, 0.05, 0.1)
    w, go = dev(p["weights"]), dev(p["grad_output"])
    to, idx, off = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    psw = dev(p["per_sample_weights"])
    st = torch.zeros(w.shape[0], device=DEV)
    plan = ext.plan_backward(w, to, idx, off)
    out = ext.forward(w, to, idx, off, psw, 200, 1, False)  # the forward the plan is meant to overlap
    code = tbe_native.OPT_SGD if optimizer == "sgd" else tbe_native.OPT_ROWWISE_ADAGRAD
    gpsw = plan.apply(code, go, w, psw, st if optimizer != "sgd" else None, 0.05, 0.1, False)
    torch.cuda.synchronize()
    assert out.shape == (200, 3, 64)
    assert w.cpu().numpy().tobytes() == want["weights"].tobytes()
    if optimizer == "adagrad":
        assert st.cpu().numpy().tobytes() == want["state"].tobytes()
        assert gpsw.cpu().numpy().tobytes() == want["grad_psw"].tobytes()

    ops.LookupFunction.plan_ahead = True
    try:
        cc = ops.TableBatchedEmbeddingBags(3, 500, 64, optimizer=ops.Optimizer.SGD if optimizer == "sgd" else
                                           ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.05, eps=0.1).cuda()
        cc.embedding_weights.data.copy_(dev(p["weights"]))
        cc(idx, off, psw).backward(go)
        torch.cuda.synchronize()
        assert cc.embedding_weights.detach().cpu().numpy().tobytes() == want["weights"].tobytes()
    finally:
        ops.LookupFunction.plan_ahead = False
