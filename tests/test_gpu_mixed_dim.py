"""GPU parity of the per-table-dimension path (tbe_forward_mixed / tbe_backward_mixed through
the C ABI and the MixedDimTableBatchedEmbeddingBags mirror) against the CPU oracle.
Tolerances as for the uniform path: fp32 1e-5, fp16 1e-2, fp64 1e-7."""
import numpy as np
import pytest
import torch

from conftest import make_mixed_problem
from gpu_util import DEV, assert_close, dev

import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float16): 1e-2, np.dtype(np.float64): 1e-7}
TABLE_SETS = [
    [(30, 8), (7, 32), (100, 4), (16, 12)],
    [(50, 128), (1000, 64), (3, 520)],          # includes a row wider than one wavefront pass
    [(20, 16)],
    [(11, 24), (13, 40), (5, 8), (900, 256), (64, 4)],
]


def _gpu_forward(p):
    return ext.forward_mixed_D(dev(p["weights"]), dev(p["table_offsets"]), dev(p["dim_offsets"]),
                               int(p["dim_offsets"][-1]), dev(p["indices"]), dev(p["offsets"]),
                               dev(p["per_sample_weights"]), 200, 1, False).cpu().numpy()


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("tables", TABLE_SETS)
def test_forward_mixed_matches_oracle(oracle, tables, weighted, dtype):
    p = make_mixed_problem(len(tables), tables, B=19, L=9, dtype=dtype, weighted=weighted)
    want = oracle.forward_mixed(p["weights"], p["table_offsets"], p["dim_offsets"], p["indices"], p["offsets"],
                                p["per_sample_weights"])
    got = _gpu_forward(p)
    assert got.shape == want.shape and got.dtype == want.dtype
    assert_close(got, want, TOL[np.dtype(dtype)])


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
@pytest.mark.parametrize("mode", ["sgd", "adagrad", "adagrad_weighted"])
@pytest.mark.parametrize("tables", TABLE_SETS)
def test_backward_mixed_matches_oracle(oracle, tables, mode, dtype):
    _check_backward_mixed(oracle, tables, mode, dtype, B=23, L=8)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("mode", ["sgd", "adagrad", "adagrad_weighted"])
def test_backward_mixed_hot_rows(oracle, mode, dtype):
    """Thousands of lookups per table: rows with one occurrence (strip fast path), a few (strip
    batches), 9..256 (one chunk record, one wavefront) and more than 256 (several chunks, partial
    rows, the finishing kernel), also in a table whose rows are wider than 64 vectors, and more
    than 64 unique rows per table."""
    tables = [(3, 520), (2000, 36), (5, 64), (4000, 128), (1, 8), (700, 200)]
    _check_backward_mixed(oracle, tables, mode, dtype, B=300, L=24)


@pytest.mark.parametrize("T", [37, 100])
@pytest.mark.parametrize("mode", ["sgd", "adagrad_weighted"])
def test_backward_mixed_many_small_tables(oracle, mode, T):
    """Dozens of tables of a few rows each: a strip of 64 unique rows spans many tables of
    different widths (narrow, odd vector counts, wider than 64 vectors side by side), and the
    bag of a gradient row id b*T+t is found for table counts that are not small powers of two."""
    widths = [4, 8, 12, 260, 64, 20, 36, 128, 4, 100]
    tables = [(1 + (3 * t) % 9, widths[t % len(widths)]) for t in range(T)]
    _check_backward_mixed(oracle, tables, mode, np.float32, B=50, L=3)


def _check_backward_mixed(oracle, tables, mode, dtype, B, L):
    weighted = mode.endswith("weighted")
    p = make_mixed_problem(len(tables) + 7, tables, B=B, L=L, dtype=dtype, weighted=weighted)
    optimizer = "sgd" if mode == "sgd" else "adagrad"
    w_ref = p["weights"].copy()
    st_dtype = np.float64 if dtype == np.float64 else np.float32
    st_ref = np.zeros(sum(p["rows"]), st_dtype)
    gpsw_ref = oracle.backward_mixed(optimizer, p["grad_output"], w_ref, p["table_offsets"], p["table_dim_offsets"],
                                     p["dim_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st_ref,
                                     p["per_sample_weights"])
    w = dev(p["weights"])
    st = torch.zeros(sum(p["rows"]), device=DEV, dtype=torch.float64 if dtype == np.float64 else torch.float32)
    args = (dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"]), int(p["dim_offsets"][-1]),
            dev(p["indices"]), dev(p["offsets"]))
    if optimizer == "sgd":
        gpsw = ext.backward_sgd_mixed_D(dev(p["grad_output"]), w, *args, st, 0.05)
    else:
        gpsw = ext.backward_exact_adagrad_mixed_D(dev(p["grad_output"]), w, *args, dev(p["per_sample_weights"]), st,
                                                  0.05, 0.1, False, 1)
    torch.cuda.synchronize()
    tol = TOL[np.dtype(dtype)]
    assert_close(w.cpu().numpy(), w_ref, tol)
    if optimizer == "adagrad":
        assert_close(st.cpu().numpy(), st_ref, 1e-3 if dtype == np.float16 else max(tol, 1e-6))
    if weighted:
        assert_close(gpsw.cpu().numpy(), gpsw_ref, tol)
    # rows no lookup touches keep their bits
    keys = p["table_dim_offsets"][np.repeat(np.arange(p["T"] * p["B"]), np.diff(p["offsets"])) // p["B"]] + \
        p["indices"]
    touched = np.zeros(sum(p["rows"]), bool)
    touched[keys] = True
    for t, (E, D) in enumerate(tables):
        sl = slice(int(p["table_offsets"][t]), int(p["table_offsets"][t + 1]))
        rows_t = ~touched[p["table_dim_offsets"][t]:p["table_dim_offsets"][t + 1]]
        assert w.cpu().numpy()[sl].reshape(E, D)[rows_t].tobytes() == p["weights"][sl].reshape(E, D)[rows_t].tobytes()


def test_equal_dims_reproduce_the_uniform_kernels():
    """With every D_t equal the mixed path computes the same sums as the uniform-D path; the
    forward outputs agree to rounding and the layouts map onto each other ([B, T*D] == [B, T, D])."""
    tables = [(200, 64)] * 4
    p = make_mixed_problem(5, tables, B=40, L=10, dtype=np.float32)
    got = _gpu_forward(p)
    uni = ext.forward(dev(p["weights"].reshape(800, 64)), dev(p["table_dim_offsets"][:-1].copy()),
                      dev(p["indices"]), dev(p["offsets"]), None, 200, 1, False).cpu().numpy()
    assert_close(got, uni.reshape(40, 256), 1e-6)


def test_module_mixed_like_the_reference_test(oracle):
    """test_backward_adagrad_mixed (test_table_batched_embeddings.py:395-521) through the module:
    weights set per table via split_embedding_weights, outputs read via split_output, state via
    split_optimizer_state."""
    embeddings = [(100, 16), (100, 64), (100, 8)]
    B, L = 32, 5
    cc = ops.MixedDimTableBatchedEmbeddingBags(embeddings, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD,
                                               learning_rate=0.5, eps=0.2).cuda()
    assert cc.total_D == 88 and cc.table_offsets.dtype == torch.int64 and cc.dim_offsets.tolist() == [0, 16, 80, 88]
    assert cc.table_dim_offsets.tolist() == [0, 100, 200, 300] and cc.optimizer_state.shape == (300,)
    p = make_mixed_problem(9, embeddings, B, L, np.float32, zipf=1.1)
    for t, w_t in enumerate(cc.split_embedding_weights()):
        lo, hi = int(p["table_offsets"][t]), int(p["table_offsets"][t + 1])
        w_t.copy_(dev(p["weights"][lo:hi].reshape(embeddings[t])))
    out = cc(dev(p["indices"]), dev(p["offsets"]))
    want = oracle.forward_mixed(p["weights"], p["table_offsets"], p["dim_offsets"], p["indices"], p["offsets"])
    for t, o_t in enumerate(cc.split_output(out)):
        assert_close(o_t.detach().cpu().numpy(), want[:, p["dim_offsets"][t]:p["dim_offsets"][t + 1]], 1e-5)
    out.backward(dev(p["grad_output"]))
    w_ref = p["weights"].copy()
    st_ref = np.zeros(300, np.float32)
    oracle.backward_mixed("adagrad", p["grad_output"], w_ref, p["table_offsets"], p["table_dim_offsets"],
                          p["dim_offsets"], p["indices"], p["offsets"], 0.5, 0.2, st_ref)
    for t, (w_t, s_t) in enumerate(zip(cc.split_embedding_weights(), cc.split_optimizer_state())):
        lo, hi = int(p["table_offsets"][t]), int(p["table_offsets"][t + 1])
        assert_close(w_t.cpu().numpy(), w_ref[lo:hi].reshape(embeddings[t]), 1e-5)
        assert_close(s_t.cpu().numpy(), st_ref[p["table_dim_offsets"][t]:p["table_dim_offsets"][t + 1]], 1e-5)


def test_mixed_bad_arguments():
    w = torch.zeros(64, device=DEV)
    i32 = torch.zeros(3, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="int64"):
        ext.forward_mixed_D(w, i32[:2], i32[:2], 4, i32[:1], i32[:2], None, 200, 1, False)
    with pytest.raises(RuntimeError, match="multiple of 4"):
        ext.forward_mixed_D(w, torch.tensor([0, 6], device=DEV), torch.tensor([0, 6], dtype=torch.int32, device=DEV),
                            6, i32[:1], i32[:2], None, 200, 1, False)


@pytest.mark.parametrize("seed", range(24))
def test_backward_mixed_random_sweep(oracle, seed):
    """Seeded random table sets: 1..12 tables, rows from 1 to thousands, widths from 4 to wider
    than a wavefront pass (power-of-two and odd vector counts), bags from a handful to hundreds,
    so that single-occurrence rows, batches, rows of one chunk and rows of several chunks all occur."""
    rs = np.random.RandomState(500 + seed)
    T = int(rs.choice([1, 2, 3, 6, 12]))
    tables = [(int(rs.choice([1, 3, 40, 600, 5000])), int(rs.choice([4, 8, 12, 20, 32, 64, 100, 128, 256, 264, 520])))
              for _ in range(T)]
    dtype = [np.float32, np.float16, np.float64][seed % 3]
    mode = ["sgd", "adagrad", "adagrad_weighted"][(seed // 3) % 3]
    B = int(rs.choice([1, 9, 70, 400]))
    L = int(rs.choice([1, 5, 20]))
    _check_backward_mixed(oracle, tables, mode, dtype, B=B, L=L)


def test_backward_mixed_rows_of_many_chunks_across_queue_boundaries(oracle):
    """Eight tables of one or two rows each, hundreds of lookups per bag: every row is summed in
    several chunks, and the rows -- one or two per eighth of the sorted positions -- put their chunk
    records into different per-XCD queues; widths of 1, 3, 12 and 64 vectors."""
    tables = [(1, 4), (2, 12), (1, 48), (2, 256), (1, 8), (2, 100), (1, 64), (2, 36)]
    for mode in ("sgd", "adagrad_weighted"):
        _check_backward_mixed(oracle, tables, mode, np.float32, B=40, L=60)


def test_backward_mixed_densest_chunk_records(oracle):
    """Every row nine times: the most chunk records a batch can queue (one per nine lookups), in
    every one of the eight per-XCD queues, with strips of 64 unique rows straddling the boundaries
    between the queues' eighths of the sorted positions and between tables of different widths."""
    rows, times = 6400, 9
    tables = [(rows, 8), (rows, 24), (rows, 4), (rows, 12), (rows, 8), (rows, 40), (rows, 4), (rows, 16)]
    B, L = 960, 60  # B * L = rows * times lookups per table
    p = make_mixed_problem(11, tables, B=B, L=L, dtype=np.float32)
    rs = np.random.RandomState(12)
    T = len(tables)
    p["offsets"] = np.arange(0, T * B * L + 1, L, dtype=np.int32)
    p["indices"] = np.concatenate([rs.permutation(np.repeat(np.arange(rows, dtype=np.int32), times))
                                   for _ in range(T)])
    p["n"] = p["indices"].size
    for mode in ("sgd", "adagrad"):
        w_ref = p["weights"].copy()
        st_ref = np.zeros(T * rows, np.float32)
        oracle.backward_mixed(mode, p["grad_output"], w_ref, p["table_offsets"], p["table_dim_offsets"],
                              p["dim_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st_ref)
        w, st = dev(p["weights"]), torch.zeros(T * rows, device=DEV)
        args = (dev(p["grad_output"]), w, dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"]),
                int(p["dim_offsets"][-1]), dev(p["indices"]), dev(p["offsets"]))
        if mode == "sgd":
            ext.backward_sgd_mixed_D(*args, st, 0.05)
        else:
            ext.backward_exact_adagrad_mixed_D(*args, None, st, 0.05, 0.1, False, 1)
        torch.cuda.synchronize()
        assert_close(w.cpu().numpy(), w_ref, 1e-5)
        if mode == "adagrad":
            assert_close(st.cpu().numpy(), st_ref, 1e-5)


def test_backward_mixed_workspace_size_is_checked():
    """The workspace must follow tbe_backward_mixed_workspace_layout: a smaller one (here the
    layout of uniform tables of four columns) is refused, not overrun."""
    import tbe_native
    p = make_mixed_problem(3, [(50, 8), (20, 16), (10, 4)], B=10, L=4, dtype=np.float32)
    n, T = p["n"], 3
    need = tbe_native.backward_mixed_workspace_layout(n, tbe_native.DTYPE_F32, T).total_bytes
    small = tbe_native.backward_workspace_layout(n, 4, tbe_native.DTYPE_F32, T).total_bytes
    assert small < need
    ws = torch.zeros(small, dtype=torch.uint8, device=DEV)
    w, go = dev(p["weights"]), dev(p["grad_output"])
    to, tdo, do = dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"])
    idx, off = dev(p["indices"]), dev(p["offsets"])
    vp = lambda t: t.data_ptr()
    rc = tbe_native.load().tbe_backward_mixed(
        tbe_native.OPT_SGD, vp(go), vp(w), tbe_native.DTYPE_F32, 4, 80, 0, vp(to), vp(tdo), vp(do),
        int(p["dim_offsets"][-1]), 3, vp(idx), idx.numel(), vp(off), 10, None, None, 0.1, 0.0, None, 0, 0, 0,
        vp(ws), ws.numel(), None)
    assert rc == 2  # TBE_ERR_WORKSPACE
    assert "workspace" in tbe_native.load().tbe_last_error().decode()
    torch.cuda.synchronize()
    np.testing.assert_array_equal(w.cpu().numpy(), p["weights"])
