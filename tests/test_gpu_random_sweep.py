"""Seeded random sweep of small problems through the C ABI against the oracle.

Every case draws its own shape: number of tables, per-table row counts (ragged, down to one row),
row width (any multiple of 4 up to wide rows), bag count and lengths (empty bags, empty tables, a
few bags of more than 64 lookups), index skew, dtype, optimizer and weighting.  Forward outputs,
the integer stages (sorted keys, stable positions, segment boundaries: bit-exact) and the updated
weights / optimizer state / per-sample-weight gradients (1e-5 fp32, 1e-2 fp16, 1e-7 fp64) are
compared with the oracle; rows without a lookup must keep their bits."""
import numpy as np
import pytest

from gpu_util import assert_close, gpu_backward, gpu_forward

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float16): 1e-2, np.dtype(np.float64): 1e-7}


def _draw(seed):
    rs = np.random.RandomState(1000 + seed)
    T = int(rs.choice([1, 2, 3, 5, 9, 40]))
    rows = [int(rs.choice([1, 2, 7, 50, 333, 2000, 70000])) for _ in range(T)]
    D = int(rs.choice([4, 8, 12, 16, 32, 36, 64, 128, 256, 260, 520]))
    B = int(rs.choice([1, 2, 17, 64, 129, 400]))
    L = int(rs.choice([1, 3, 8, 30]))
    dtype = [np.float32, np.float16, np.float64][seed % 3]
    mode = ["sgd", "adagrad", "adagrad_weighted"][(seed // 3) % 3]
    lengths = rs.randint(0, L + 1, size=(T, B))
    if rs.rand() < 0.5:
        lengths[rs.randint(T)] = 0  # a table nobody looks up
    if rs.rand() < 0.3:
        lengths[rs.randint(T), rs.randint(B)] = int(rs.randint(65, 300))  # more than one slice of 64
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    n = int(offsets[-1])
    per_table = lengths.sum(axis=1)
    zipf = float(rs.choice([0.0, 1.1, 1.6]))
    chunks = []
    for t in range(T):
        m = int(per_table[t])
        draw = rs.zipf(zipf, size=m) % rows[t] if zipf else rs.randint(0, rows[t], size=m)
        chunks.append(draw.astype(np.int32))
    indices = np.concatenate(chunks) if n else np.zeros(0, np.int32)
    table_offsets = np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32)
    weights = rs.uniform(-0.01, 0.01, size=(int(sum(rows)), D)).astype(dtype)
    grad_output = rs.randn(B, T, D).astype(dtype)
    psw = rs.uniform(0, 1, size=n).astype(dtype) if mode.endswith("weighted") else None
    p = dict(T=T, B=B, D=D, rows=rows, table_offsets=table_offsets, offsets=offsets, indices=indices,
             weights=weights, grad_output=grad_output, per_sample_weights=psw, n=n)
    return p, mode, np.dtype(dtype)


@pytest.mark.parametrize("seed", range(45))
def test_random_problem_matches_oracle(oracle, seed):
    p, mode, dtype = _draw(seed)
    tol = TOL[dtype]
    want_out = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"], p["per_sample_weights"])
    assert_close(gpu_forward(p), want_out, tol, "forward")

    optimizer = "sgd" if mode == "sgd" else "adagrad"
    w = p["weights"].copy()
    st = np.zeros(w.shape[0], np.float64 if dtype == np.float64 else np.float32)
    ref = oracle.backward(optimizer, p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.05, 0.1,
                          st, p["per_sample_weights"])
    got = gpu_backward(p, optimizer, 0.05, 0.1)
    if p["n"]:
        v = got["views"]
        np.testing.assert_array_equal(v["keys_sorted"], ref["keys_sorted"])
        np.testing.assert_array_equal(v["positions_sorted"], ref["positions_sorted"])
        np.testing.assert_array_equal(v["segment_starts"], ref["segment_starts"])
    assert_close(got["weights"], w, tol, "weights")
    touched = np.zeros(w.shape[0], bool)
    touched[ref["keys_sorted"]] = True
    assert got["weights"][~touched].tobytes() == p["weights"][~touched].tobytes()
    if optimizer == "adagrad":
        assert_close(got["state"], st, 1e-3 if dtype == np.float16 else max(tol, 1e-6), "state")
    if ref["grad_psw"] is not None:
        assert_close(got["grad_psw"], ref["grad_psw"], tol, "grad_psw")
