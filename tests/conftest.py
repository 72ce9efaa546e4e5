import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PACKAGE = os.path.join(ROOT, "sparse-ads-baselines_amd")
for p in (ROOT, PACKAGE):
    if p not in sys.path:
        sys.path.insert(0, p)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_golden(name):
    with np.load(os.path.join(GOLDEN, name + ".npz"), allow_pickle=False) as z:
        d = {k: z[k] for k in z.files}
    for k in ("T", "E", "D", "B"):
        d[k] = int(d[k])
    d["lr"], d["eps"], d["optimizer"] = float(d["lr"]), float(d["eps"]), str(d["optimizer"])
    return d


GOLDEN_CASES = ["cfg1_sgd_f32", "ragged_adagrad_f32", "weighted_adagrad_f32", "weighted_adagrad_f16", "sgd_f64",
                "hot_row_sgd_f32"]


def make_problem(seed, T, E, D, B, L, dtype, ragged=True, weighted=False, zipf=None, rows=None):
    """Seeded synthetic problem in the layout of test_table_batched_embeddings.py:24-31:
    table-major int32 indices, int32 offsets of length T*B+1.  `rows` = per-table row counts
    (default E for every table)."""
    rs = np.random.RandomState(seed)
    rows = [E] * T if rows is None else list(rows)
    lengths = rs.randint(0, L + 1, size=(T, B)) if ragged else np.full((T, B), L)
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    n = int(offsets[-1])
    per_table = lengths.sum(axis=1)
    chunks = []
    for t in range(T):
        m = int(per_table[t])
        if zipf:
            chunks.append((rs.zipf(zipf, size=m) % rows[t]).astype(np.int32))
        else:
            chunks.append(rs.randint(0, rows[t], size=m).astype(np.int32))
    indices = np.concatenate(chunks) if chunks else np.zeros(0, np.int32)
    table_offsets = np.concatenate([[0], np.cumsum(rows[:-1])]).astype(np.int32)
    weights = rs.uniform(-0.01, 0.01, size=(int(sum(rows)), D)).astype(dtype)
    grad_output = rs.randn(B, T, D).astype(dtype)
    psw = rs.uniform(0, 1, size=n).astype(dtype) if weighted else None
    return dict(T=T, B=B, D=D, rows=rows, table_offsets=table_offsets, offsets=offsets, indices=indices,
                weights=weights, grad_output=grad_output, per_sample_weights=psw, n=n)


@pytest.fixture(scope="session")
def oracle():
    from oracle import tbe_oracle
    tbe_oracle.lib()
    return tbe_oracle


def make_mixed_problem(seed, embeddings, B, L, dtype, weighted=False, zipf=1.2):
    """Seeded problem for tables with per-table (rows, dim): flat 1-D weights and the three offset
    arrays of MixedDimTableBatchedEmbeddingBags (table_batched_embeddings_ops.py:356-369)."""
    rs = np.random.RandomState(seed)
    rows, dims = zip(*embeddings)
    T = len(embeddings)
    lengths = rs.randint(0, L + 1, size=(T, B))
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    per_table = lengths.sum(axis=1)
    indices = np.concatenate([(rs.zipf(zipf, size=int(per_table[t])) % rows[t]) for t in range(T)]).astype(np.int32)
    n = indices.size
    return dict(T=T, B=B, rows=list(rows), dims=list(dims), n=n, offsets=offsets, indices=indices,
                table_offsets=np.concatenate([[0], np.cumsum([r * d for r, d in embeddings])]).astype(np.int64),
                table_dim_offsets=np.concatenate([[0], np.cumsum(rows)]).astype(np.int32),
                dim_offsets=np.concatenate([[0], np.cumsum(dims)]).astype(np.int32),
                weights=rs.uniform(-0.01, 0.01, size=sum(r * d for r, d in embeddings)).astype(dtype),
                grad_output=rs.randn(B, sum(dims)).astype(dtype),
                per_sample_weights=rs.uniform(0, 1, size=n).astype(dtype) if weighted else None)
