"""GPU parity of the pooled forward (tbe_forward through the C ABI) against the CPU oracle,
the EmbeddingBag fixtures, and size-independent properties at the benchmark's full shape.

Tolerances (north star): fp32 1e-5 relative, fp16 1e-2; fp64 1e-12.  The kernel sums a
bag in a different (fixed) order than the oracle's serial loop, so fp results are compared
with a tolerance; everything that involves no rounding is compared bit for bit."""
import numpy as np
import pytest
import torch

from conftest import GOLDEN_CASES, load_golden, make_problem
from gpu_util import DEV, assert_close, dev, gpu_forward

import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float16): 1e-2, np.dtype(np.float64): 1e-12}

# (T, E, D, B, L): D covers every lane-group width: 4 -> 1 vector ... 256 -> 64 vectors, 12/520 -> generic / wide
SHAPES = [(2, 1000, 32, 64, 4), (3, 50, 128, 33, 20), (1, 7, 4, 5, 3), (2, 100, 12, 17, 9), (2, 30, 520, 9, 5),
          (4, 20, 64, 70, 40), (2, 100, 256, 50, 70), (1, 300, 8, 40, 130), (2, 64, 16, 31, 6), (1, 10, 2048, 3, 4)]


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
def test_forward_matches_oracle(oracle, shape, weighted, dtype):
    T, E, D, B, L = shape
    p = make_problem(hash(shape) % 1000, T, E, D, B, L, dtype, ragged=True, weighted=weighted, zipf=1.3)
    want = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"], p["per_sample_weights"])
    got = gpu_forward(p)
    assert got.dtype == want.dtype and got.shape == (B, T, D)
    assert_close(got, want, TOL[np.dtype(dtype)])


@pytest.mark.parametrize("dtype,D", [(np.float32, 128), (np.float16, 64), (np.float32, 12), (np.float64, 16)])
@pytest.mark.parametrize("weighted", [False, True])
def test_forward_thousands_of_ragged_bags(oracle, dtype, D, weighted):
    """Nine thousand ragged bags: empty ones, bags of more than 64 lookups (several index slices
    per bag), a bag count that is not a multiple of the wavefronts per workgroup."""
    p = make_problem(77, T=3, E=400, D=D, B=3001, L=9, dtype=dtype, ragged=True, weighted=weighted, zipf=1.2)
    lengths = np.diff(p["offsets"]).copy()
    rs = np.random.RandomState(5)
    lengths[rs.randint(0, lengths.size, size=40)] = rs.randint(65, 200, size=40)  # a few long bags
    p["offsets"] = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    p["n"] = int(p["offsets"][-1])
    p["indices"] = rs.randint(0, 400, size=p["n"]).astype(np.int32)
    if weighted:
        p["per_sample_weights"] = rs.uniform(0, 1, size=p["n"]).astype(dtype)
    want = oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"], p["per_sample_weights"])
    got = gpu_forward(p)
    assert_close(got, want, TOL[np.dtype(dtype)])
    assert not got[(lengths == 0).reshape(3, 3001).T].any()  # empty bags give zeros


@pytest.mark.parametrize("name", GOLDEN_CASES)
def test_forward_matches_embeddingbag_fixture(name):
    g = load_golden(name)
    g["table_offsets"] = (np.arange(g["T"]) * g["E"]).astype(np.int32)
    got = gpu_forward(g)
    assert_close(got, g["expected_output"], TOL[g["weights"].dtype])


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
def test_single_lookup_bags_copy_rows_bit_exact(dtype):
    p = make_problem(1, T=5, E=999, D=128, B=257, L=1, dtype=dtype, ragged=False)
    got = gpu_forward(p)
    rows = p["table_offsets"][np.arange(5)[:, None]] + p["indices"].reshape(5, 257)
    want = p["weights"][rows].transpose(1, 0, 2)  # [B][T][D]
    # 0 + w == w exactly for every w except that 0 + (-0) is +0, so compare values, not bytes
    assert got.dtype == want.dtype and np.array_equal(got, want)


def test_empty_bags_and_all_empty_input():
    p = make_problem(2, T=3, E=30, D=64, B=200, L=2, dtype=np.float32)
    got = gpu_forward(p)
    empty = np.diff(p["offsets"]) == 0
    assert empty.any()
    for bag in np.nonzero(empty)[0]:
        assert not got[bag % 200, bag // 200].any()
    p0 = make_problem(3, T=2, E=30, D=32, B=7, L=0, dtype=np.float32)
    assert p0["n"] == 0
    assert not gpu_forward(p0).any()


def test_unit_weights_equal_unweighted_bit_exact():
    p = make_problem(4, T=2, E=500, D=128, B=100, L=25, dtype=np.float32, weighted=True)
    p["per_sample_weights"][:] = 1.0
    assert gpu_forward(p, weighted=True).tobytes() == gpu_forward(p, weighted=False).tobytes()


def test_two_runs_are_bit_identical():
    p = make_problem(5, T=4, E=2000, D=64, B=300, L=30, dtype=np.float16, weighted=True, zipf=1.1)
    assert gpu_forward(p).tobytes() == gpu_forward(p).tobytes()


def test_per_table_row_counts():
    p = make_problem(6, T=4, E=0, D=32, B=50, L=8, dtype=np.float32, rows=[5, 1700, 3, 40])
    from oracle import tbe_oracle
    want = tbe_oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"])
    assert_close(gpu_forward(p), want, 1e-5)


def test_module_api_forward_and_launch_knobs_do_not_matter():
    """The drop-in surface: module(indices, offsets[, per_sample_weights]) as in
    test_table_batched_embeddings.py:145-160; BT_block_size / shmem / L_max change nothing
    (table_batched_embeddings_benchmark.py:179-206)."""
    T, E, D, B, L = 3, 100, 64, 16, 5
    p = make_problem(7, T, E, D, B, L, np.float32, ragged=False, weighted=True)
    cc = ops.TableBatchedEmbeddingBags(T, E, D).cuda()
    assert tuple(cc.embedding_weights.shape) == (T * E, D) and cc.table_offsets.tolist() == [0, E, 2 * E]
    assert cc.optimizer_state.shape == (T * E,) and cc.optimizer_state.dtype == torch.float32
    assert set(cc.state_dict()) == {"embedding_weights", "table_offsets", "optimizer_state"}
    for t in range(T):
        cc.embedding_weights.data.view(T, E, D)[t, :, :] = dev(p["weights"][t * E:(t + 1) * E])
    y = cc(dev(p["indices"]), dev(p["offsets"]), dev(p["per_sample_weights"]))
    from oracle import tbe_oracle
    want = tbe_oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"], p["per_sample_weights"])
    assert_close(y.detach().cpu().numpy(), want, 1e-5)
    y0 = ext.forward(cc.embedding_weights.data, cc.table_offsets, dev(p["indices"]), dev(p["offsets"]), None, L, 1,
                     False)
    for bt in (1, 2, 4, 128):
        for shmem in (True, False):
            y1 = ext.forward(cc.embedding_weights.data, cc.table_offsets, dev(p["indices"]), dev(p["offsets"]),
                             None, 200, bt, shmem)
            assert torch.equal(y0, y1)


def test_bad_arguments_raise_runtime_error():
    w = torch.zeros(10, 6, device=DEV)
    i32 = torch.zeros(2, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 4"):
        ext.forward(w, i32[:1], i32[:1], i32, None, 200, 1, False)
    w = torch.zeros(10, 8, device=DEV)
    with pytest.raises(RuntimeError, match="int32"):
        ext.forward(w, i32[:1].long(), i32[:1], i32, None, 200, 1, False)


def test_full_size_forward_properties():
    """The shape of bench.py --config 2 (T=64, E=1e5, D=128 fp32, B=4096, L=20, uniform indices).
    The oracle is too slow for 5.2 M lookups, so: (a) the first two tables are compared with
    the oracle; (b) column checksum: sum_b,t out[b,t,:] == sum_p W[key_p,:] computed by an
    independent torch gather in fp64; (c) every output row of a table filled with a per-table
    constant equals L * constant exactly."""
    from oracle import tbe_oracle
    T, E, D, B, L = 64, 100000, 128, 4096, 20
    gen = torch.Generator(device=DEV).manual_seed(0)
    W = torch.empty(T * E, D, device=DEV).uniform_(-0.01, 0.01, generator=gen)
    idx = torch.randint(0, E, (T * B * L,), device=DEV, dtype=torch.int32, generator=gen)
    offsets = torch.arange(0, T * B * L + 1, L, dtype=torch.int32, device=DEV)
    table_offsets = (torch.arange(T, dtype=torch.int32, device=DEV) * E)
    out = ext.forward(W, table_offsets, idx, offsets, None, 200, 1, False)
    assert tuple(out.shape) == (B, T, D)
    # (a)
    k = 2
    want = tbe_oracle.forward(W[:k * E].cpu().numpy(), table_offsets[:k].cpu().numpy(), idx[:k * B * L].cpu().numpy(),
                              offsets[:k * B + 1].cpu().numpy())
    assert_close(out[:, :k, :].cpu().numpy(), want, 1e-5)
    # (b)
    keys = idx.long() + torch.arange(T, device=DEV).repeat_interleave(B * L) * E
    col = torch.zeros(D, dtype=torch.float64, device=DEV)
    for lo in range(0, keys.numel(), 1 << 20):
        col += W[keys[lo:lo + (1 << 20)]].double().sum(0)
    got = out.double().sum((0, 1))
    assert_close(got.cpu().numpy(), col.cpu().numpy(), 1e-5)
    # (c)
    W.view(T, E, D)[:] = (torch.arange(T, device=DEV, dtype=torch.float32) + 1).view(T, 1, 1) / 64
    out = ext.forward(W, table_offsets, idx, offsets, None, 200, 1, False)
    want_c = ((torch.arange(T, device=DEV, dtype=torch.float32) + 1) / 64 * L).view(1, T, 1).expand(B, T, D)
    assert torch.equal(out, want_c)


def test_benchmark_cli_runs_with_reference_flags():
    """The micro-benchmark keeps the reference's flag names (table_batched_embeddings_benchmark.py:360-370)."""
    import json
    import os
    import subprocess
    import sys
    from conftest import PACKAGE
    cmd = [sys.executable, os.path.join(PACKAGE, "table_batched_embeddings_benchmark.py"), "--num-tables", "4",
           "--num-embeddings", "1000", "--embedding-dim", "32", "--batch-size", "64", "--bag-size", "8", "--iters",
           "3", "--fp16"]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=280)
    assert out.returncode == 0, out.stderr[-2000:]
    records = [json.loads(line) for line in out.stdout.splitlines() if line.startswith("{")]
    # the reference's rows (:240, :266-357) for fp16 weights, plus exact SGD
    assert [r["op"] for r in records] == [
        "Forward", "Backward-SGD-EXACT", "Backward-ADAGRAD-nonstochastic-APPROX-NR",
        "Backward-ADAGRAD-stochastic-APPROX-NR", "Backward-ADAGRAD-nonstochastic-EXACT-NR",
        "Backward-ADAGRAD-stochastic-EXACT-NR"]
    assert all(r["BW_GBps"] > 0 for r in records)
    for extra in (["--managed"], ["--mixed"]):  # host-resident tables / per-table dimensions
        out = subprocess.run(cmd[:-1] + extra, capture_output=True, text=True, timeout=280)
        assert out.returncode == 0, out.stderr[-2000:]
        ops_run = [json.loads(line)["op"] for line in out.stdout.splitlines() if line.startswith("{")]
        assert ops_run == ["Forward", "Backward-SGD-EXACT", "Backward-ADAGRAD-nonstochastic-APPROX-NR",
                           "Backward-ADAGRAD-nonstochastic-EXACT-NR"]
