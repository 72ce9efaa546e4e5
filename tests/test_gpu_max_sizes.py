"""Maximum sizes: tables whose concatenated row count is the largest the int32 key type allows
(2^31 - 2 rows, 17 to 34 GB of weights).  Keys, sort digits and row addresses are exercised up to
their last bit: lookups hit the last rows of the last table and the rows on either side of every
power-of-two boundary of the byte and element offsets.

The expected values come from the same lookups on a compacted problem that keeps only the rows
touched, in the same order (an order-preserving renumbering leaves the sorted order, the runs
and every sum unchanged): the HIP path on the compacted tables must agree bit for bit, and the
oracle on the compacted tables within the usual tolerance."""
import numpy as np
import pytest
import torch

import table_batched_embeddings as ext
from gpu_util import DEV, assert_close, dev

pytestmark = pytest.mark.gpu

ROWS = [1000, 2 ** 31 - 2 - 1000]
FILL = 0.25


def _lookups(seed, B, L):
    """Ragged bags over both tables; table 1 draws from a pool of boundary rows, the last rows
    and random rows, with one row repeated often enough to take the long-run path."""
    rs = np.random.RandomState(seed)
    E1 = ROWS[1]
    pool = [E1 - 1 - k for k in range(48)]
    for bit in range(20, 31):
        pool += [(1 << bit) - 1000 + d for d in (-1, 0, 1)]   # key = row + 1000 sits on 2^bit - 1, 2^bit, 2^bit + 1
    pool += list(rs.randint(0, E1, size=200))
    pool = np.array(pool, dtype=np.int64)
    hot = E1 - 7
    lengths = rs.randint(0, L + 1, size=(2, B))
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    n0, n1 = int(lengths[0].sum()), int(lengths[1].sum())
    idx0 = rs.randint(0, ROWS[0], size=n0)
    idx1 = pool[rs.randint(0, pool.size, size=n1)]
    idx1[rs.rand(n1) < 0.15] = hot
    indices = np.concatenate([idx0, idx1]).astype(np.int32)
    assert (idx1 == hot).sum() > 32
    return indices, offsets


def _compact(indices, offsets, B):
    """Order-preserving renumbering of the touched rows: (keys of the touched rows, ascending;
    compact table_offsets; compact indices)."""
    table_offsets = np.array([0, ROWS[0]], dtype=np.int64)
    n0 = int(offsets[B])
    keys = np.concatenate([indices[:n0].astype(np.int64), indices[n0:].astype(np.int64) + table_offsets[1]])
    touched = np.unique(keys)
    rank = np.searchsorted(touched, keys)
    first_of_table1 = int(np.searchsorted(touched, table_offsets[1]))
    compact_offsets = np.array([0, first_of_table1], dtype=np.int32)
    compact_indices = rank.copy()
    compact_indices[n0:] -= first_of_table1
    return touched, compact_offsets, compact_indices.astype(np.int32)


@pytest.mark.parametrize("mode,dtype,D", [("sgd", torch.float32, 4), ("adagrad_weighted", torch.float16, 8),
                                          ("approx", torch.float32, 4)])
def test_rows_up_to_the_int32_limit(oracle, mode, dtype, D):
    B, L = 48, 12
    total = sum(ROWS)
    assert total == 2 ** 31 - 2
    need = total * D * torch.empty(0, dtype=dtype).element_size() + total * 4 + (4 << 30)
    free, _ = torch.cuda.mem_get_info()
    if free < need:
        pytest.skip("needs %.0f GB of free device memory, %.0f GB are free" % (need / 1e9, free / 1e9))
    indices, offsets = _lookups(5, B, L)
    touched, compact_offsets, compact_indices = _compact(indices, offsets, B)
    n = indices.size
    gen = torch.Generator(device=DEV).manual_seed(17)
    rows0 = (torch.rand(touched.size, D, device=DEV, generator=gen, dtype=torch.float32) * 0.2 - 0.1).to(dtype)
    touched_d = torch.from_numpy(touched).to(DEV)

    big = torch.full((total, D), FILL, dtype=dtype, device=DEV)
    big[touched_d] = rows0
    small = rows0.clone()
    go = torch.randn(B, 2, D, device=DEV, generator=gen, dtype=torch.float32).to(dtype)
    weighted = mode.endswith("weighted")
    psw = torch.rand(n, device=DEV, generator=gen, dtype=torch.float32).to(dtype) if weighted else None
    big_to = dev(np.array([0, ROWS[0]], dtype=np.int32))
    small_to = dev(compact_offsets)
    idx_big, idx_small, off = dev(indices), dev(compact_indices), dev(offsets)

    # forward
    out_big = ext.forward(big, big_to, idx_big, off, psw, 200, 1, False)
    out_small = ext.forward(small, small_to, idx_small, off, psw, 200, 1, False)
    assert torch.equal(out_big, out_small)
    w_np = rows0.cpu().numpy()
    want_out = oracle.forward(w_np, compact_offsets, compact_indices, offsets,
                              None if psw is None else psw.cpu().numpy())
    assert_close(out_big.cpu().numpy(), want_out, 1e-5 if dtype == torch.float32 else 2e-3, "forward")

    # update
    lr, eps = 0.05, 0.1
    state_big = state_small = None
    if mode != "sgd":
        state_big = torch.zeros(total, device=DEV)
        state_small = torch.zeros(touched.size, device=DEV)
    if mode == "sgd":
        ext.backward_sgd(go, big, big_to, idx_big, off, lr, 200, 1, False)
        ext.backward_sgd(go, small, small_to, idx_small, off, lr, 200, 1, False)
        g_big = g_small = None
        oracle.backward("sgd", go.cpu().numpy(), w_np, compact_offsets, compact_indices, offsets, lr)
        want_g, want_state = None, None
    elif mode == "approx":
        g_big = ext.backward_approx_adagrad(go, big, big_to, idx_big, off, psw, state_big, lr, eps, 200, False, 1)
        g_small = ext.backward_approx_adagrad(go, small, small_to, idx_small, off, psw, state_small, lr, eps, 200,
                                              False, 1)
        want_state = np.zeros(touched.size, np.float32)
        want_g = oracle.backward_approx(go.cpu().numpy(), w_np, compact_offsets, compact_indices, offsets, lr, eps,
                                        want_state)
    else:
        g_big = ext.backward_exact_adagrad(go, big, big_to, idx_big, off, psw, state_big, lr, eps, False, 1)
        g_small = ext.backward_exact_adagrad(go, small, small_to, idx_small, off, psw, state_small, lr, eps, False, 1)
        want_state = np.zeros(touched.size, np.float32)
        want_g = oracle.backward("adagrad", go.cpu().numpy(), w_np, compact_offsets, compact_indices, offsets, lr,
                                 eps, want_state, psw.cpu().numpy())["grad_psw"]
    torch.cuda.synchronize()
    got_rows = big[touched_d]
    assert torch.equal(got_rows, small), "rows of the full-size tables differ from the compacted run"
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    assert_close(got_rows.cpu().numpy(), w_np, tol, "weights")   # w_np was updated in place by the oracle
    if state_big is not None:
        assert torch.equal(state_big[touched_d], state_small)
        assert_close(state_small.cpu().numpy(), want_state, 1e-5, "state")
        state_big[touched_d] = 0
        assert not bool(state_big.any()), "optimizer state written outside the touched rows"
    if g_big is not None:
        assert torch.equal(g_big, g_small)
        assert_close(g_big.cpu().numpy(), want_g, 2e-3, "grad_psw")
    # no other row of the 2^31 - 2 was written
    big[touched_d] = FILL
    assert bool((big == FILL).all()), "weights written outside the touched rows"
    del big, state_big
    torch.cuda.empty_cache()


@pytest.mark.parametrize("mode", ["adagrad_weighted", "approx"])
def test_mixed_dim_rows_up_to_the_int32_limit(oracle, mode):
    """The same for tables of different widths (a narrow table of 2^31 - 1002 rows after a wider
    one of 1000): flat weights of 8.6 G elements, int64 element offsets, the row-number keys up
    to their last bit."""
    B, L = 48, 12
    dims = [8, 4]
    indices, offsets = _lookups(9, B, L)
    touched, compact_row_offsets, compact_indices = _compact(indices, offsets, B)
    n = indices.size
    first1 = int(compact_row_offsets[1])
    rows_small = [first1, touched.size - first1]
    gen = torch.Generator(device=DEV).manual_seed(23)
    small = torch.rand(rows_small[0] * dims[0] + rows_small[1] * dims[1], device=DEV, generator=gen) * 0.2 - 0.1
    elements = [ROWS[0] * dims[0], ROWS[1] * dims[1]]
    big = torch.full((sum(elements),), FILL, device=DEV)
    # touched rows of the full-size tables take the compacted tables' values
    keys0 = torch.from_numpy(touched[:first1]).to(DEV)
    keys1 = torch.from_numpy(touched[first1:] - ROWS[0]).to(DEV)
    big[:elements[0]].view(ROWS[0], dims[0])[keys0] = small[:rows_small[0] * dims[0]].view(-1, dims[0])
    big[elements[0]:].view(ROWS[1], dims[1])[keys1] = small[rows_small[0] * dims[0]:].view(-1, dims[1])
    go = torch.randn(B, sum(dims), device=DEV, generator=gen)
    weighted = mode.endswith("weighted")
    psw = torch.rand(n, device=DEV, generator=gen) if weighted else None
    dim_offsets = dev(np.array([0, dims[0], sum(dims)], dtype=np.int32))

    def arguments(rows):
        return (dev(np.array([0, rows[0] * dims[0], rows[0] * dims[0] + rows[1] * dims[1]], dtype=np.int64)),
                dev(np.array([0, rows[0], rows[0] + rows[1]], dtype=np.int32)))
    big_to, big_rows = arguments(ROWS)
    small_to, small_rows = arguments(rows_small)
    idx_big, idx_small, off = dev(indices), dev(compact_indices), dev(offsets)

    out_big = ext.forward_mixed_D(big, big_to, dim_offsets, sum(dims), idx_big, off, psw, 200, 1, False)
    out_small = ext.forward_mixed_D(small, small_to, dim_offsets, sum(dims), idx_small, off, psw, 200, 1, False)
    assert torch.equal(out_big, out_small)
    w_np = small.cpu().numpy()
    psw_np = None if psw is None else psw.cpu().numpy()
    want_out = oracle.forward_mixed(w_np, small_to.cpu().numpy(), dim_offsets.cpu().numpy(), compact_indices, offsets,
                                    psw_np)
    assert_close(out_big.cpu().numpy(), want_out, 1e-5, "forward")

    lr, eps = 0.05, 0.1
    state_big = torch.zeros(sum(ROWS), device=DEV)
    state_small = torch.zeros(touched.size, device=DEV)
    want_state = np.zeros(touched.size, np.float32)
    if mode == "approx":
        run = lambda w, to, rows, idx, st: ext.backward_approx_adagrad_mixed_D(
            go, w, to, rows, dim_offsets, sum(dims), idx, off, psw, st, lr, eps, 200, False, 1)
        want_g = oracle.backward_approx_mixed(go.cpu().numpy(), w_np, small_to.cpu().numpy(),
                                              small_rows.cpu().numpy(), dim_offsets.cpu().numpy(), compact_indices,
                                              offsets, lr, eps, want_state, psw_np)
    else:
        run = lambda w, to, rows, idx, st: ext.backward_exact_adagrad_mixed_D(
            go, w, to, rows, dim_offsets, sum(dims), idx, off, psw, st, lr, eps, False, 1)
        want_g = oracle.backward_mixed("adagrad", go.cpu().numpy(), w_np, small_to.cpu().numpy(),
                                       small_rows.cpu().numpy(), dim_offsets.cpu().numpy(), compact_indices, offsets,
                                       lr, eps, want_state, psw_np)
    g_big = run(big, big_to, big_rows, idx_big, state_big)
    g_small = run(small, small_to, small_rows, idx_small, state_small)
    torch.cuda.synchronize()
    got0 = big[:elements[0]].view(ROWS[0], dims[0])[keys0].reshape(-1)
    got1 = big[elements[0]:].view(ROWS[1], dims[1])[keys1].reshape(-1)
    got = torch.cat([got0, got1])
    assert torch.equal(got, small), "rows of the full-size tables differ from the compacted run"
    assert_close(got.cpu().numpy(), w_np, 1e-5, "weights")
    touched_d = torch.from_numpy(touched).to(DEV)
    assert torch.equal(state_big[touched_d], state_small)
    assert_close(state_small.cpu().numpy(), want_state, 1e-5, "state")
    if weighted:
        assert torch.equal(g_big, g_small)
        assert_close(g_big.cpu().numpy(), want_g, 1e-5, "grad_psw")
    state_big[touched_d] = 0
    assert not bool(state_big.any()), "optimizer state written outside the touched rows"
    big[:elements[0]].view(ROWS[0], dims[0])[keys0] = FILL
    big[elements[0]:].view(ROWS[1], dims[1])[keys1] = FILL
    assert bool((big == FILL).all()), "weights written outside the touched rows"
    del big, state_big
    torch.cuda.empty_cache()
