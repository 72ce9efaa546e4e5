"""GPU parity of the approximate row-wise Adagrad (tbe_backward_approx_adagrad and
tbe_backward_mixed with TBE_OPT_APPROX_ROWWISE_ADAGRAD, through the extension-module mirror)
against the oracle's one-lookup-at-a-time restatement of the reference kernel
(table_batched_embeddings_cuda.cu:648-704).  Rows repeat inside bags and across bags in every
case here; tolerances: fp32 1e-5, fp16 1e-2 (weights are rounded after every lookup on both
sides), fp64 1e-7."""
import numpy as np
import pytest
import torch

from conftest import make_mixed_problem, make_problem
from gpu_util import DEV, assert_close, dev

import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float16): 1e-2, np.dtype(np.float64): 1e-7}


def _run_gpu(p, lr, eps, state0=None, stochastic=False):
    w = dev(p["weights"])
    st_dtype = torch.float64 if w.dtype == torch.float64 else torch.float32
    st = torch.zeros(w.shape[0], dtype=st_dtype, device=DEV) if state0 is None else dev(state0)
    g = ext.backward_approx_adagrad(dev(p["grad_output"]), w, dev(p["table_offsets"]), dev(p["indices"]),
                                    dev(p["offsets"]), dev(p["per_sample_weights"]), st, lr, eps, 200, stochastic, 1)
    torch.cuda.synchronize()
    return w.cpu().numpy(), st.cpu().numpy(), None if g is None else g.cpu().numpy()


def _run_oracle(oracle, p, lr, eps, state0=None, stochastic_rounding=None):
    w = p["weights"].copy()
    st = np.zeros(w.shape[0], np.float64 if w.dtype == np.float64 else np.float32) if state0 is None else state0.copy()
    g = oracle.backward_approx(p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], lr, eps, st,
                               p["per_sample_weights"], stochastic_rounding)
    return w, st, g


@pytest.mark.parametrize("dtype,D", [(np.float32, 128), (np.float32, 4), (np.float32, 12), (np.float16, 64),
                                     (np.float16, 36), (np.float64, 8), (np.float32, 520), (np.float16, 1032)])
@pytest.mark.parametrize("weighted", [False, True])
def test_approx_adagrad_matches_oracle_with_repeated_rows(oracle, dtype, D, weighted):
    p = make_problem(31, T=3, E=60, D=D, B=90, L=7, dtype=dtype, weighted=weighted, zipf=1.3)
    assert np.unique(p["indices"]).size < p["n"] // 4  # rows repeat, inside bags and across them
    state0 = np.random.RandomState(1).uniform(0, 2, size=p["weights"].shape[0]).astype(
        np.float64 if dtype == np.float64 else np.float32)
    w, st, g = _run_gpu(p, 0.05, 0.1, state0)
    w_ref, st_ref, g_ref = _run_oracle(oracle, p, 0.05, 0.1, state0)
    tol = TOL[np.dtype(dtype)]
    assert_close(st, st_ref, 1e-5 if dtype != np.float64 else 1e-10, "state")
    assert_close(w, w_ref, tol, "weights")
    if weighted:
        assert_close(g, g_ref, tol if dtype != np.float16 else 2e-2, "grad of per-sample weights")
    # rows no lookup touches keep their bits
    touched = np.zeros(p["weights"].shape[0], bool)
    bag_table = np.repeat(np.arange(p["T"] * p["B"]), np.diff(p["offsets"])) // p["B"]
    touched[p["table_offsets"][bag_table] + p["indices"]] = True
    assert w[~touched].tobytes() == p["weights"][~touched].tobytes()
    assert st[~touched].tobytes() == state0[~touched].tobytes()


def test_approx_differs_from_exact_where_it_should_and_reruns_are_bit_identical(oracle):
    p = make_problem(32, T=2, E=30, D=32, B=200, L=5, dtype=np.float32, zipf=1.2)
    a = _run_gpu(p, 0.05, 0.1)
    b = _run_gpu(p, 0.05, 0.1)
    assert a[0].tobytes() == b[0].tobytes() and a[1].tobytes() == b[1].tobytes()
    w_exact, st_exact = p["weights"].copy(), np.zeros(60, np.float32)
    oracle.backward("adagrad", p["grad_output"], w_exact, p["table_offsets"], p["indices"], p["offsets"], 0.05, 0.1,
                    st_exact)
    # per-lookup sums of squares exceed the square of the summed gradient whenever gradients cancel
    assert np.abs(a[1] - st_exact).max() > 1.0


def test_approx_adagrad_hot_row_and_long_bags(oracle):
    """One row takes 70 % of 24 k lookups (a serial chain of ~17 k updates in one lane group),
    bags of up to 300 lookups (the reference caps a bag at L_max = 200 shared-memory slots,
    table_batched_embeddings_cuda.cu:738; there is no cap here)."""
    rs = np.random.RandomState(33)
    p = make_problem(33, T=2, E=40, D=64, B=80, L=300, dtype=np.float32, weighted=True)
    hot = rs.rand(p["n"]) < 0.7
    p["indices"][hot] = 5
    w, st, g = _run_gpu(p, 0.001, 0.1)
    w_ref, st_ref, g_ref = _run_oracle(oracle, p, 0.001, 0.1)
    assert_close(st, st_ref, 1e-5)
    assert_close(w, w_ref, 1e-5)
    assert_close(g, g_ref, 1e-4)  # dot products of rows that 17 k fp32 updates have moved


@pytest.mark.parametrize("dtype,D", [(np.float32, 8), (np.float32, 64), (np.float32, 128), (np.float32, 200),
                                     (np.float32, 256), (np.float16, 64), (np.float16, 100), (np.float16, 256),
                                     (np.float16, 512), (np.float64, 64), (np.float64, 128)])
@pytest.mark.parametrize("weighted", [False, True])
def test_approx_adagrad_rows_of_many_occurrences_in_every_lane_layout(oracle, dtype, D, weighted):
    """Rows with more than 16 occurrences get a wavefront each, whose lanes hold 1, 2, 4 or 8 elements of
    the row and which takes the occurrences 64 at a time.  The run lengths drawn here end inside the first
    batch, on a batch boundary, one past it and several batches on, in blocks of every parity."""
    rs = np.random.RandomState(36)
    lengths = [17, 31, 32, 33, 48, 49, 63, 64, 65, 80, 96, 127, 128, 129, 200, 333]
    T, E, L = 2, 40, 8
    B = (sum(lengths) + 120 + L - 1) // L
    p = make_problem(36, T=T, E=E, D=D, B=B, L=L, dtype=dtype, ragged=False, weighted=weighted)
    for t in range(T):
        rows = np.concatenate([np.full(n, r, np.int32) for r, n in enumerate(lengths)])
        rest = rs.randint(len(lengths), E, size=B * L - rows.size).astype(np.int32)
        p["indices"][t * B * L:(t + 1) * B * L] = rs.permutation(np.concatenate([rows, rest]))
    state0 = rs.uniform(0, 2, size=p["weights"].shape[0]).astype(np.float64 if dtype == np.float64 else np.float32)
    w, st, g = _run_gpu(p, 0.01, 0.1, state0)
    w_ref, st_ref, g_ref = _run_oracle(oracle, p, 0.01, 0.1, state0)
    tol = TOL[np.dtype(dtype)]
    assert_close(st, st_ref, 1e-5 if dtype != np.float64 else 1e-10, "state")
    assert_close(w, w_ref, tol, "weights")
    if weighted:
        assert_close(g, g_ref, tol if dtype != np.float16 else 2e-2, "grad of per-sample weights")


@pytest.mark.timeout(300)
@pytest.mark.parametrize("dtype,T,D,stochastic", [(torch.float32, 64, 256, False), (torch.float16, 256, 128, False),
                                                  (torch.float16, 256, 128, True)])
def test_approx_adagrad_with_a_gradient_tensor_beyond_4GiB(dtype, T, D, stochastic):
    """Below 4 GiB the wavefront-per-row kernel addresses gradient rows through a buffer descriptor with
    32-bit offsets, from 4 GiB on with 64-bit addresses.  A batch whose few non-empty bags are spread over a
    4.3 GB grad_output must come out bit for bit like the same bags packed into a small one -- fp32 rows
    (summed in chunks), fp16 rows (walked by a wavefront) and fp16 rows with stochastic rounding (the row of
    1 700 occurrences is walked by a workgroup)."""
    B, E, L = 1 << 16, 50, 8
    t_used, bags = 37, 300
    rs = np.random.RandomState(38)
    gen = torch.Generator(device=DEV).manual_seed(38)
    grad_big = torch.randn(B, T, D, device=DEV, generator=gen, dtype=dtype)
    assert grad_big.numel() * grad_big.element_size() >= 1 << 32
    chosen = np.sort(np.concatenate([rs.choice(B - 2, bags - 2, replace=False), [B - 2, B - 1]])).astype(np.int64)
    idx = rs.randint(0, E, size=(bags, L)).astype(np.int32)
    idx[rs.rand(bags, L) < 0.7] = 3
    lengths = np.zeros((T, B), np.int64)
    lengths[t_used, chosen] = L
    offsets_big = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    weights = rs.uniform(-0.01, 0.01, size=(T * E, D)).astype(np.float32 if dtype == torch.float32 else np.float16)
    table_offsets = (np.arange(T) * E).astype(np.int32)

    def run(grad, table_offsets, offsets, w):
        st = torch.zeros(w.shape[0], dtype=torch.float32, device=DEV)
        torch.manual_seed(5)  # the same random stream for both runs
        ext.backward_approx_adagrad(grad, w, dev(table_offsets), dev(idx.reshape(-1)), dev(offsets), None, st, 0.01,
                                    0.1, 200, stochastic, 1)
        torch.cuda.synchronize()
        return w.cpu().numpy(), st.cpu().numpy()

    w_big, st_big = run(grad_big, table_offsets, offsets_big, dev(weights))
    grad_small = grad_big[torch.from_numpy(chosen).to(DEV), t_used].reshape(bags, 1, D).contiguous()
    del grad_big
    rows = slice(t_used * E, (t_used + 1) * E)
    # (the whole table again, entered at the used table's first row: a row keeps its place in the
    # table, on which the random words of the stochastic rounding depend)
    w_small, st_small = run(grad_small, np.full(1, t_used * E, np.int32), (np.arange(bags + 1) * L).astype(np.int32),
                            dev(weights))
    assert st_big.tobytes() == st_small.tobytes()
    assert w_big.tobytes() == w_small.tobytes()
    assert st_big[3 + t_used * E] > 0 and np.bincount(idx.reshape(-1)).max() > 1500
    untouched = np.ones(T * E, bool)
    untouched[rows] = False
    assert w_big[untouched].tobytes() == weights[untouched].tobytes()


@pytest.mark.timeout(600)
@pytest.mark.parametrize("weighted", [False, True])
def test_full_size_approx_adagrad_against_the_fp64_closed_form(oracle, weighted):
    """The benchmark's headline shape (T=64, E=1e5, D=128 fp32, B=4096, L=20, Zipf(1.05): 5.2 M lookups,
    the hottest row of a table some 4000 times).  The serial per-lookup update has a closed form that
    torch evaluates in fp64 on the device: with the lookups of a row in position order,
        state_k = state_0 + sum_{j<=k} wss_j,   mult_k = (psw_k *) lr / (sqrt(state_k) + eps),
        row_final = row_0 - sum_k mult_k * g_k,   grad_psw_k = <row_0 - sum_{j<k} mult_j g_j, g_k>.
    State and weights of every row are compared with it; the per-sample-weight gradients, whose closed
    form is quadratic in a row's occurrences, and the first table's rows are compared with the oracle."""
    T, E, D, B, L = 64, 100000, 128, 4096, 20
    lr, eps = 0.05, 0.1
    n = T * B * L
    rs = np.random.RandomState(40)
    idx_np = (rs.zipf(1.05, size=n) % E).astype(np.int32)
    gen = torch.Generator(device=DEV).manual_seed(40)
    W = torch.empty(T * E, D, device=DEV).uniform_(-0.01, 0.01, generator=gen)
    W0 = W.clone()
    go = torch.randn(B, T, D, device=DEV, generator=gen) * 0.1
    state = torch.empty(T * E, device=DEV).uniform_(0.0, 2.0, generator=gen)
    state0 = state.clone()
    psw = torch.empty(n, device=DEV).uniform_(0.0, 1.0, generator=gen) if weighted else None
    idx = torch.from_numpy(idx_np).to(DEV)
    offsets = torch.arange(0, n + 1, L, dtype=torch.int32, device=DEV)
    table_offsets = torch.arange(T, dtype=torch.int32, device=DEV) * E
    g_psw = ext.backward_approx_adagrad(go, W, table_offsets, idx, offsets, psw, state, lr, eps, 200, False, 1)
    torch.cuda.synchronize()

    pos = torch.arange(n, device=DEV)
    t_of = pos // (B * L)
    b_of = (pos % (B * L)) // L
    key = idx.long() + t_of * E
    wss = (go.double() ** 2).sum(-1)[b_of, t_of]
    if weighted:
        wss = wss * psw.double() ** 2
    order = torch.sort(key, stable=True)[1]          # (row, position) order
    key_s, wss_s = key[order], wss[order]
    csum = torch.cumsum(wss_s, 0)
    head = torch.ones(n, dtype=torch.bool, device=DEV)
    head[1:] = key_s[1:] != key_s[:-1]
    seg_of = torch.cumsum(head.long(), 0) - 1
    before = (csum - wss_s)[head][seg_of]             # sum of the earlier rows' addends
    state_k = state0.double()[key_s] + (csum - before)
    mult = lr / (torch.sqrt(state_k) + eps)
    if weighted:
        mult = mult * psw.double()[order]
    want_state = state0.double().index_add(0, key, wss)
    assert_close(state.cpu().numpy(), want_state.cpu().numpy(), 1e-5, "state")
    delta = torch.zeros(T * E, D, dtype=torch.float64, device=DEV)
    chunk = 1 << 20
    for lo in range(0, n, chunk):                     # (pieces: the products of all lookups would take 5 GB)
        sel = order[lo:lo + chunk]
        delta.index_add_(0, key_s[lo:lo + chunk], mult[lo:lo + chunk, None] * go[b_of[sel], t_of[sel]].double())
    want_W = W0.double() - delta
    err = (W.double() - want_W).abs().max().item()
    scale = want_W.abs().max().item()
    assert err <= 1e-5 * scale, (err, scale)
    touched = torch.zeros(T * E, dtype=torch.bool, device=DEV)
    touched[key] = True
    assert torch.equal(W[~touched], W0[~touched]) and torch.equal(state[~touched], state0[~touched])
    # the first table (81 920 lookups) against the oracle, gradients of the per-sample weights included
    w_ref = W0[:E].cpu().numpy().copy()
    st_ref = state0[:E].cpu().numpy().copy()
    g_ref = oracle.backward_approx(go[:, :1, :].contiguous().cpu().numpy(), w_ref, np.zeros(1, np.int32),
                                   idx_np[:B * L], offsets[:B + 1].cpu().numpy(), lr, eps, st_ref,
                                   psw[:B * L].cpu().numpy() if weighted else None, None)
    assert_close(W[:E].cpu().numpy(), w_ref, 1e-5, "first table")
    assert_close(state[:E].cpu().numpy(), st_ref, 1e-5, "first table's state")
    if weighted:
        assert_close(g_psw[:B * L].cpu().numpy(), g_ref, 1e-4, "first table's per-sample-weight gradients")


@pytest.mark.timeout(600)
def test_full_size_weighted_fp16_approx_adagrad_properties(oracle):
    """The shape of bench.py --config 4 (T=32, E=1e6, D=64 fp16, B=8192, bag lengths uniform in [0, 40] with
    empty bags, per-sample weights, Zipf(1.2): 5.2 M lookups, the hottest row of a table some 29 000 times)
    with the approximate optimizer.  fp16 rows are rounded after every lookup, so the weights have no closed
    form; size-independent properties instead: the state of every row grows by the sum of its lookups'
    ||g||^2 * psw^2 (fp64 sum at 1e-5), rows without a lookup keep their bits, reruns are bit-identical, and the
    first table's rows, state and per-sample-weight gradients equal the oracle's serial walk."""
    T, E, D, B = 32, 1000000, 64, 8192
    lr, eps = 0.01, 0.1
    rs = np.random.RandomState(42)
    lengths = rs.randint(0, 41, size=(T, B))
    offsets_np = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    n = int(offsets_np[-1])
    idx_np = (rs.zipf(1.2, size=n) % E).astype(np.int32)
    gen = torch.Generator(device=DEV).manual_seed(42)
    W0 = torch.empty(T * E, D, device=DEV).uniform_(-0.01, 0.01, generator=gen).half()
    go = (torch.randn(B, T, D, device=DEV, generator=gen) * 0.1).half()
    state0 = torch.empty(T * E, device=DEV).uniform_(0.0, 2.0, generator=gen)
    psw = torch.empty(n, device=DEV).uniform_(0.0, 1.0, generator=gen).half()
    idx, offsets = torch.from_numpy(idx_np).to(DEV), torch.from_numpy(offsets_np).to(DEV)
    table_offsets = torch.arange(T, dtype=torch.int32, device=DEV) * E

    def run():
        W, state = W0.clone(), state0.clone()
        g = ext.backward_approx_adagrad(go, W, table_offsets, idx, offsets, psw, state, lr, eps, 200, False, 1)
        torch.cuda.synchronize()
        return W, state, g

    W, state, g_psw = run()
    W2, state2, g2 = run()
    assert torch.equal(W, W2) and torch.equal(state, state2) and torch.equal(g_psw, g2)
    bag_of = torch.repeat_interleave(torch.arange(T * B, device=DEV), torch.from_numpy(lengths.reshape(-1)).to(DEV))
    t_of, b_of = bag_of // B, bag_of % B
    key = idx.long() + t_of * E
    wss = (go.double() ** 2).sum(-1)[b_of, t_of] * psw.double() ** 2
    want_state = state0.double().index_add(0, key, wss)
    assert_close(state.cpu().numpy(), want_state.cpu().numpy(), 1e-5, "state")
    touched = torch.zeros(T * E, dtype=torch.bool, device=DEV)
    touched[key] = True
    assert torch.equal(W[~touched], W0[~touched]) and torch.equal(state[~touched], state0[~touched])
    assert int(torch.bincount(idx[:int(offsets_np[B])].long()).max()) > 20000
    # the first table against the oracle
    n0 = int(offsets_np[B])
    w_ref = W0[:E].cpu().numpy().copy()
    st_ref = state0[:E].cpu().numpy().copy()
    g_ref = oracle.backward_approx(go[:, :1, :].contiguous().cpu().numpy(), w_ref, np.zeros(1, np.int32), idx_np[:n0],
                                   offsets_np[:B + 1], lr, eps, st_ref, psw[:n0].cpu().numpy(), None)
    assert_close(state[:E].cpu().numpy(), st_ref, 1e-5, "first table's state")
    assert_close(W[:E].float().cpu().numpy(), w_ref.astype(np.float32), 1e-2, "first table")
    assert_close(g_psw[:n0].float().cpu().numpy(), g_ref.astype(np.float32), 2e-2, "first table's per-sample-weight gradients")


@pytest.mark.timeout(600)
def test_full_size_mixed_D_approx_adagrad_against_the_fp64_closed_form():
    """The mixed-D benchmark's shape (64 tables of 1e5 rows, widths 64 ... 192 in steps of 4, fp32, B=4096,
    L=20, Zipf(1.05)) against the same closed form, table by table."""
    T, E, B, L = 64, 100000, 4096, 20
    lr, eps = 0.05, 0.1
    n = T * B * L
    rs = np.random.RandomState(41)
    dims = [int((rs.randint(64, 193) + 3) // 4 * 4) for _ in range(T)]
    dim_offsets = np.concatenate([[0], np.cumsum(dims)]).astype(np.int32)
    total_D = int(dim_offsets[-1])
    table_offsets = np.concatenate([[0], np.cumsum([E * d for d in dims])]).astype(np.int64)
    table_dim_offsets = (np.arange(T + 1) * E).astype(np.int32)
    idx_np = (rs.zipf(1.05, size=n) % E).astype(np.int32)
    gen = torch.Generator(device=DEV).manual_seed(41)
    W = torch.empty(int(table_offsets[-1]), device=DEV).uniform_(-0.01, 0.01, generator=gen)
    W0 = W.clone()
    go = torch.randn(B, total_D, device=DEV, generator=gen) * 0.1
    state = torch.empty(T * E, device=DEV).uniform_(0.0, 2.0, generator=gen)
    state0 = state.clone()
    idx = torch.from_numpy(idx_np).to(DEV)
    offsets = torch.arange(0, n + 1, L, dtype=torch.int32, device=DEV)
    ext.backward_approx_adagrad_mixed_D(go, W, dev(table_offsets), dev(table_dim_offsets), dev(dim_offsets), total_D,
                                        idx, offsets, None, state, lr, eps, 200, False, 1)
    torch.cuda.synchronize()
    pos = torch.arange(B * L, device=DEV)
    b_of = pos // L
    worst = 0.0
    for t in range(T):
        g = go[:, int(dim_offsets[t]):int(dim_offsets[t + 1])].double()
        key = idx[t * B * L:(t + 1) * B * L].long()
        wss = (g ** 2).sum(-1)[b_of]
        order = torch.sort(key, stable=True)[1]
        key_s, wss_s = key[order], wss[order]
        csum = torch.cumsum(wss_s, 0)
        head = torch.ones(B * L, dtype=torch.bool, device=DEV)
        head[1:] = key_s[1:] != key_s[:-1]
        before = (csum - wss_s)[head][torch.cumsum(head.long(), 0) - 1]
        st0 = state0[t * E:(t + 1) * E].double()
        mult = lr / (torch.sqrt(st0[key_s] + (csum - before)) + eps)
        want_state = st0.index_add(0, key, wss)
        assert_close(state[t * E:(t + 1) * E].cpu().numpy(), want_state.cpu().numpy(), 1e-5, "state of table %d" % t)
        rows = slice(int(table_offsets[t]), int(table_offsets[t + 1]))
        delta = torch.zeros(E, dims[t], dtype=torch.float64, device=DEV)
        delta.index_add_(0, key_s, mult[:, None] * g[b_of[order]])
        want = W0[rows].view(E, dims[t]).double() - delta
        got = W[rows].view(E, dims[t]).double()
        worst = max(worst, ((got - want).abs().max() / want.abs().max()).item())
        untouched = torch.ones(E, dtype=torch.bool, device=DEV)
        untouched[key] = False
        assert torch.equal(W[rows].view(E, dims[t])[untouched], W0[rows].view(E, dims[t])[untouched])
    assert worst <= 1e-5, worst


def test_approx_adagrad_stochastic_rounding_of_rows_of_many_occurrences(oracle):
    """The k-th update of a hot row draws the oracle's random words in the wavefront-per-row kernel too."""
    p = make_problem(37, T=2, E=12, D=64, B=64, L=10, dtype=np.float16, ragged=False, weighted=False, zipf=1.5)
    assert np.bincount(p["indices"][:640]).max() > 130
    torch.manual_seed(99)
    gen = torch.cuda.default_generators[0]
    seed, offset = gen.initial_seed() & 0xFFFFFFFFFFFFFFFF, gen.get_offset()
    w, st, _ = _run_gpu(p, 0.05, 0.1, stochastic=True)
    w_ref, st_ref, _ = _run_oracle(oracle, p, 0.05, 0.1, stochastic_rounding=(seed, offset))
    assert_close(st, st_ref, 1e-5)
    assert (w.view(np.uint16) != w_ref.view(np.uint16)).mean() < 0.05
    assert_close(w, w_ref, 1e-2)


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("D,B", [(8, 700), (64, 700), (100, 700), (128, 700), (256, 700), (64, 64)])
def test_approx_adagrad_stochastic_rounding_bit_for_bit_with_dyadic_gradients(oracle, D, B, weighted):
    """With gradient entries in {0, +-0.5, +-1} and per-sample weights in {0.5, 1, 2} every sum of
    squares is exact in fp32 whatever its order and every product with the multiplier is exact, so
    the kernels and the oracle compute the same fp32 values and, drawing the same random words,
    must leave the same fp16 bits -- in the rows of a few occurrences, in the rows that get a
    wavefront (17 to 256 occurrences) and in the rows of more than 256 occurrences, which up to
    128 elements wide are walked by a workgroup whose other wavefronts draw the random bits
    (D = 256: a single wavefront; B = 64: one table of 512 lookups, a grid too small to set
    workgroups aside for them)."""
    rs = np.random.RandomState(D + B)
    T, E, L = (2 if B > 100 else 1), 60, 8
    p = make_problem(40, T=T, E=E, D=D, B=B, L=L, dtype=np.float16, ragged=False, weighted=weighted)
    n_t = B * L
    hot = [257, 300, 1000, 2049] if B > 100 else [300]
    mid = [17, 64, 65, 200, 256] if B > 100 else [40]
    for t in range(T):
        rows = np.concatenate([np.full(c, r, np.int32) for r, c in enumerate(hot + mid)])
        rest = rs.randint(len(hot + mid), E, size=n_t - rows.size).astype(np.int32)
        p["indices"][t * n_t:(t + 1) * n_t] = rs.permutation(np.concatenate([rows, rest]))
    p["grad_output"] = rs.choice(np.array([0, 0.5, -0.5, 1, -1], np.float16), size=p["grad_output"].shape)
    if weighted:
        p["per_sample_weights"] = rs.choice(np.array([0.5, 1, 2], np.float16), size=p["n"])
    torch.cuda.init()
    torch.manual_seed(D)
    gen = torch.cuda.default_generators[0]
    seed, offset = gen.initial_seed() & 0xFFFFFFFFFFFFFFFF, gen.get_offset()
    w, st, g = _run_gpu(p, 0.02, 0.1, stochastic=True)
    w_ref, st_ref, g_ref = _run_oracle(oracle, p, 0.02, 0.1, stochastic_rounding=(seed, offset))
    assert st.tobytes() == st_ref.tobytes()
    differing = np.flatnonzero((w.view(np.uint16) != w_ref.view(np.uint16)).any(axis=1))
    assert differing.size == 0, "rows with other bits than the oracle's: %s" % differing[:10]
    if weighted:
        assert_close(g, g_ref, 2e-2, "grad of per-sample weights")
    w_rn, _, _ = _run_gpu(p, 0.02, 0.1, stochastic=False)
    assert (w.view(np.uint16) != w_rn.view(np.uint16)).mean() > 0.05  # and it is not round-to-nearest


def _hot_row_problem(D, B, weighted, seed):
    """fp16 tables whose first rows occur 257 ... 2049 times (and others 17 ... 256 times), gradient
    entries in {0, +-0.5, +-1} and per-sample weights in {0.5, 1, 2}: every sum of squares and every
    product with a multiplier is exact in fp32 whatever its order."""
    rs = np.random.RandomState(seed)
    T, E, L = (2 if B > 100 else 1), 60, 8
    p = make_problem(43, T=T, E=E, D=D, B=B, L=L, dtype=np.float16, ragged=False, weighted=weighted)
    n_t = B * L
    hot = [257, 384, 385, 1000, 2049] if B > 100 else [300]
    mid = [17, 64, 65, 200, 256] if B > 100 else [40]
    for t in range(T):
        rows = np.concatenate([np.full(c, r, np.int32) for r, c in enumerate(hot + mid)])
        rest = rs.randint(len(hot + mid), E, size=n_t - rows.size).astype(np.int32)
        p["indices"][t * n_t:(t + 1) * n_t] = rs.permutation(np.concatenate([rows, rest]))
    p["grad_output"] = rs.choice(np.array([0, 0.5, -0.5, 1, -1], np.float16), size=p["grad_output"].shape)
    if weighted:
        p["per_sample_weights"] = rs.choice(np.array([0.5, 1, 2], np.float16), size=p["n"])
    return p, T, E, L


@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("D,B", [(8, 900), (36, 900), (64, 900), (100, 900), (128, 900), (256, 900), (64, 64), (128, 64)])
def test_approx_adagrad_fp16_rows_of_many_occurrences_staged_through_lds(oracle, D, B, weighted):
    """fp16 rows of more than 256 occurrences, up to 128 elements wide, are walked by a workgroup whose
    other wavefronts stage gradient rows and multipliers in LDS, 128 occurrences a step (D = 100, 128:
    two elements per lane, 64 occurrences a step; D = 256: a single wavefront; run lengths: one past
    a step boundary, exactly on one, one more, many; B = 64: a grid too small to set workgroups
    aside).  Checked against the kernels that do not stage: the same lookups fed in fifteen calls of
    B / 15 bags each leave every row with fewer than 257 occurrences per call, i.e. to the
    single-wavefront walk and the short-row kernel, and with exact sums (see _hot_row_problem) the
    fifteen calls must leave the state of the one call bit for bit, and bit for bit the rows that
    the single-wavefront walk takes in every call (it rounds like the staged walk).  Against the oracle:
    the state bit for bit, the rows at the fp16 tolerance (the kernels' fused multiply-add rounds
    row - mult * grad once, the oracle, like the reference, to fp32 and then to fp16, which now
    and then lands on the neighbouring value)."""
    p, T, E, L = _hot_row_problem(D, B, weighted, 3 * D + B)
    w, st, g = _run_gpu(p, 0.02, 0.1)
    w_ref, st_ref, g_ref = _run_oracle(oracle, p, 0.02, 0.1)
    assert st.tobytes() == st_ref.tobytes()
    assert_close(w, w_ref, 1e-2)
    if weighted:
        assert_close(g, g_ref, 2e-2, "grad of per-sample weights")
    if B % 15 == 0:
        calls = 15
        per = B // calls
        idx = p["indices"].reshape(T, B, L)
        psw = p["per_sample_weights"].reshape(T, B, L) if weighted else None
        w_dev = dev(p["weights"])
        st_dev = torch.zeros(w_dev.shape[0], dtype=torch.float32, device=DEV)
        fewest = np.full(T * E, 1 << 30)
        most = np.zeros(T * E, int)
        for c in range(calls):
            sub = idx[:, c * per:(c + 1) * per, :]
            counts = np.bincount((sub + np.arange(T)[:, None, None] * E).reshape(-1), minlength=T * E)
            fewest, most = np.minimum(fewest, counts), np.maximum(most, counts)
            ext.backward_approx_adagrad(
                dev(p["grad_output"][c * per:(c + 1) * per]), w_dev, dev(p["table_offsets"]),
                dev(np.ascontiguousarray(sub).reshape(-1)),
                dev(np.arange(0, T * per * L + 1, L, dtype=np.int32)),
                dev(np.ascontiguousarray(psw[:, c * per:(c + 1) * per, :]).reshape(-1)) if weighted else None,
                st_dev, 0.02, 0.1, 200, False, 1)
        torch.cuda.synchronize()
        assert st_dev.cpu().numpy().tobytes() == st.tobytes()
        # the rows that the one call stages and every one of the fifteen calls gives to the single-wavefront
        # walk (17 to 256 occurrences per call; with fewer the short-row kernel takes them, whose separate
        # conversion rounds twice like the oracle's)
        total = np.bincount((idx + np.arange(T)[:, None, None] * E).reshape(-1), minlength=T * E)
        walked = np.flatnonzero((total > 256) & (fewest >= 17) & (most <= 256))
        assert walked.size >= 2 * T
        assert (w.view(np.uint16)[walked] == w_dev.cpu().numpy().view(np.uint16)[walked]).all(), \
            "staged rows that differ from the single-wavefront walk's"
        assert_close(w, w_dev.cpu().numpy(), 1e-2)
    if not weighted:
        # per-sample weights of one change no value of the update
        ones = dict(p, per_sample_weights=np.ones(p["n"], np.float16))
        w_one, st_one, _ = _run_gpu(ones, 0.02, 0.1)
        assert st_one.tobytes() == st.tobytes()
        assert (w.view(np.uint16) == w_one.view(np.uint16)).all()


def test_approx_adagrad_stochastic_rounding_more_long_rows_than_workgroups_set_aside(oracle):
    """1100 rows of 300 occurrences each: more rows for the cooperative walk than the 1024
    workgroups (half the largest grid) that are set aside for them, so those take a second
    row each.  Dyadic gradients as above: bit for bit the oracle's result."""
    rs = np.random.RandomState(8)
    T, E, D, B, L = 1, 1100, 8, 41250, 8
    p = make_problem(41, T=T, E=E, D=D, B=B, L=L, dtype=np.float16, ragged=False, weighted=False)
    p["indices"][:] = rs.permutation(np.repeat(np.arange(E, dtype=np.int32), 300))
    p["grad_output"] = rs.choice(np.array([0, 0.5, -0.5, 1, -1], np.float16), size=p["grad_output"].shape)
    torch.cuda.init()
    torch.manual_seed(3)
    gen = torch.cuda.default_generators[0]
    seed, offset = gen.initial_seed() & 0xFFFFFFFFFFFFFFFF, gen.get_offset()
    w, st, _ = _run_gpu(p, 0.02, 0.1, stochastic=True)
    w_ref, st_ref, _ = _run_oracle(oracle, p, 0.02, 0.1, stochastic_rounding=(seed, offset))
    assert st.tobytes() == st_ref.tobytes()
    assert w.tobytes() == w_ref.tobytes()


def test_approx_adagrad_stochastic_rounding_matches_oracle_stream(oracle):
    p = make_problem(34, T=2, E=25, D=32, B=60, L=6, dtype=np.float16, weighted=False, zipf=1.2)
    torch.manual_seed(1234)
    gen = torch.cuda.default_generators[0]
    seed, offset = gen.initial_seed() & 0xFFFFFFFFFFFFFFFF, gen.get_offset()
    w, st, _ = _run_gpu(p, 0.05, 0.1, stochastic=True)
    assert gen.get_offset() == offset + 4
    w_ref, st_ref, _ = _run_oracle(oracle, p, 0.05, 0.1, stochastic_rounding=(seed, offset))
    assert_close(st, st_ref, 1e-5)
    # same random words for the k-th update of every element: the rounded rows agree except where
    # the fp32 value differs in its last bits (different summation order of ||g||^2)
    differing = (w.view(np.uint16) != w_ref.view(np.uint16)).mean()
    assert differing < 0.02, differing
    assert_close(w, w_ref, 1e-2)
    w_rn, _, _ = _run_gpu(p, 0.05, 0.1, stochastic=False)
    assert (w.view(np.uint16) != w_rn.view(np.uint16)).mean() > 0.2  # and it is not round-to-nearest


@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.float64])
@pytest.mark.parametrize("weighted", [False, True])
def test_approx_adagrad_mixed_D_matches_oracle(oracle, dtype, weighted):
    tables = [(30, 8), (7, 32), (100, 4), (16, 12), (3, 520), (40, 128)]
    p = make_mixed_problem(35, tables, B=40, L=9, dtype=dtype, weighted=weighted)
    w = dev(p["weights"])
    st_np = np.zeros(sum(r for r, _ in tables), np.float64 if dtype == np.float64 else np.float32)
    st = dev(st_np)
    g = ext.backward_approx_adagrad_mixed_D(
        dev(p["grad_output"]), w, dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"]),
        int(p["dim_offsets"][-1]), dev(p["indices"]), dev(p["offsets"]), dev(p["per_sample_weights"]), st, 0.05, 0.1,
        200, False, 1)
    w_ref = p["weights"].copy()
    g_ref = oracle.backward_approx_mixed(p["grad_output"], w_ref, p["table_offsets"], p["table_dim_offsets"],
                                         p["dim_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st_np,
                                         p["per_sample_weights"])
    tol = TOL[np.dtype(dtype)]
    assert_close(st.cpu().numpy(), st_np, 1e-5 if dtype != np.float64 else 1e-10)
    assert_close(w.cpu().numpy(), w_ref, tol)
    if weighted:
        assert_close(g.cpu().numpy(), g_ref, tol if dtype != np.float16 else 2e-2)


def test_module_with_the_approximate_optimizer_and_repeated_rows(oracle):
    """Optimizer.APPROX_ROWWISE_ADAGRAD through the module, with replacement (the reference's test
    has to draw without, test_table_batched_embeddings.py:244): two steps against the oracle."""
    T, E, D, B, L = 3, 50, 32, 40, 6
    p = make_problem(36, T, E, D, B, L, np.float32, ragged=True, weighted=True, zipf=1.2)
    cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.APPROX_ROWWISE_ADAGRAD, learning_rate=0.5,
                                       eps=0.2).cuda()
    cc.embedding_weights.data.copy_(dev(p["weights"]))
    w_ref, st_ref = p["weights"].copy(), np.zeros(T * E, np.float32)
    for _ in range(2):
        psw = dev(p["per_sample_weights"]).requires_grad_(True)
        cc(dev(p["indices"]), dev(p["offsets"]), psw).backward(dev(p["grad_output"]))
        g_ref = oracle.backward_approx(p["grad_output"], w_ref, p["table_offsets"], p["indices"], p["offsets"], 0.5,
                                       0.2, st_ref, p["per_sample_weights"])
        assert_close(psw.grad.cpu().numpy(), g_ref, 1e-5)
    assert_close(cc.optimizer_state.cpu().numpy(), st_ref, 1e-5)
    assert_close(cc.embedding_weights.detach().cpu().numpy(), w_ref, 1e-5)
    # behind the row cache the module follows the same trajectory, bit for bit
    plain = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.APPROX_ROWWISE_ADAGRAD, learning_rate=0.5,
                                          eps=0.2).cuda()
    cached = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.APPROX_ROWWISE_ADAGRAD, learning_rate=0.5,
                                           eps=0.2, managed=ops.EmbeddingLocation.HOST_CACHED, cache_slots=128,
                                           cache_stage_slots=64).cuda()
    plain.embedding_weights.data.copy_(dev(p["weights"]))
    cached.embedding_weights.data.copy_(dev(p["weights"]))
    for _ in range(3):
        psw_a = dev(p["per_sample_weights"]).requires_grad_(True)
        psw_b = dev(p["per_sample_weights"]).requires_grad_(True)
        a = plain(dev(p["indices"]), dev(p["offsets"]), psw_a)
        a.backward(dev(p["grad_output"]))
        b = cached(dev(p["indices"]), dev(p["offsets"]), psw_b)
        b.backward(dev(p["grad_output"]))
        assert torch.equal(a, b) and torch.equal(psw_a.grad, psw_b.grad)
    sd = cached.state_dict()
    torch.cuda.synchronize()
    assert torch.equal(sd["embedding_weights"], plain.embedding_weights.data)
    assert torch.equal(sd["optimizer_state"], plain.optimizer_state)


@pytest.mark.parametrize("stochastic", [False, True])
@pytest.mark.parametrize("weighted", [False, True])
def test_approx_adagrad_mixed_D_fp16_rows_of_many_occurrences(oracle, weighted, stochastic):
    """Mixed-D tables: fp16 rows of more than 256 occurrences and at most 128 elements are listed by the
    strip kernel for a workgroup's walk (staged through LDS, or with the random bits drawn by the other
    wavefronts), wider ones and rows of 9 ... 256 occurrences for a single wavefront's.  Tables of 8, 36,
    64, 100, 128 (a workgroup), 256 (a wavefront) and 520 elements (the wide rows' kernel), each with rows
    of 257 ... 2049 and of 17 ... 256 occurrences; gradients and weights chosen so that every sum is exact
    (see _hot_row_problem): the state equals the oracle's bit for bit, the rows at the fp16 tolerance --
    and, with round to nearest, a table of 64 columns comes out bit for bit as the same table does among
    uniform tables for the rows that a walk takes there as well (more than 16 occurrences)."""
    rs = np.random.RandomState(77)
    dims = [8, 36, 64, 100, 128, 256, 520]
    E, B, L = 60, 900, 8
    tables = [(E, d) for d in dims]
    T = len(tables)
    p = make_mixed_problem(44, tables, B=B, L=L, dtype=np.float16, weighted=weighted)
    hot, mid = [257, 384, 385, 1000, 2049], [17, 64, 65, 200, 256]
    n_t = B * L
    p["offsets"] = np.arange(0, T * n_t + 1, L, dtype=np.int32)
    indices = np.empty(T * n_t, np.int32)
    for t in range(T):
        rows = np.concatenate([np.full(c, r, np.int32) for r, c in enumerate(hot + mid)])
        rest = rs.randint(len(hot + mid), E, size=n_t - rows.size).astype(np.int32)
        indices[t * n_t:(t + 1) * n_t] = rs.permutation(np.concatenate([rows, rest]))
    p["indices"] = indices
    total_D = int(p["dim_offsets"][-1])
    p["grad_output"] = rs.choice(np.array([0, 0.5, -0.5, 1, -1], np.float16), size=(B, total_D))
    psw = rs.choice(np.array([0.5, 1, 2], np.float16), size=T * n_t) if weighted else None
    w = dev(p["weights"])
    st_np = np.zeros(T * E, np.float32)
    st = dev(st_np)
    g = ext.backward_approx_adagrad_mixed_D(
        dev(p["grad_output"]), w, dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"]), total_D,
        dev(p["indices"]), dev(p["offsets"]), dev(psw) if weighted else None, st, 0.02, 0.1, 200, stochastic, 1)
    w_ref = p["weights"].copy()
    g_ref = oracle.backward_approx_mixed(p["grad_output"], w_ref, p["table_offsets"], p["table_dim_offsets"],
                                         p["dim_offsets"], p["indices"], p["offsets"], 0.02, 0.1, st_np, psw)
    assert st.cpu().numpy().tobytes() == st_np.tobytes()
    got = w.cpu().numpy()
    if stochastic:
        # every update lands on one of the two fp16 neighbours of its exact value, so a row drifts from the
        # round-to-nearest trajectory like a random walk of its occurrences: unbiased, and small
        drift = got.astype(np.float64) - w_ref.astype(np.float64)
        assert np.isfinite(drift).all() and np.abs(drift).max() < 0.5 and abs(drift.mean()) < 2e-3
        assert (got.view(np.uint16) != w_ref.view(np.uint16)).mean() > 0.2   # and it is not round to nearest
        return
    assert_close(got, w_ref, 1e-2)
    if weighted:
        assert_close(g.cpu().numpy(), g_ref, 2e-2, "grad of per-sample weights")
    # the table of 64 columns alone, as a uniform table
    t = dims.index(64)
    lo, hi = int(p["table_offsets"][t]), int(p["table_offsets"][t + 1])
    c0 = int(p["dim_offsets"][t])
    w_uni = dev(p["weights"][lo:hi].reshape(E, 64))
    st_uni = torch.zeros(E, dtype=torch.float32, device=DEV)
    ext.backward_approx_adagrad(
        dev(np.ascontiguousarray(p["grad_output"][:, c0:c0 + 64]).reshape(B, 1, 64)), w_uni, dev(np.zeros(1, np.int32)),
        dev(indices[t * n_t:(t + 1) * n_t].copy()), dev(np.arange(0, n_t + 1, L, dtype=np.int32)),
        dev(psw[t * n_t:(t + 1) * n_t].copy()) if weighted else None, st_uni, 0.02, 0.1, 200, False, 1)
    torch.cuda.synchronize()
    assert st_uni.cpu().numpy().tobytes() == st_np[t * E:(t + 1) * E].tobytes()
    counts = np.bincount(indices[t * n_t:(t + 1) * n_t], minlength=E)
    walked = np.flatnonzero(counts > 16)
    assert walked.size >= 10
    mixed_rows = got[lo:hi].reshape(E, 64).view(np.uint16)
    assert (mixed_rows[walked] == w_uni.cpu().numpy().view(np.uint16)[walked]).all()


@pytest.mark.parametrize("seed", range(18))
def test_approx_adagrad_mixed_D_random_sweep(oracle, seed):
    """Seeded random mixed-D table sets for the approximate update: 1..12 tables, from one row (every
    lookup of a bag set on it: hundreds or thousands of occurrences, the workgroup walks for fp16 rows of
    up to 128 elements, the single wavefront's otherwise) to thousands, widths from 4 to more than 64
    vectors, with and without per-sample weights, all three types."""
    rs = np.random.RandomState(800 + seed)
    T = int(rs.choice([1, 2, 3, 6, 12]))
    tables = [(int(rs.choice([1, 3, 40, 600, 5000])), int(rs.choice([4, 8, 12, 20, 32, 64, 100, 128, 256, 264, 520])))
              for _ in range(T)]
    dtype = [np.float16, np.float32, np.float64][seed % 3]
    weighted = bool((seed // 3) % 2)
    B = int(rs.choice([9, 70, 400]))
    L = int(rs.choice([1, 5, 20]))
    p = make_mixed_problem(60 + seed, tables, B=B, L=L, dtype=dtype, weighted=weighted)
    w = dev(p["weights"])
    st_np = np.zeros(sum(r for r, _ in tables), np.float64 if dtype == np.float64 else np.float32)
    st = dev(st_np)
    g = ext.backward_approx_adagrad_mixed_D(
        dev(p["grad_output"]), w, dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"]),
        int(p["dim_offsets"][-1]), dev(p["indices"]), dev(p["offsets"]), dev(p["per_sample_weights"]), st, 0.05, 0.1,
        200, False, 1)
    w_ref = p["weights"].copy()
    g_ref = oracle.backward_approx_mixed(p["grad_output"], w_ref, p["table_offsets"], p["table_dim_offsets"],
                                         p["dim_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st_np,
                                         p["per_sample_weights"])
    tol = TOL[np.dtype(dtype)]
    assert_close(st.cpu().numpy(), st_np, 1e-5 if dtype != np.float64 else 1e-10)
    assert_close(w.cpu().numpy(), w_ref, tol)
    if weighted:
        assert_close(g.cpu().numpy(), g_ref, tol if dtype != np.float16 else 2e-2)
