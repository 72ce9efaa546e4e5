"""The forward and the fused backward inside a HIP graph.

The entry points launch kernels on the caller's stream and do nothing else there (no
allocation, no host synchronisation, no memset nodes), so a step can be captured once and
replayed with new indices, weights and gradients copied into the captured buffers.  Every replay
is compared bit for bit with the same step run eagerly, with eager work and synchronisations
between the replays.  The number of lookups is part of the captured launch configuration: the
batches of one graph differ in indices, bag lengths and values, not in their total length."""
import numpy as np
import pytest
import torch

import table_batched_embeddings as ext
from gpu_util import DEV, dev

pytestmark = pytest.mark.gpu


def _batch(rs, T, E, B, n):
    """Ragged bags with exactly n lookups in total, Zipf-skewed rows (some rows repeat often)."""
    cuts = np.sort(rs.randint(0, n + 1, size=T * B - 1))
    offsets = np.concatenate([[0], cuts, [n]]).astype(np.int32)
    indices = (rs.zipf(1.3, size=n) % E).astype(np.int32)
    return indices, offsets


@pytest.mark.parametrize("mode,dtype,D", [("sgd", torch.float32, 128), ("adagrad_weighted", torch.float16, 64),
                                          ("approx", torch.float32, 32), ("sgd", torch.float64, 12)])
def test_captured_step_replays_like_eager(mode, dtype, D):
    T, E, B, n = 5, 400, 64, 3000
    rs = np.random.RandomState(2)
    gen = torch.Generator(device=DEV).manual_seed(4)
    table_offsets = dev((np.arange(T) * E).astype(np.int32))
    weighted = mode.endswith("weighted")
    st_dtype = torch.float64 if dtype == torch.float64 else torch.float32
    lr, eps = 0.05, 0.1

    def step(w, st, idx, off, go, psw):
        out = ext.forward(w, table_offsets, idx, off, psw, 200, 1, False)
        if mode == "sgd":
            ext.backward_sgd(go, w, table_offsets, idx, off, lr, 200, 1, False)
            return out, None
        if mode == "approx":
            return out, ext.backward_approx_adagrad(go, w, table_offsets, idx, off, psw, st, lr, eps, 200, False, 1)
        return out, ext.backward_exact_adagrad(go, w, table_offsets, idx, off, psw, st, lr, eps, False, 1)

    def draw():
        indices, offsets = _batch(rs, T, E, B, n)
        go = torch.randn(B, T, D, device=DEV, generator=gen, dtype=torch.float32).to(dtype)
        psw = torch.rand(n, device=DEV, generator=gen, dtype=torch.float32).to(dtype) if weighted else None
        return dev(indices), dev(offsets), go, psw

    # the captured buffers
    w = (torch.rand(T * E, D, device=DEV, generator=gen, dtype=torch.float32) * 0.2 - 0.1).to(dtype)
    st = torch.zeros(T * E, device=DEV, dtype=st_dtype)
    idx, off, go, psw = draw()
    # eager twins
    w_eager, st_eager = w.clone(), st.clone()

    # Warm-up outside the capture, on the stream the capture will use: the scratch buffer belongs
    # to the (device, stream) pair, so this is what sizes the buffer the captured launches get, and
    # it fills the host-side caches.  The capture itself then allocates no scratch.
    capture_stream = torch.cuda.Stream()
    capture_stream.wait_stream(torch.cuda.current_stream())
    warm_w, warm_st = w.clone(), st.clone()
    with torch.cuda.stream(capture_stream):
        step(warm_w, warm_st, idx, off, go, psw)
    torch.cuda.synchronize()
    scratch = ext.backward_workspace(torch.device(DEV))

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=capture_stream):
        out_graph, g_graph = step(w, st, idx, off, go, psw)
    assert ext.backward_workspace(torch.device(DEV)) is scratch, "the capture allocated a scratch buffer of its own"
    # the capture itself runs nothing: w and st are still the start values
    assert torch.equal(w, w_eager)

    for replay in range(5):
        if replay:
            new_idx, new_off, new_go, new_psw = draw()
            idx.copy_(new_idx)
            off.copy_(new_off)
            go.copy_(new_go)
            if weighted:
                psw.copy_(new_psw)
        graph.replay()
        out_eager, g_eager = step(w_eager, st_eager, idx.clone(), off.clone(), go.clone(),
                                  None if psw is None else psw.clone())
        torch.cuda.synchronize()
        assert torch.equal(out_graph, out_eager), "forward output differs at replay %d" % replay
        assert torch.equal(w, w_eager), "weights differ at replay %d" % replay
        assert torch.equal(st, st_eager), "optimizer state differs at replay %d" % replay
        if g_eager is not None:
            assert torch.equal(g_graph, g_eager), "per-sample-weight gradient differs at replay %d" % replay
        # unrelated eager work between replays (other kernels, another workspace user)
        other = ext.forward(w_eager, table_offsets, idx, off, psw, 200, 1, False)
        assert torch.equal(other, ext.forward(w, table_offsets, idx, off, psw, 200, 1, False))
