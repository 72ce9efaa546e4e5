"""The static-scratch backward (tbe_backward_sgd_static) against tbe_backward_sgd, through the C ABI.

Both run the same kernels, one on a caller's workspace and one on the array the library holds, so
weights and every integer stage must come out bit for bit the same -- on two calls in a row, the
second with a smaller batch (the array still holds the first call's contents then)."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import make_problem

import tbe_native

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


def _run_both(p, lr):
    lib = tbe_native.load()
    T, B, D, n = p["T"], p["B"], p["D"], p["n"]
    code = tbe_native.DTYPE_F32 if p["weights"].dtype == np.float32 else tbe_native.DTYPE_F16
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    go, toff, idx, off = dev(p["grad_output"]), dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    w_ws, w_static = dev(p["weights"]), dev(p["weights"])
    total_rows, largest = int(sum(p["rows"])), int(max(p["rows"]))
    lay = tbe_native.backward_workspace_layout(n, D, code, T)
    assert lay.total_bytes <= tbe_native.STATIC_SCRATCH_BYTES
    ws = torch.empty(lay.total_bytes, dtype=torch.uint8, device=DEV)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    print("static-scratch backward: T=%d B=%d D=%d n=%d dtype=%s" % (T, B, D, n, p["weights"].dtype), flush=True)
    tbe_native.check(lib.tbe_backward_sgd(_p(go), _p(w_ws), code, total_rows, largest, D, _p(toff), T, _p(idx), n,
                                          _p(off), B, lr, _p(ws), ws.numel(), stream))
    tbe_native.check(lib.tbe_backward_sgd_static(_p(go), _p(w_static), code, total_rows, largest, D, _p(toff), T,
                                                 _p(idx), n, _p(off), B, lr, stream))
    torch.cuda.synchronize()
    assert torch.equal(w_ws, w_static), "weights differ between the workspace and the static-scratch call"
    assert not torch.equal(w_ws, dev(p["weights"])), "the update changed nothing"
    return w_static.cpu().numpy()


def test_static_scratch_backward_equals_workspace_backward(oracle):
    big = make_problem(5, T=5, E=3000, D=64, B=700, L=40, dtype=np.float32, zipf=1.1)
    small = make_problem(6, T=3, E=500, D=64, B=90, L=12, dtype=np.float32, zipf=1.3)
    assert small["n"] < big["n"]
    for p in (big, small):  # the second call finds the first one's leftovers in the array
        got = _run_both(p, 0.05)
        want = p["weights"].copy()
        oracle.backward("sgd", p["grad_output"], want, p["table_offsets"], p["indices"], p["offsets"], 0.05)
        scale = np.abs(want).max()
        np.testing.assert_allclose(got, want, rtol=1e-5, atol=1e-5 * scale)


def test_static_scratch_backward_allocates_nothing():
    """The property the entry point is named for: once the first call on the device has resolved the
    array's address, a call neither takes device memory (free memory as the driver reports it is
    unchanged, and so is what torch's allocator has reserved) nor does anything a stream capture
    forbids -- the same call inside a capture region returns 0 and the captured graph, replayed,
    gives the update of the eager call."""
    p = make_problem(8, T=4, E=1500, D=64, B=256, L=16, dtype=np.float32, zipf=1.2)
    lib = tbe_native.load()
    code = tbe_native.DTYPE_F32
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    go, toff, idx, off = dev(p["grad_output"]), dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    T, D, B, n = p["T"], p["D"], p["B"], p["n"]
    total_rows, largest = int(sum(p["rows"])), int(max(p["rows"]))

    def call(w, stream):
        return lib.tbe_backward_sgd_static(_p(go), _p(w), code, total_rows, largest, D, _p(toff), T, _p(idx), n,
                                           _p(off), B, 0.05, ctypes.c_void_p(stream.cuda_stream))

    w_eager, w_graph = dev(p["weights"]), dev(p["weights"])
    warm = dev(p["weights"])
    assert call(warm, torch.cuda.current_stream()) == 0  # resolves the symbol on this device
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    reserved_before = torch.cuda.memory_reserved()
    assert call(w_eager, torch.cuda.current_stream()) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before, "the call took device memory"
    assert torch.cuda.memory_reserved() == reserved_before
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        rc = call(w_graph, torch.cuda.current_stream())
    assert rc == 0, lib.tbe_last_error()
    assert torch.equal(w_graph, dev(p["weights"])), "capturing must not run the update"
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(w_graph, w_eager)
    # (free memory is not compared again here: entering torch.cuda.graph collects garbage and empties
    # torch's cache, and the graph object itself may hold memory)


def test_static_scratch_backward_fp16_and_empty_batch():
    p = make_problem(7, T=4, E=2000, D=32, B=300, L=20, dtype=np.float16, zipf=1.2)
    _run_both(p, 0.01)
    lib = tbe_native.load()
    w = torch.ones(8, 4, device=DEV)
    z = torch.zeros(3, dtype=torch.int32, device=DEV)
    go = torch.ones(2, 1, 4, device=DEV)
    rc = lib.tbe_backward_sgd_static(_p(go), _p(w), tbe_native.DTYPE_F32, 8, 8, 4, _p(z), 1, ctypes.c_void_p(0), 0,
                                     _p(z), 2, 0.1, ctypes.c_void_p(0))
    assert rc == 0
    torch.cuda.synchronize()
    assert bool((w == 1).all())


def test_static_scratch_backward_rejects_a_batch_beyond_its_array():
    lib = tbe_native.load()
    n = 4 << 20
    assert tbe_native.backward_workspace_layout(n, 128, tbe_native.DTYPE_F32, 64).total_bytes > \
        tbe_native.STATIC_SCRATCH_BYTES
    one = ctypes.c_void_p(256)  # never dereferenced: the size check comes first
    rc = lib.tbe_backward_sgd_static(one, one, tbe_native.DTYPE_F32, 6400000, 100000, 128, one, 64, one, n, one, 4096,
                                     0.01, ctypes.c_void_p(0))
    assert rc == 2
    assert b"bytes of scratch" in lib.tbe_last_error()
