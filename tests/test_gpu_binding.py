"""The pybind11 module (table_batched_embeddings_cpp, the C++ counterpart of the reference's
table_batched_embeddings.cpp over the C ABI) against the Python module that binds the same
entry points: same arguments, same results bit for bit, same errors."""
import numpy as np
import pytest
import torch

from conftest import make_problem
from gpu_util import DEV, assert_close, dev

import table_batched_embeddings as ext
import tbe_native
import table_batched_embeddings_cpp as ext_cpp

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,D,weighted", [(np.float32, 128, False), (np.float16, 64, True), (np.float64, 12, True)])
def test_cpp_module_equals_python_module(oracle, dtype, D, weighted):
    p = make_problem(51, T=4, E=300, D=D, B=40, L=9, dtype=dtype, weighted=weighted, zipf=1.2)
    to, idx, off = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    psw = dev(p["per_sample_weights"])
    go = dev(p["grad_output"])
    st_dtype = torch.float64 if dtype == np.float64 else torch.float32

    out_py = ext.forward(dev(p["weights"]), to, idx, off, psw, 200, 1, False)
    out_cpp = ext_cpp.forward(dev(p["weights"]), to, idx, off, psw, 200, 1, False)
    assert torch.equal(out_py, out_cpp)
    assert_close(out_cpp.cpu().numpy(), oracle.forward(p["weights"], p["table_offsets"], p["indices"], p["offsets"],
                                                       p["per_sample_weights"]),
                 {np.float32: 1e-5, np.float16: 2e-3, np.float64: 1e-12}[dtype])

    if not weighted:
        w_py, w_cpp = dev(p["weights"]), dev(p["weights"])
        assert ext_cpp.backward_sgd(go, w_cpp, to, idx, off, 0.05, 200, 1, False) is None
        ext.backward_sgd(go, w_py, to, idx, off, 0.05, 200, 1, False)
        assert torch.equal(w_py, w_cpp)

    for fn in ("backward_exact_adagrad", "backward_approx_adagrad"):
        w_py, w_cpp = dev(p["weights"]), dev(p["weights"])
        s_py = torch.zeros(w_py.shape[0], device=DEV, dtype=st_dtype)
        s_cpp = torch.zeros_like(s_py)
        tail = (0.05, 0.1, False, 1) if fn == "backward_exact_adagrad" else (0.05, 0.1, 200, False, 1)
        g_py = getattr(ext, fn)(go, w_py, to, idx, off, psw, s_py, *tail)
        g_cpp = getattr(ext_cpp, fn)(go, w_cpp, to, idx, off, psw, s_cpp, *tail)
        assert torch.equal(w_py, w_cpp) and torch.equal(s_py, s_cpp), fn
        assert (g_py is None) == (g_cpp is None) == (not weighted)
        if weighted:
            assert torch.equal(g_py, g_cpp)


def test_cpp_module_stochastic_rounding_uses_the_generator_like_the_python_module():
    p = make_problem(52, T=2, E=50, D=32, B=30, L=6, dtype=np.float16, zipf=1.2)
    to, idx, off, go = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]), dev(p["grad_output"])
    results = []
    for module in (ext, ext_cpp):
        torch.manual_seed(77)
        gen = torch.cuda.default_generators[0]
        before = gen.get_offset()
        w = dev(p["weights"])
        st = torch.zeros(w.shape[0], device=DEV)
        module.backward_exact_adagrad(go, w, to, idx, off, None, st, 0.05, 0.1, True, 1)
        module.backward_approx_adagrad(go, w, to, idx, off, None, st, 0.05, 0.1, 200, True, 1)
        assert gen.get_offset() == before + 8
        results.append((w, st))
    assert torch.equal(results[0][0], results[1][0]) and torch.equal(results[0][1], results[1][1])


def test_cpp_module_construct_offsets_and_errors():
    rs = np.random.RandomState(5)
    T, B = 3, 7
    lengths = rs.randint(0, 5, size=(T, B)).astype(np.int32)
    starts = np.concatenate([np.zeros((T, 1), np.int32), np.cumsum(lengths, axis=1)[:, :-1]], axis=1).astype(np.int32)
    totals = lengths.sum(axis=1).astype(np.int32)
    got = ext_cpp.construct_offsets(dev(starts), dev(totals))
    assert torch.equal(got, ext.construct_offsets(dev(starts), dev(totals)))
    w = torch.zeros(8, 6, device=DEV)  # D not a multiple of 4
    i32 = torch.zeros(2, dtype=torch.int32, device=DEV)
    with pytest.raises(RuntimeError, match="multiple of 4"):
        ext_cpp.forward(w, i32[:1], i32[:1], i32, None, 200, 1, False)
    with pytest.raises(RuntimeError, match="BT_block_size"):
        ext_cpp.backward_sgd(torch.zeros(1, 1, 8, device=DEV), torch.zeros(8, 8, device=DEV), i32[:1], i32[:1], i32,
                             0.1, 200, 0, False)


@pytest.mark.parametrize("dtype,weighted", [(np.float32, False), (np.float16, True)])
def test_cpp_module_mixed_dimension_functions(dtype, weighted):
    from conftest import make_mixed_problem
    tables = [(30, 8), (7, 32), (100, 4), (900, 260), (16, 12)]
    p = make_mixed_problem(9, tables, B=21, L=9, dtype=dtype, weighted=weighted)
    to, tdo, do = dev(p["table_offsets"]), dev(p["table_dim_offsets"]), dev(p["dim_offsets"])
    idx, off, psw, go = dev(p["indices"]), dev(p["offsets"]), dev(p["per_sample_weights"]), dev(p["grad_output"])
    total_D = int(p["dim_offsets"][-1])
    out_py = ext.forward_mixed_D(dev(p["weights"]), to, do, total_D, idx, off, psw, 200, 1, False)
    out_cpp = ext_cpp.forward_mixed_D(dev(p["weights"]), to, do, total_D, idx, off, psw, 200, 1, False)
    assert torch.equal(out_py, out_cpp)
    for fn in ("backward_exact_adagrad_mixed_D", "backward_approx_adagrad_mixed_D"):
        w_py, w_cpp = dev(p["weights"]), dev(p["weights"])
        s_py = torch.zeros(sum(p["rows"]), device=DEV)
        s_cpp = torch.zeros_like(s_py)
        tail = (0.05, 0.1, False, 1) if "exact" in fn else (0.05, 0.1, 200, False, 1)
        g_py = getattr(ext, fn)(go, w_py, to, tdo, do, total_D, idx, off, psw, s_py, *tail)
        g_cpp = getattr(ext_cpp, fn)(go, w_cpp, to, tdo, do, total_D, idx, off, psw, s_cpp, *tail)
        assert torch.equal(w_py, w_cpp) and torch.equal(s_py, s_cpp), fn
        if weighted:
            assert torch.equal(g_py, g_cpp)
        else:
            assert g_py is None and g_cpp is None


@pytest.mark.parametrize("maker", ["new_host_mapped_tensor", "new_managed_tensor"])
def test_cpp_module_host_tensors(maker):
    """Tensors over host memory made by the compiled module behave like device tensors: torch ops
    and the kernels read and update them; the memory goes with the storage (the reference's
    deleters, table_batched_embeddings_cuda.cu:795-835)."""
    p = make_problem(53, T=2, E=60, D=16, B=12, L=5, dtype=np.float32)
    proto = torch.empty(1, device=DEV)
    w_host = getattr(ext_cpp, maker)(proto, [2 * 60, 16])
    assert w_host.is_cuda and w_host.dtype == torch.float32 and tuple(w_host.shape) == (120, 16)
    w_host.copy_(dev(p["weights"]))
    w_dev = dev(p["weights"])
    to, idx, off, go = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]), dev(p["grad_output"])
    assert torch.equal(ext_cpp.forward(w_host, to, idx, off, None, 200, 1, False),
                       ext_cpp.forward(w_dev, to, idx, off, None, 200, 1, False))
    ext_cpp.backward_sgd(go, w_host, to, idx, off, 0.1, 200, 1, False)
    ext_cpp.backward_sgd(go, w_dev, to, idx, off, 0.1, 200, 1, False)
    torch.cuda.synchronize()
    assert torch.equal(w_host, w_dev)
    view = w_host[3:5]
    del w_host          # the view keeps the storage, and with it the memory, alive
    torch.cuda.synchronize()
    assert torch.equal(view, w_dev[3:5])
    del view
    torch.cuda.synchronize()


@pytest.mark.parametrize("optimizer,fp16,weighted,managed", [("SGD", False, False, "DEVICE"),
                                                             ("EXACT_ROWWISE_ADAGRAD", True, True, "DEVICE"),
                                                             ("APPROX_ROWWISE_ADAGRAD", False, False, "HOST_MAPPED")])
def test_module_over_the_compiled_extension(optimizer, fp16, weighted, managed):
    """table_batched_embeddings_ops.py over the compiled module -- the reference's own layering
    (Python module -> pybind11 extension -> kernels): the same training trajectory, bit for bit,
    as over the Python binding."""
    import table_batched_embeddings_ops as ops
    T, E, D, B, L = 3, 200, 32, 24, 6
    rs = np.random.RandomState(14)
    results = []
    for module in (ext, ext_cpp):
        previous = ops.use_extension(module)
        try:
            torch.manual_seed(21)
            cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=getattr(ops.Optimizer, optimizer), learning_rate=0.05,
                                               eps=0.1, fp16=fp16, managed=getattr(ops.EmbeddingLocation, managed)).cuda()
            steps = np.random.RandomState(15)
            for _ in range(3):
                indices = dev((steps.zipf(1.3, size=T * B * L) % E).astype(np.int32))
                offsets = dev(np.arange(0, T * B * L + 1, L, dtype=np.int32))
                psw = None
                if weighted:
                    psw = dev(steps.rand(T * B * L).astype(np.float16 if fp16 else np.float32)).requires_grad_()
                out = cc(indices, offsets, psw)
                out.backward(dev(steps.randn(B, T, D).astype(np.float16 if fp16 else np.float32)))
            torch.cuda.synchronize()
            results.append((cc.embedding_weights.detach().clone(), cc.optimizer_state.clone(),
                            None if psw is None else psw.grad.clone()))
        finally:
            ops.use_extension(previous)
    assert torch.equal(results[0][0], results[1][0])
    assert torch.equal(results[0][1], results[1][1])
    if weighted:
        assert torch.equal(results[0][2], results[1][2])


@pytest.mark.parametrize("module", [ext, ext_cpp], ids=["python", "cpp"])
def test_backward_calls_on_two_streams_do_not_share_scratch(module):
    """Each stream of a device has its own workspace, so two backward calls issued on two streams
    without any ordering between them give what they give one after the other."""
    problems = [make_problem(61, T=8, E=5000, D=64, B=512, L=20, dtype=np.float32, zipf=1.1),
                make_problem(62, T=6, E=3000, D=64, B=700, L=15, dtype=np.float32, zipf=1.3)]
    args, expect = [], []
    for p in problems:
        to, idx, off, go = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]), dev(p["grad_output"])
        args.append((go, to, idx, off))
        w = dev(p["weights"])
        module.backward_sgd(go, w, to, idx, off, 0.05, 200, 1, False)
        expect.append(w)
    torch.cuda.synchronize()
    for _ in range(3):
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        weights = [dev(p["weights"]) for p in problems]
        torch.cuda.synchronize()
        for s, w, (go, to, idx, off) in zip(streams, weights, args):
            with torch.cuda.stream(s):
                module.backward_sgd(go, w, to, idx, off, 0.05, 200, 1, False)
        torch.cuda.synchronize()
        for w, want in zip(weights, expect):
            assert torch.equal(w, want)


@pytest.mark.parametrize("module", [ext, ext_cpp], ids=["python", "cpp"])
@pytest.mark.parametrize("maker", ["new_host_mapped_tensor", "new_managed_tensor"])
def test_host_tensors_of_zero_size(module, maker):
    """Both bindings give an empty tensor for an empty size (it still owns a one-byte allocation)."""
    proto = torch.empty(1, device=DEV, dtype=torch.float16)
    for sizes in ([0, 16], [0]):
        t = getattr(module, maker)(proto, sizes)
        assert t.is_cuda and t.dtype == torch.float16 and list(t.shape) == sizes and t.numel() == 0
        del t
    torch.cuda.synchronize()


@pytest.mark.parametrize("module", [ext, ext_cpp], ids=["python", "cpp"])
def test_workspaces_are_bounded_and_can_be_released(module):
    """Every stream that runs a backward gets a scratch buffer; only the most recently used ones
    are kept, and release_workspaces() drops them all.  Results do not depend on any of it."""
    p = make_problem(71, T=4, E=800, D=32, B=64, L=8, dtype=np.float32, zipf=1.2)
    to, idx, off, go = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]), dev(p["grad_output"])
    want = dev(p["weights"])
    module.backward_sgd(go, want, to, idx, off, 0.05, 200, 1, False)
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream() for _ in range(12)]
    for s in streams:
        w = dev(p["weights"])
        torch.cuda.synchronize()
        with torch.cuda.stream(s):
            module.backward_sgd(go, w, to, idx, off, 0.05, 200, 1, False)
        torch.cuda.synchronize()
        assert torch.equal(w, want)
    if module is ext:
        assert len(ext._workspaces) <= ext.MAX_WORKSPACES
    module.release_workspaces()
    if module is ext:
        assert len(ext._workspaces) == 0 and ext.backward_workspace(torch.device(DEV)) is None
    lay = tbe_native.backward_workspace_layout(p["n"], p["D"], tbe_native.DTYPE_F32, p["T"])
    if module is ext:
        ext.reserve_workspace(lay.total_bytes, DEV)
        held = ext.backward_workspace(torch.device(DEV))
        assert held is not None and held.numel() >= lay.total_bytes
    else:
        ext_cpp.reserve_workspace(want, lay.total_bytes)
    w = dev(p["weights"])
    module.backward_sgd(go, w, to, idx, off, 0.05, 200, 1, False)
    torch.cuda.synchronize()
    assert torch.equal(w, want)
    if module is ext:
        assert ext.backward_workspace(torch.device(DEV)) is held  # the reserved buffer served the call


@pytest.mark.parametrize("module", [ext, ext_cpp], ids=["python", "cpp"])
def test_two_host_threads_on_one_stream_do_not_interleave(module):
    """Two host threads issue backward calls on the same (default) stream: a call holds the stream's
    scratch buffer until its launches are enqueued, so each update is what it is alone."""
    import threading

    problems = [make_problem(81, T=8, E=4000, D=64, B=256, L=20, dtype=np.float32, zipf=1.1),
                make_problem(82, T=5, E=2500, D=64, B=300, L=12, dtype=np.float32, zipf=1.3)]
    args, expect = [], []
    for p in problems:
        to, idx, off, go = dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]), dev(p["grad_output"])
        w = dev(p["weights"])
        for _ in range(4):
            module.backward_sgd(go, w, to, idx, off, 0.05, 200, 1, False)
        args.append((go, to, idx, off))
        expect.append(w)
    torch.cuda.synchronize()
    weights = [dev(p["weights"]) for p in problems]
    errors = []

    def worker(w, a):
        try:
            torch.cuda.set_device(0)
            for _ in range(4):
                module.backward_sgd(a[0], w, a[1], a[2], a[3], 0.05, 200, 1, False)
        except Exception as e:  # surfaced below: an assertion inside a thread is lost otherwise
            errors.append(e)

    threads = [threading.Thread(target=worker, args=(w, a)) for w, a in zip(weights, args)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    assert not errors, errors
    for w, want in zip(weights, expect):
        assert torch.equal(w, want)
