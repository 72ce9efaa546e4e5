"""Helpers shared by the GPU parity tests: move a numpy problem to the device, run the
HIP path through the extension-module mirror (which calls the C ABI), bring results back."""
import numpy as np
import torch

import table_batched_embeddings as ext
import tbe_native

DEV = "cuda:0"
TORCH_DTYPES = {np.dtype(np.float32): torch.float32, np.dtype(np.float16): torch.float16,
                np.dtype(np.float64): torch.float64}
CODES = {np.dtype(np.float32): tbe_native.DTYPE_F32, np.dtype(np.float16): tbe_native.DTYPE_F16,
         np.dtype(np.float64): tbe_native.DTYPE_F64}


def dev(a):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def gpu_forward(p, weighted=None):
    psw = p.get("per_sample_weights") if weighted is None or weighted else None
    out = ext.forward(dev(p["weights"]), dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]), dev(psw),
                      200, 1, False)
    return out.cpu().numpy()


def workspace_views(n, D, dtype, T):
    """Sorted keys, sorted positions and segment starts left in the workspace by the last backward."""
    lay = tbe_native.backward_workspace_layout(n, D, CODES[np.dtype(dtype)], T)
    ws = ext.backward_workspace(DEV if isinstance(DEV, torch.device) else torch.device(DEV))

    def view(off, count):
        return ws[off:off + 4 * count].view(torch.int32).cpu().numpy()

    U = int(view(lay.num_unique, 1)[0])
    return dict(keys_sorted=view(lay.keys_sorted, n),
                positions_sorted=view(lay.positions_sorted, n), segment_starts=view(lay.segment_starts, U + 1),
                num_unique=U, counters=view(lay.num_unique, 320))


def gpu_backward(p, optimizer, lr, eps=0.0, state=None):
    """Runs the fused backward in place on copies; returns dict(weights, state, grad_psw, views)."""
    w = dev(p["weights"])
    go = dev(p["grad_output"])
    psw = dev(p.get("per_sample_weights"))
    args = (dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"]))
    st = None
    gpsw = None
    if optimizer == "sgd":
        assert psw is None
        ext.backward_sgd(go, w, *args, lr, 200, 1, False)
    else:
        st_dtype = torch.float64 if w.dtype == torch.float64 else torch.float32
        st = torch.zeros(w.shape[0], dtype=st_dtype, device=DEV) if state is None else dev(state)
        gpsw = ext.backward_exact_adagrad(go, w, *args, psw, st, lr, eps, False, 1)
    torch.cuda.synchronize()
    views = workspace_views(p["n"], p["D"], p["weights"].dtype, p["T"]) if p["n"] else None
    return dict(weights=w.cpu().numpy(), state=None if st is None else st.cpu().numpy(),
                grad_psw=None if gpsw is None else gpsw.cpu().numpy(), views=views)


def assert_close(got, want, tol, what=""):
    """|got - want| <= tol * (|want| + scale).  For arrays of rows (two or more dimensions) `scale` is
    the largest magnitude of the element's own row (last axis), so a small element is held to `tol`
    of its row and not of some other, larger row of the array; elements of a row may cancel to
    near zero, which is why the row is the floor.  For vectors (one value per row or lookup) the
    floor is the vector's largest magnitude."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, "%s: shape %s, expected %s" % (what, got.shape, want.shape)
    if want.size == 0:
        return
    if want.ndim >= 2:
        scale = np.abs(want).max(axis=-1, keepdims=True)
    else:
        scale = np.abs(want).max()
    err = np.abs(got - want)
    bound = tol * (np.abs(want) + scale)
    bad = ~(err <= bound)  # also catches NaN
    if bad.any():
        worst = np.unravel_index(np.argmax(np.where(bad, err / np.maximum(bound, 1e-300), 0.0)), want.shape)
        raise AssertionError("%s: %d of %d elements differ by more than %g of (|element| + row scale); worst at %s: "
                             "got %r, expected %r" % (what, int(bad.sum()), want.size, tol, worst, got[worst],
                                                      want[worst]))
