"""Drop-in for the reference's `table_batched_embeddings` extension module.

Same ten function names and positional signatures as the pybind11 module in
table_batched_embeddings.cpp:56-70, taking torch tensors; each call validates
its tensors, then hands raw device pointers and the current HIP stream to the
C-ABI library (include/tbe_hip.h).  torch is used for device memory and streams
only -- no arithmetic happens here.
"""
import collections
import contextlib
import ctypes
import threading
import weakref

import torch

import tbe_native as _native

_DTYPE_CODES = {torch.float32: _native.DTYPE_F32, torch.float16: _native.DTYPE_F16,
                torch.float64: _native.DTYPE_F64}

# Grow-only scratch buffers for the backward pipeline (keys, sort buffers, segment lists), one per
# (device, stream) that has run a backward, the MAX_WORKSPACES most recently used ones.  The
# reference allocates these per call (table_batched_embeddings_cuda.cu:1618-1647).
MAX_WORKSPACES = 8
_workspaces = collections.OrderedDict()  # (device, stream handle) -> [uint8 tensor, lock]
_workspaces_lock = threading.Lock()
_last_workspace = {}  # device -> the one used last
# Owners of the host-resident allocations handed out by new_*_tensor (weak), keyed by device address.
_host_allocations = {}


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else ctypes.c_void_p(0)


def _stream(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _check_common(weights, table_offsets, indices, offsets):
    _require(weights.is_cuda, "weights must be a GPU tensor")
    _require(weights.dim() == 2 and weights.is_contiguous(), "weights must be a contiguous [rows, D] tensor")
    _require(weights.dtype in _DTYPE_CODES, "weights must be float16, float32 or float64")
    for name, t in (("table_offsets", table_offsets), ("indices", indices), ("offsets", offsets)):
        _require(t.dtype == torch.int32, "%s must be int32 (got %s)" % (name, t.dtype))
        _require(t.is_cuda and t.device == weights.device, "%s must live on the weights' device" % name)
        _require(t.dim() == 1 and t.is_contiguous(), "%s must be a contiguous 1-D tensor" % name)
    T = table_offsets.numel()
    _require(T > 0, "T must be positive")
    B = (offsets.numel() - 1) // T  # table_batched_embeddings_cuda.cu:266
    _require(B > 0, "B must be positive")
    _require(offsets.numel() == T * B + 1, "offsets must hold T*B+1 entries")
    return T, B


_table_rows = {}  # id(table_offsets) -> (weak reference, tensor version, total_rows, largest table)


def max_table_rows(table_offsets, total_rows):
    """Rows of the largest table, read back from `table_offsets` once per tensor (one device to
    host copy, then cached for as long as the tensor lives and is not written).  The backward
    sorts that many key bits per table instead of the bits of `total_rows`.  total_rows=None:
    `table_offsets` has T+1 entries and ends with the total."""
    ident = id(table_offsets)
    hit = _table_rows.get(ident)
    if hit is not None and hit[0]() is table_offsets and hit[1:3] == (table_offsets._version, total_rows):
        return hit[3]
    starts = table_offsets.cpu().tolist() + ([total_rows] if total_rows is not None else [])
    sizes = [b - a for a, b in zip(starts, starts[1:])]
    largest = max(sizes) if min(sizes) >= 0 and starts[0] >= 0 else 0  # 0: unknown, sort all the bits
    ref = weakref.ref(table_offsets, lambda _, ident=ident: _table_rows.pop(ident, None))
    _table_rows[ident] = (ref, table_offsets._version, total_rows, largest)
    return largest


def _rounding_stream(device):
    """(seed, offset) for one stochastically rounded backward call, taken from PyTorch's
    generator of `device` the way the reference reserves Philox offsets
    (table_batched_embeddings_cuda.cu:1685-1691); every call gets a fresh offset."""
    gen = torch.cuda.default_generators[device.index if device.index is not None else torch.cuda.current_device()]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + 4)
    return seed & 0xFFFFFFFFFFFFFFFF, offset


@contextlib.contextmanager
def _workspace(device, nbytes):
    """The grow-only scratch buffer of the device's current stream, and that stream: one buffer per
    (device, stream), so that calls issued on different streams of a device may overlap.  The
    buffer is held for the duration of the `with` block (the call that enqueues a backward's
    launches), so two host threads that drive one stream cannot interleave their launch sequences
    on one buffer.  At most MAX_WORKSPACES buffers are kept: the one least recently used goes (its
    memory returns to the allocator in the order of the stream it was allocated on, and a captured
    graph keeps the pool it was captured into)."""
    handle = torch.cuda.current_stream(device).cuda_stream
    key = (device, handle)
    with _workspaces_lock:
        entry = _workspaces.get(key)
        if entry is None:
            entry = _workspaces[key] = [None, threading.Lock()]
        _workspaces.move_to_end(key)
        while len(_workspaces) > MAX_WORKSPACES:
            _workspaces.popitem(last=False)
    with entry[1]:
        if entry[0] is None or entry[0].numel() < nbytes:
            entry[0] = torch.empty(int(nbytes * 1.25) + 256, dtype=torch.uint8, device=device)
        _last_workspace[device] = entry[0]
        yield entry[0], ctypes.c_void_p(handle)


def reserve_workspace(nbytes, device=None):
    """Sizes the scratch buffer of `device`'s current stream for backward calls that need up to
    `nbytes` (tbe_native.backward_workspace_layout(...).total_bytes), so that no later call on that
    stream allocates -- e.g. before capturing a graph on it.  An eager step run on the same stream
    has the same effect."""
    device = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    with _workspace(device, int(nbytes)):
        pass


def release_workspaces(device=None):
    """Drops the scratch buffers of `device` (all devices if None).  Work already enqueued keeps
    running on them: the allocator hands the memory out again in stream order."""
    with _workspaces_lock:
        for key in [k for k in _workspaces if device is None or k[0] == torch.device(device)]:
            del _workspaces[key]
        for dev in [d for d in _last_workspace if device is None or d == torch.device(device)]:
            del _last_workspace[dev]


def backward_workspace(device):
    """The scratch buffer last used by a backward call on `device` (for inspection)."""
    return _last_workspace.get(torch.device(device))


class BackwardPlan:
    """The index-only half of a backward pass (keys, stable sort, run boundaries), computed
    ahead of time on a side stream so that it overlaps the forward gather."""

    _side_streams = {}

    def __init__(self, weights, table_offsets, indices, offsets):
        T, B = _check_common(weights, table_offsets, indices, offsets)
        self.T, self.B, self.n = T, B, indices.numel()
        self.D = weights.size(1)
        self.code = _DTYPE_CODES[weights.dtype]
        self.total_rows = weights.size(0)
        self.device = weights.device
        layout = _native.backward_workspace_layout(self.n, self.D, self.code, T)
        # one buffer per call: it lives from the forward to the backward of the same step
        self.workspace = torch.empty(layout.total_bytes, dtype=torch.uint8, device=self.device)
        side = BackwardPlan._side_streams.get(self.device)
        if side is None:
            side = BackwardPlan._side_streams[self.device] = torch.cuda.Stream(device=self.device)
        # the buffer is written on the side stream: the allocator must not recycle it (e.g. when a
        # forward is never followed by its backward) before that stream is done with it
        self.workspace.record_stream(side)
        for t in (table_offsets, indices, offsets):
            t.record_stream(side)
        main = torch.cuda.current_stream(self.device)
        side.wait_stream(main)  # indices / offsets may still be in flight on the caller's stream
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_plan_batch(
                _ptr(table_offsets), T, _ptr(indices), self.n, _ptr(offsets), B, self.total_rows,
                max_table_rows(table_offsets, self.total_rows), self.D, self.code, _ptr(self.workspace), self.workspace.numel(), ctypes.c_void_p(side.cuda_stream)))
        self.ready = torch.cuda.Event()
        self.ready.record(side)

    def apply(self, optimizer, grad_output, weights, indice_weights, optimizer_state, learning_rate, eps,
              stochastic_rounding):
        """Gradient reduction + optimizer on the current stream, after the plan is ready."""
        grad_output = _check_grad(grad_output, weights, self.T, self.B)
        grad_indice_weights = None
        if indice_weights is not None:
            grad_indice_weights = torch.empty(self.n, dtype=grad_output.dtype, device=self.device)
        stochastic = bool(stochastic_rounding) and weights.dtype == torch.float16
        seed, offset = _rounding_stream(self.device) if stochastic else (0, 0)
        torch.cuda.current_stream(self.device).wait_event(self.ready)
        _last_workspace[self.device] = self.workspace  # keep backward_workspace() pointing at the last plan
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_backward_planned(
                optimizer, _ptr(grad_output), _ptr(weights), self.code, self.total_rows, self.D, self.T, self.B,
                self.n, _ptr(indice_weights), _ptr(optimizer_state), float(learning_rate), float(eps or 0.0),
                _ptr(grad_indice_weights), int(stochastic), seed, offset, _ptr(self.workspace),
                self.workspace.numel(), _stream(self.device)))
        return grad_indice_weights


def plan_backward(weights, table_offsets, indices, offsets):
    """Starts the index-only half of the backward on a side stream (no counterpart in the
    reference, which sorts inside its backward call, table_batched_embeddings_cuda.cu:1629-1655)."""
    return BackwardPlan(weights, table_offsets, indices, offsets)


def forward(weights, table_offsets, indices, offsets, indice_weights, L_max, BT_block_size, shmem):
    """batched_embedding_forward_cuda (table_batched_embeddings_cuda.cu:253-316).

    L_max, BT_block_size and shmem are the reference's launch knobs; results do
    not depend on them and they are ignored apart from the BT_block_size != 0 check."""
    T, B = _check_common(weights, table_offsets, indices, offsets)
    _require(BT_block_size != 0, "BT_block_size must be non-zero")
    D = weights.size(1)
    if indice_weights is not None:
        _require(indice_weights.dtype == weights.dtype, "indice_weights must have the weights' dtype")
        _require(indice_weights.is_contiguous() and indice_weights.numel() == indices.numel(),
                 "indice_weights must be contiguous with one entry per index")
        _require(indice_weights.device == weights.device, "indice_weights must live on the weights' device")
    output = torch.empty((B, T, D), dtype=weights.dtype, device=weights.device)
    with torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_forward(
            _ptr(weights), _DTYPE_CODES[weights.dtype], D, _ptr(table_offsets), T, _ptr(indices),
            indices.numel(), _ptr(offsets), B, _ptr(indice_weights), _ptr(output), _stream(weights.device)))
    return output


def _check_grad(grad_output, weights, T, B):
    _require(grad_output.dtype == weights.dtype, "grad_output must have the weights' dtype")
    _require(grad_output.device == weights.device, "grad_output must live on the weights' device")
    _require(tuple(grad_output.shape) == (B, T, weights.size(1)), "grad_output must be [B, T, D]")
    return grad_output.contiguous()


def backward_sgd(grad_output, weights, table_offsets, indices, offsets, learning_rate, L_max,
                 BT_block_size, shmem):
    """batched_embedding_backward_sgd_cuda (table_batched_embeddings_cuda.cu:383-435), made
    exact: every distinct row receives -lr * (sum of its gradients) once."""
    T, B = _check_common(weights, table_offsets, indices, offsets)
    _require(BT_block_size > 0, "BT_block_size must be positive")
    grad_output = _check_grad(grad_output, weights, T, B)
    D = weights.size(1)
    code = _DTYPE_CODES[weights.dtype]
    layout = _native.backward_workspace_layout(indices.numel(), D, code, T)
    with _workspace(weights.device, layout.total_bytes) as (ws, stream), torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_backward_sgd(
            _ptr(grad_output), _ptr(weights), code, weights.size(0),
            max_table_rows(table_offsets, weights.size(0)), D, _ptr(table_offsets), T,
            _ptr(indices), indices.numel(), _ptr(offsets), B, float(learning_rate), _ptr(ws), ws.numel(),
            stream))
    return None


def backward_exact_adagrad(grad_output, weights, table_offsets, indices, offsets, indice_weights,
                           optimizer_state, learning_rate, eps, stochastic_rounding, BT_block_size):
    """batched_embedding_backward_adagrad_exact_cuda (table_batched_embeddings_cuda.cu:1589-1706).

    Returns the gradient w.r.t. indice_weights ([N], grad_output's dtype) or None when unweighted.
    The weighted case, which the reference asserts out (:1678-1679), is served."""
    T, B = _check_common(weights, table_offsets, indices, offsets)
    _require(BT_block_size > 0, "BT_block_size must be positive")
    grad_output = _check_grad(grad_output, weights, T, B)
    D = weights.size(1)
    code = _DTYPE_CODES[weights.dtype]
    state_dtype = torch.float64 if weights.dtype == torch.float64 else torch.float32
    _require(optimizer_state.dtype == state_dtype, "optimizer_state must be %s" % state_dtype)
    _require(optimizer_state.is_contiguous() and optimizer_state.numel() == weights.size(0),
             "optimizer_state must be contiguous with one entry per row")
    _require(optimizer_state.device == weights.device, "optimizer_state must live on the weights' device")
    grad_indice_weights = None
    if indice_weights is not None:
        _require(indice_weights.dtype == weights.dtype, "indice_weights must have the weights' dtype")
        _require(indice_weights.is_contiguous() and indice_weights.numel() == indices.numel(),
                 "indice_weights must be contiguous with one entry per index")
        grad_indice_weights = torch.empty(indices.shape, dtype=grad_output.dtype, device=weights.device)
    layout = _native.backward_workspace_layout(indices.numel(), D, code, T)
    with _workspace(weights.device, layout.total_bytes) as (ws, stream), torch.cuda.device(weights.device):
        if stochastic_rounding and weights.dtype == torch.float16:
            seed, offset = _rounding_stream(weights.device)
            _native.check(_native.load().tbe_backward_exact_adagrad_stochastic(
                _ptr(grad_output), _ptr(weights), code, weights.size(0),
                max_table_rows(table_offsets, weights.size(0)), D, _ptr(table_offsets), T,
                _ptr(indices), indices.numel(), _ptr(offsets), B, _ptr(indice_weights), _ptr(optimizer_state),
                float(learning_rate), float(eps), _ptr(grad_indice_weights), seed, offset, _ptr(ws), ws.numel(),
                stream))
        else:  # rounding to nearest; stochastic rounding only exists for fp16 (tbe.cu:557-578)
            _native.check(_native.load().tbe_backward_exact_adagrad(
                _ptr(grad_output), _ptr(weights), code, weights.size(0),
                max_table_rows(table_offsets, weights.size(0)), D, _ptr(table_offsets), T,
                _ptr(indices), indices.numel(), _ptr(offsets), B, _ptr(indice_weights), _ptr(optimizer_state),
                float(learning_rate), float(eps), _ptr(grad_indice_weights), _ptr(ws), ws.numel(),
                stream))
    return grad_indice_weights


def _check_adagrad_args(grad_output, weights, table_offsets, indices, offsets, indice_weights, optimizer_state,
                        BT_block_size):
    T, B = _check_common(weights, table_offsets, indices, offsets)
    _require(BT_block_size > 0, "BT_block_size must be positive")
    grad_output = _check_grad(grad_output, weights, T, B)
    state_dtype = torch.float64 if weights.dtype == torch.float64 else torch.float32
    _require(optimizer_state.dtype == state_dtype, "optimizer_state must be %s" % state_dtype)
    _require(optimizer_state.is_contiguous() and optimizer_state.numel() == weights.size(0),
             "optimizer_state must be contiguous with one entry per row")
    _require(optimizer_state.device == weights.device, "optimizer_state must live on the weights' device")
    grad_indice_weights = None
    if indice_weights is not None:
        _require(indice_weights.dtype == weights.dtype, "indice_weights must have the weights' dtype")
        _require(indice_weights.is_contiguous() and indice_weights.numel() == indices.numel(),
                 "indice_weights must be contiguous with one entry per index")
        grad_indice_weights = torch.empty(indices.shape, dtype=grad_output.dtype, device=weights.device)
    return T, B, grad_output, grad_indice_weights


def backward_approx_adagrad(grad_output, weights, table_offsets, indices, offsets, indice_weights,
                            optimizer_state, learning_rate, eps, L_max, stochastic_rounding,
                            BT_block_size):
    """batched_embedding_backward_adagrad_approx_cuda (table_batched_embeddings_cuda.cu:706-793):
    every lookup adds its bag's ||grad||^2 (times its squared weight) to the row's state and
    moves the row by its own multiplier.  The lookups of a row are applied one at a time in
    position order, so the result equals the reference's wherever that is defined (no row twice
    in the batch) and is the serial, reproducible one where the reference races.  L_max (the
    reference's shared-memory bound on the bag length, :738) does not exist here."""
    T, B, grad_output, grad_indice_weights = _check_adagrad_args(
        grad_output, weights, table_offsets, indices, offsets, indice_weights, optimizer_state, BT_block_size)
    D = weights.size(1)
    code = _DTYPE_CODES[weights.dtype]
    layout = _native.backward_workspace_layout(indices.numel(), D, code, T)
    stochastic = bool(stochastic_rounding) and weights.dtype == torch.float16
    seed, offset = _rounding_stream(weights.device) if stochastic else (0, 0)
    with _workspace(weights.device, layout.total_bytes) as (ws, stream), torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_backward_approx_adagrad(
            _ptr(grad_output), _ptr(weights), code, weights.size(0), max_table_rows(table_offsets, weights.size(0)),
            D, _ptr(table_offsets), T, _ptr(indices), indices.numel(), _ptr(offsets), B, _ptr(indice_weights),
            _ptr(optimizer_state), float(learning_rate), float(eps), _ptr(grad_indice_weights), int(stochastic),
            seed, offset, _ptr(ws), ws.numel(), stream))
    return grad_indice_weights


def _check_mixed(weights, table_offsets, dim_offsets, indices, offsets):
    _require(weights.is_cuda and weights.dim() == 1 and weights.is_contiguous(),
             "weights must be a contiguous 1-D GPU tensor")
    _require(weights.dtype in _DTYPE_CODES, "weights must be float16, float32 or float64")
    _require(table_offsets.dtype == torch.int64, "table_offsets must be int64 (got %s)" % table_offsets.dtype)
    for name, t in (("dim_offsets", dim_offsets), ("indices", indices), ("offsets", offsets)):
        _require(t.dtype == torch.int32, "%s must be int32 (got %s)" % (name, t.dtype))
    for name, t in (("table_offsets", table_offsets), ("dim_offsets", dim_offsets), ("indices", indices),
                    ("offsets", offsets)):
        _require(t.is_cuda and t.device == weights.device, "%s must live on the weights' device" % name)
        _require(t.dim() == 1 and t.is_contiguous(), "%s must be a contiguous 1-D tensor" % name)
    T = table_offsets.numel() - 1  # table_batched_embeddings_cuda.cu:952
    _require(T > 0, "T must be positive")
    _require(dim_offsets.numel() == T + 1, "dim_offsets must hold T+1 entries")
    B = (offsets.numel() - 1) // T
    _require(B > 0, "B must be positive")
    _require(offsets.numel() == T * B + 1, "offsets must hold T*B+1 entries")
    return T, B


# fp16 rows are moved 16 bytes at a time when every table's D allows it, else 8 bytes.  The choice
# (and the one-time check that every D_t is a positive multiple of 4) needs the per-table dims on
# the host; it is cached per dim_offsets tensor, identified the way max_table_rows identifies its
# tensor: a data pointer says nothing once the allocator has recycled the block.
_fp16_width = {}  # id(dim_offsets) -> (weak reference, tensor version, vector width)


def _fp16_vector_width(dim_offsets):
    ident = id(dim_offsets)
    hit = _fp16_width.get(ident)
    if hit is not None and hit[0]() is dim_offsets and hit[1] == dim_offsets._version:
        return hit[2]
    dims = torch.diff(dim_offsets).cpu()
    _require(bool((dims % 4 == 0).all()) and bool((dims > 0).all()), "every D_t must be a positive multiple of 4")
    width = 8 if bool((dims % 8 == 0).all()) else 4
    ref = weakref.ref(dim_offsets, lambda _, ident=ident: _fp16_width.pop(ident, None))
    _fp16_width[ident] = (ref, dim_offsets._version, width)
    return width


def forward_mixed_D(weights, table_offsets, dim_offsets, total_D, indices, offsets, indice_weights, L_max,
                    BT_block_size, shmem):
    """batched_embedding_forward_mixed_D_cuda (table_batched_embeddings_cuda.cu:945-1004):
    output [B, total_D], table t in columns dim_offsets[t]:dim_offsets[t+1]."""
    T, B = _check_mixed(weights, table_offsets, dim_offsets, indices, offsets)
    _require(BT_block_size != 0, "BT_block_size must be non-zero")
    if indice_weights is not None:
        _require(indice_weights.dtype == weights.dtype and indice_weights.is_contiguous()
                 and indice_weights.numel() == indices.numel(),
                 "indice_weights must be contiguous, of the weights' dtype, with one entry per index")
    output = torch.empty((B, int(total_D)), dtype=weights.dtype, device=weights.device)
    with torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_forward_mixed(
            _ptr(weights), _DTYPE_CODES[weights.dtype], _fp16_vector_width(dim_offsets), _ptr(table_offsets),
            _ptr(dim_offsets), int(total_D), T, _ptr(indices), indices.numel(), _ptr(offsets), B,
            _ptr(indice_weights), _ptr(output), _stream(weights.device)))
    return output


def _backward_mixed(optimizer, grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, total_D, indices,
                    offsets, indice_weights, optimizer_state, learning_rate, eps, stochastic_rounding):
    T, B = _check_mixed(weights, table_offsets, dim_offsets, indices, offsets)
    _require(table_dim_offsets.dtype == torch.int32 and table_dim_offsets.numel() == T + 1,
             "table_dim_offsets must be int32 with T+1 entries")
    _require(grad_output.dtype == weights.dtype and tuple(grad_output.shape) == (B, int(total_D)),
             "grad_output must be [B, total_D] of the weights' dtype")
    grad_output = grad_output.contiguous()
    code = _DTYPE_CODES[weights.dtype]
    total_rows = optimizer_state.numel()  # table_batched_embeddings_cuda.cu:1404
    grad_indice_weights = None
    if indice_weights is not None:
        _require(indice_weights.dtype == weights.dtype and indice_weights.is_contiguous()
                 and indice_weights.numel() == indices.numel(),
                 "indice_weights must be contiguous, of the weights' dtype, with one entry per index")
        grad_indice_weights = torch.empty(indices.shape, dtype=grad_output.dtype, device=weights.device)
    state_dtype = torch.float64 if weights.dtype == torch.float64 else torch.float32
    _require(optimizer_state.dtype == state_dtype and optimizer_state.is_contiguous(),
             "optimizer_state must be contiguous %s" % state_dtype)
    layout = _native.backward_mixed_workspace_layout(indices.numel(), code, T)
    stochastic = bool(stochastic_rounding) and weights.dtype == torch.float16
    seed, offset = _rounding_stream(weights.device) if stochastic else (0, 0)
    with _workspace(weights.device, layout.total_bytes) as (ws, stream), torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_backward_mixed(
            optimizer, _ptr(grad_output), _ptr(weights), code, _fp16_vector_width(dim_offsets), total_rows,
            max_table_rows(table_dim_offsets, None), _ptr(table_offsets), _ptr(table_dim_offsets), _ptr(dim_offsets), int(total_D), T, _ptr(indices),
            indices.numel(), _ptr(offsets), B, _ptr(indice_weights), _ptr(optimizer_state), float(learning_rate),
            float(eps or 0.0), _ptr(grad_indice_weights), int(stochastic), seed, offset, _ptr(ws), ws.numel(),
            stream))
    return grad_indice_weights


def backward_exact_adagrad_mixed_D(grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, total_D,
                                   indices, offsets, indice_weights, optimizer_state, learning_rate, eps,
                                   stochastic_rounding, BT_block_size):
    """batched_embedding_backward_adagrad_exact_mixed_D_cuda (table_batched_embeddings_cuda.cu:1350-1469)."""
    _require(BT_block_size > 0, "BT_block_size must be positive")
    return _backward_mixed(_native.OPT_ROWWISE_ADAGRAD, grad_output, weights, table_offsets, table_dim_offsets,
                           dim_offsets, total_D, indices, offsets, indice_weights, optimizer_state, learning_rate,
                           eps, stochastic_rounding)


def backward_approx_adagrad_mixed_D(grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, total_D,
                                    indices, offsets, indice_weights, optimizer_state, learning_rate, eps, L_max,
                                    stochastic_rounding, BT_block_size):
    """batched_embedding_backward_adagrad_approx_mixed_D_cuda (table_batched_embeddings_cuda.cu:1076-1163,
    table_batched_embeddings.cpp:38-43): the per-lookup update of backward_approx_adagrad for
    tables with per-table dimension."""
    _require(BT_block_size > 0, "BT_block_size must be positive")
    return _backward_mixed(_native.OPT_APPROX_ROWWISE_ADAGRAD, grad_output, weights, table_offsets, table_dim_offsets,
                           dim_offsets, total_D, indices, offsets, indice_weights, optimizer_state, learning_rate,
                           eps, stochastic_rounding)


def backward_sgd_mixed_D(grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, total_D, indices,
                         offsets, optimizer_state, learning_rate):
    """Exact SGD for mixed-dimension tables (no counterpart in the reference, whose mixed module
    only accepts the Adagrad optimizers, table_batched_embeddings_ops.py:269)."""
    return _backward_mixed(_native.OPT_SGD, grad_output, weights, table_offsets, table_dim_offsets, dim_offsets,
                           total_D, indices, offsets, None, optimizer_state, learning_rate, 0.0, False)


def construct_offsets(batch_offsets_per_table, total_indices_per_table):
    """construct_offsets (table_batched_embeddings_cuda.cu:1190-1213): [T,B] bag starts and [T]
    totals -> int32 [1+T*B] bag lengths with a leading zero; the caller cumsums."""
    _require(batch_offsets_per_table.is_cuda, "batch_offsets_per_table must be a GPU tensor")
    _require(batch_offsets_per_table.dim() == 2, "batch_offsets_per_table must be [T, B]")
    _require(batch_offsets_per_table.dtype == torch.int32 and total_indices_per_table.dtype == torch.int32,
             "construct_offsets takes int32 tensors")
    _require(total_indices_per_table.device == batch_offsets_per_table.device,
             "both arguments must live on one device")
    T, B = batch_offsets_per_table.shape
    _require(total_indices_per_table.numel() == T, "total_indices_per_table must be [T]")
    per_table = batch_offsets_per_table.contiguous()
    totals = total_indices_per_table.contiguous()
    output = torch.empty(1 + T * B, dtype=torch.int32, device=per_table.device)
    with torch.cuda.device(per_table.device):
        _native.check(_native.load().tbe_construct_offsets(
            _ptr(per_table), _ptr(totals), T, B, _ptr(output), _stream(per_table.device)))
    return output


class _HostAllocation:
    """Owner of one host-resident allocation, exposed to torch through __cuda_array_interface__.

    torch.as_tensor keeps a reference to the exporting object inside the tensor's storage and drops
    it when the last tensor (or view, or Parameter) on that storage dies, so releasing the memory
    here ties it to the storage's lifetime -- the role of the deleters that the reference attaches
    to its DataPtrs (CUDAManagedDeleter / CUDAHostMappedDeleter,
    table_batched_embeddings_cuda.cu:795-835).  free_host_tensor() releases it early."""

    def __init__(self, device_ptr, numel, typestr, device, release):
        self.__cuda_array_interface__ = {"shape": (int(numel),), "typestr": typestr, "data": (device_ptr, False),
                                         "version": 2, "strides": None}
        self.device_ptr = device_ptr
        self._device = device
        self._release = release

    def release(self):
        """Frees the allocation once (kernels that still use it are waited for); returns the
        library's return code, or None when it was released before."""
        release, self._release = self._release, None
        if release is None:
            return None
        _host_allocations.pop(self.device_ptr, None)
        try:
            torch.cuda.synchronize(self._device)
        except Exception:  # interpreter shutdown: the runtime may be gone already
            pass
        code = release()
        for callback in list(release_observers):
            callback(self.device_ptr)
        return code

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


# Called with the device address of every host allocation that is released (tests observe this).
release_observers = []

_TYPESTR = {torch.float32: "<f4", torch.float16: "<f2", torch.float64: "<f8"}


def _wrap_host_memory(self, sizes, device_ptr, release):
    numel = 1
    for s in sizes:
        numel *= int(s)
    owner = _HostAllocation(device_ptr, numel, _TYPESTR[self.dtype], self.device, release)
    tensor = torch.as_tensor(owner, device=self.device).view(*[int(s) for s in sizes])
    # weak: the storage holds the only strong reference, so dropping the tensor frees the memory
    _host_allocations[device_ptr] = weakref.ref(owner)
    return tensor


def new_managed_tensor(self, sizes):
    """new_managed_tensor (table_batched_embeddings_cuda.cu:864-871): a tensor tagged with
    `self`'s device and dtype whose pages are managed memory preferring the host.  The memory is
    released when the tensor's storage dies, as the reference's CUDAManagedDeleter does (:795)."""
    _require(self.is_cuda and self.dtype in _TYPESTR, "prototype must be a floating GPU tensor")
    nbytes = self.element_size()
    for s in sizes:
        _require(int(s) >= 0, "sizes must not be negative")
        nbytes *= int(s)
    nbytes = max(nbytes, 1)  # an empty tensor still owns an allocation, as in the compiled binding
    lib = _native.load()
    ptr = ctypes.c_void_p()
    with torch.cuda.device(self.device):
        _native.check(lib.tbe_managed_alloc(nbytes, self.device.index or 0, ctypes.byref(ptr)))
    address = ptr.value
    return _wrap_host_memory(self, sizes, address, lambda: lib.tbe_managed_free(ctypes.c_void_p(address)))


def new_host_mapped_tensor(self, sizes):
    """new_host_mapped_tensor (table_batched_embeddings_cuda.cu:873-880): pinned host memory
    mapped into the device's address space, tagged as a tensor on `self`'s device; released when
    the tensor's storage dies (CUDAHostMappedDeleter, :812-818).  Unlike the reference (:823) the
    pages are not write-combined: the host reads this table (checkpoints, state_dict, the CPU
    side of tests), and reads of write-combined memory bypass the CPU caches; the GPU's accesses
    over the link are the same either way."""
    _require(self.is_cuda and self.dtype in _TYPESTR, "prototype must be a floating GPU tensor")
    nbytes = self.element_size()
    for s in sizes:
        _require(int(s) >= 0, "sizes must not be negative")
        nbytes *= int(s)
    nbytes = max(nbytes, 1)  # an empty tensor still owns an allocation, as in the compiled binding
    lib = _native.load()
    host, dev = ctypes.c_void_p(), ctypes.c_void_p()
    with torch.cuda.device(self.device):
        _native.check(lib.tbe_host_mapped_alloc(nbytes, ctypes.byref(host), ctypes.byref(dev)))
    host_address = host.value
    return _wrap_host_memory(self, sizes, dev.value,
                             lambda: lib.tbe_host_mapped_free(ctypes.c_void_p(host_address)))


def free_host_tensor(tensor):
    """Releases the storage behind a tensor made by new_managed_tensor / new_host_mapped_tensor
    right away instead of when its storage dies.  The tensor (and every view of it) must not be
    used afterwards."""
    ref = _host_allocations.get(tensor.data_ptr())
    owner = ref() if ref is not None else None
    _require(owner is not None, "tensor was not allocated by this module")
    _native.check(owner.release() or 0)
