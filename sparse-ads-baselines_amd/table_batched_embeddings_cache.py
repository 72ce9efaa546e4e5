"""Host side of the HBM row cache that fronts a host-resident embedding table.

`RowCache` owns the cache state in device memory (tags, recency / frequency words, the
cached rows), two scratch workspaces and a side stream, and drives the C-ABI cache entry
points of include/tbe_hip.h.  The reference has no cache: its HOST_MAPPED location reads
every row over the bus (table_batched_embeddings_ops.py:159-167).
"""
import ctypes

import torch

import tbe_native as _native
from table_batched_embeddings import max_table_rows as _max_table_rows

_DTYPE_CODES = {torch.float32: _native.DTYPE_F32, torch.float16: _native.DTYPE_F16,
                torch.float64: _native.DTYPE_F64}
_POLICIES = {"lru": _native.CACHE_LRU, "lfu": _native.CACHE_LFU}
STAT_NAMES = ("unique_rows", "hits", "misses", "inserted", "written_back", "uncached", "staged", "from_staging")


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None and t.numel() > 0 else 0)


class RowCache:
    def __init__(self, backing_weights, cache_slots, policy="lru", stage_slots=0, deferred_write_back=True):
        """backing_weights: [rows, D] tensor whose storage is device-visible host memory
        (table_batched_embeddings.new_host_mapped_tensor) -- or plain device memory, which is
        useful for tests.  cache_slots is rounded down to a multiple of 64 (one set).
        stage_slots: rows of HBM that hold, for one step, the rows no slot could take (every way
        of their set already serves the step): they then cross the host link once per step and
        direction instead of once per lookup.  Sized for the misses of a step it stages them all.
        deferred_write_back (with a staging area): staged rows go back to the table during the NEXT
        prepare(), beside its fetches, so that both directions of the host link work at once; a row
        that the next batch needs again is taken from its staging row and not written back at all.
        This takes a second staging area and four bytes per row of the table in HBM."""
        if policy not in _POLICIES:
            raise ValueError("cache policy must be 'lru' or 'lfu'")
        if not backing_weights.is_cuda or backing_weights.dim() != 2 or not backing_weights.is_contiguous():
            raise RuntimeError("backing_weights must be a contiguous [rows, D] GPU-visible tensor")
        self.device = backing_weights.device
        self.backing = backing_weights
        self.D = backing_weights.size(1)
        self.dtype_code = _DTYPE_CODES[backing_weights.dtype]
        self.num_sets = int(cache_slots) // _native.CACHE_WAYS
        if self.num_sets < 1:
            raise ValueError("cache_slots must be at least %d" % _native.CACHE_WAYS)
        slots = self.num_sets * _native.CACHE_WAYS
        self.tags = torch.empty(slots, dtype=torch.int32, device=self.device)
        self.last_used = torch.empty(slots, dtype=torch.int32, device=self.device)
        self.use_count = torch.empty(slots, dtype=torch.int32, device=self.device)
        self.stage_slots = int(stage_slots)
        if self.stage_slots < 0:
            raise ValueError("stage_slots must not be negative")
        self.deferred_write_back = bool(deferred_write_back) and self.stage_slots > 0
        areas = 2 if self.deferred_write_back else 1
        self.rows = torch.empty(slots + areas * self.stage_slots, self.D, dtype=backing_weights.dtype,
                                device=self.device)
        self.stage_of_row = self.stage_keys = None
        if self.deferred_write_back:
            self.stage_of_row = torch.empty(backing_weights.size(0), dtype=torch.int32, device=self.device)
            self.stage_keys = torch.empty(2 * self.stage_slots, dtype=torch.int32, device=self.device)
        self.handle = _native.Cache(_ptr(self.tags), _ptr(self.last_used), _ptr(self.use_count), _ptr(self.rows),
                                    _ptr(self.backing), self.num_sets, _POLICIES[policy], self.stage_slots,
                                    _ptr(self.stage_of_row), _ptr(self.stage_keys), backing_weights.size(0))
        self.side_stream = torch.cuda.Stream(device=self.device)  # default priority
        self.step = 0
        # prepare() leaves ONE plan (sort, slots of this batch's rows) in the workspaces; plan_id
        # names it, so that a backward can tell whether the plan is still the one of its forward
        self.plan_id = 0
        self._plan_ws = None
        self._cache_ws = None
        self._layout = None
        self._plan_layout = None
        self._n = 0
        self._planned_backward_done = True  # nothing is planned yet
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_cache_init(ctypes.byref(self.handle), self._stream()))

    def _stream(self):
        return ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def _grow(self, current, nbytes):
        if current is None or current.numel() < nbytes:
            return torch.empty(int(nbytes * 1.25) + 256, dtype=torch.uint8, device=self.device)
        return current

    def _view(self, ws, offset, count):
        return ws[offset:offset + 4 * count].view(torch.int32)

    def prepare(self, table_offsets, indices, offsets):
        """Sorts the batch, probes / fills the cache for its unique rows and builds the
        per-lookup slot table.  Must precede forward() and backward() of the same batch."""
        T = table_offsets.numel()
        B = (offsets.numel() - 1) // T
        n = indices.numel()
        self.step += 1
        self.plan_id += 1
        self._n, self._T, self._B = n, T, B
        self._planned_backward_done = False
        self._plan_layout = _native.backward_workspace_layout(n, self.D, self.dtype_code, T)
        self._layout = _native.cache_workspace_layout(n, self.num_sets)
        self._plan_ws = self._grow(self._plan_ws, self._plan_layout.total_bytes)
        self._cache_ws = self._grow(self._cache_ws, self._layout.total_bytes)
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_cache_prepare(
                ctypes.byref(self.handle), self.dtype_code, self.backing.size(0),
                _max_table_rows(table_offsets, self.backing.size(0)), self.D, _ptr(table_offsets), T,
                _ptr(indices), n, _ptr(offsets), B, self.step, _ptr(self._plan_ws), self._plan_ws.numel(),
                _ptr(self._cache_ws), self._cache_ws.numel(), self._stream(),
                ctypes.c_void_p(self.side_stream.cuda_stream)))

    @property
    def lookup_slots(self):
        return self._view(self._cache_ws, self._layout.lookup_slots, self._n)

    def unique_slots(self):
        U = int(self._view(self._plan_ws, self._plan_layout.num_unique, 1)[0])
        return self._view(self._cache_ws, self._layout.unique_slots, U)

    def unique_keys(self):
        U = int(self._view(self._plan_ws, self._plan_layout.num_unique, 1)[0])
        starts = self._view(self._plan_ws, self._plan_layout.segment_starts, U).long()
        return self._view(self._plan_ws, self._plan_layout.keys_sorted, self._n)[starts]

    def evicted_keys(self):
        U = int(self._view(self._plan_ws, self._plan_layout.num_unique, 1)[0])
        return self._view(self._cache_ws, self._layout.evicted_keys, U)

    def stats(self):
        """Counters of the last prepare() (synchronises)."""
        values = self._view(self._cache_ws, self._layout.stats, 8).tolist()
        return dict(zip(STAT_NAMES, values))

    def forward(self, table_offsets, indices, offsets, per_sample_weights=None):
        T, B = self._T, self._B
        output = torch.empty((B, T, self.D), dtype=self.backing.dtype, device=self.device)
        slots = self.lookup_slots if self._n else None
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_forward_cached(
                ctypes.byref(self.handle), self.dtype_code, self.D, _ptr(table_offsets), T, _ptr(indices), self._n,
                _ptr(offsets), B, _ptr(per_sample_weights), _ptr(slots), _ptr(output), self._stream()))
        return output

    def backward(self, optimizer, grad_output, per_sample_weights, optimizer_state, learning_rate, eps,
                 stochastic_rounding=None, plan_id=None):
        """optimizer: 'sgd' or 'adagrad'.  Updates rows where they live; returns the gradient
        w.r.t. per_sample_weights or None.  stochastic_rounding: None, or the (seed, offset) of
        the random stream that rounds updated fp16 weights (Adagrad only).  plan_id: the value of
        self.plan_id after the prepare() of the batch this gradient belongs to; a later prepare()
        has replaced that batch's plan and slots (and may have evicted its rows), so the call is
        refused instead of applying the gradient to another batch's rows."""
        if plan_id is not None and plan_id != self.plan_id:
            raise RuntimeError(
                "the row cache was prepared for another batch since this batch's forward (plan %d, now %d): "
                "a cache-fronted module holds one planned batch at a time -- run each forward's backward "
                "before the next forward" % (plan_id, self.plan_id))
        if self._planned_backward_done:
            raise RuntimeError("this batch's backward has already run; its plan serves one update")
        if (grad_output.dtype != self.backing.dtype or grad_output.device != self.device
                or tuple(grad_output.shape) != (self._B, self._T, self.D)):
            raise RuntimeError("grad_output must be [B=%d, T=%d, D=%d] of %s on %s (got %s of %s)"
                               % (self._B, self._T, self.D, self.backing.dtype, self.device,
                                  tuple(grad_output.shape), grad_output.dtype))
        self._planned_backward_done = True
        grad_output = grad_output.contiguous()
        grad_psw = None
        if per_sample_weights is not None:
            grad_psw = torch.empty(self._n, dtype=grad_output.dtype, device=self.device)
        code = _native.OPT_SGD if optimizer == "sgd" else _native.OPT_ROWWISE_ADAGRAD
        unique = self._view(self._cache_ws, self._layout.unique_slots, max(self._n, 1))
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_backward_cached(
                code, _ptr(grad_output), ctypes.byref(self.handle), self.dtype_code, self.backing.size(0), self.D,
                self._T, self._B, self._n, _ptr(per_sample_weights),
                _ptr(optimizer_state) if optimizer != "sgd" else ctypes.c_void_p(0), float(learning_rate),
                float(eps or 0.0), _ptr(grad_psw), int(stochastic_rounding is not None),
                stochastic_rounding[0] if stochastic_rounding else 0,
                stochastic_rounding[1] if stochastic_rounding else 0, _ptr(self._plan_ws), self._plan_ws.numel(),
                _ptr(unique), self._stream()))
        return grad_psw

    def flush(self):
        """Writes every resident row (and every staged row whose write-back is still pending) back to
        the backing table."""
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_cache_flush(ctypes.byref(self.handle), self.dtype_code, self.D,
                                                         self._stream()))

    def invalidate(self, write_back=True):
        """Empties the cache (tags, recency and frequency words back to their initial values), after
        writing the resident rows back to the backing table unless write_back is False.  Needed
        whenever the backing table is written behind the cache's back (loading a checkpoint,
        assigning to the weights): a resident row would otherwise keep serving, and later write
        back, its old value.  Any planned batch is dropped."""
        if write_back:
            self.flush()
        self.plan_id += 1
        self._planned_backward_done = True
        self._n = 0
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_cache_init(ctypes.byref(self.handle), self._stream()))

    def resident_keys(self):
        """Sorted keys of the rows currently held (synchronises)."""
        return torch.sort(self.tags[self.tags >= 0])[0]
