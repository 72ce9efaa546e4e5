"""Host side of the HBM row cache that fronts a host-resident embedding table.

`RowCache` owns the cache state in device memory (tags, recency / frequency words, the
cached rows and staging areas), the workspaces of two planned batches and two side streams, and
drives the C-ABI cache entry points of include/tbe_hip.h.  The reference has no cache: its
HOST_MAPPED location reads every row over the bus (table_batched_embeddings_ops.py:159-167).

A batch goes through three calls: prepare() (sort the batch, decide slots, move rows), forward(),
backward().  With deferred write-back, prefetch() does the first part of prepare() for the NEXT
batch ahead of time, on the side streams, while the current batch computes:

    cache.prefetch(to, indices[0], offsets[0])
    for i in range(steps):
        if i + 1 < steps:
            cache.prefetch(to, indices[i + 1], offsets[i + 1])   # before this step's forward
        cache.prepare(to, indices[i], offsets[i])                # takes the prefetched plan
        out = cache.forward(to, indices[i], offsets[i])
        cache.backward("sgd", grad, None, None, lr, 0.0)

All calls of one cache are expected from one host thread with one current stream.
"""
import ctypes

import torch

import tbe_native as _native
from table_batched_embeddings import max_table_rows as _max_table_rows
from table_batched_embeddings import _fp16_vector_width

_DTYPE_CODES = {torch.float32: _native.DTYPE_F32, torch.float16: _native.DTYPE_F16,
                torch.float64: _native.DTYPE_F64}
_POLICIES = {"lru": _native.CACHE_LRU, "lfu": _native.CACHE_LFU}
STAT_NAMES = ("unique_rows", "hits", "misses", "inserted", "written_back", "uncached", "staged", "from_staging",
              "written_out", "late_fetches", "no_landing_row")
STAGE_AREAS = 3  # deferred write-back: staging areas that take turns by the plan's sequence number


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr() if t is not None and t.numel() > 0 else 0)


class _Plan:
    """One planned batch: where its workspaces are and how far it has got."""

    PREFETCHED, COMMITTED, FORWARDED, DONE, REPLACED = range(5)

    def __init__(self, **kw):
        self.__dict__.update(kw)


class MixedTables:
    """Tables of different widths behind one cache (the layout of MixedDimTableBatchedEmbeddingBags,
    table_batched_embeddings_ops.py:324-379): table_offsets int64 [T+1] (first element of each table in
    the 1-D weights), table_dim_offsets int32 [T+1] (first global row id of each table), dim_offsets
    int32 [T+1] (first output column of each table), all on the weights' device."""

    def __init__(self, table_offsets, table_dim_offsets, dim_offsets):
        self.table_offsets = table_offsets
        self.table_dim_offsets = table_dim_offsets
        self.dim_offsets = dim_offsets
        self.T = dim_offsets.numel() - 1
        dims = dim_offsets.cpu().tolist()
        self.total_D = dims[-1]
        self.widest = max(b - a for a, b in zip(dims, dims[1:]))
        self.total_rows = int(table_dim_offsets[-1])
        # what prepare() / prefetch() / forward() take as `table_offsets`: the first row of each table
        self.table_rows = table_dim_offsets[:self.T]
        self.vector_width = _fp16_vector_width(dim_offsets)


class RowCache:
    def __init__(self, backing_weights, cache_slots, policy="lru", stage_slots=0, deferred_write_back=True,
                 mixed=None):
        """backing_weights: [rows, D] tensor whose storage is device-visible host memory
        (table_batched_embeddings.new_host_mapped_tensor) -- or plain device memory, which is
        useful for tests.  With tables of different widths (mixed: a MixedTables) it is their 1-D
        weights; a cache row then has the widest table's width, of which a narrower row uses the
        front.
        cache_slots is rounded down to a multiple of 64 (one set).
        stage_slots: rows of HBM that hold, for one step, the rows no slot could take (every way
        of their set already serves the step): they then cross the host link once per step and
        direction instead of once per lookup.  Sized for the misses of a step it stages them all.
        deferred_write_back (with a staging area): staged and evicted rows stay in the staging area
        after the update and go back to the table two steps later, beside that step's fetches, so
        that both directions of the host link work at once; a row that a later batch needs again is
        taken from its staging row and not written back at all.  Row traffic then never waits for a
        step's kernels, which is what lets prefetch() overlap it with them.  This takes three
        staging areas and four bytes per row of the table in HBM."""
        if policy not in _POLICIES:
            raise ValueError("cache policy must be 'lru' or 'lfu'")
        self.mixed = mixed
        if mixed is None:
            if not backing_weights.is_cuda or backing_weights.dim() != 2 or not backing_weights.is_contiguous():
                raise RuntimeError("backing_weights must be a contiguous [rows, D] GPU-visible tensor")
            self.D = backing_weights.size(1)
            self.total_rows = backing_weights.size(0)
        else:
            if not backing_weights.is_cuda or backing_weights.dim() != 1 or not backing_weights.is_contiguous():
                raise RuntimeError("backing_weights of tables of different widths must be a contiguous 1-D "
                                   "GPU-visible tensor")
            self.D = mixed.widest
            self.total_rows = mixed.total_rows
        self.device = backing_weights.device
        self.backing = backing_weights
        self.dtype_code = _DTYPE_CODES[backing_weights.dtype]
        self.num_sets = int(cache_slots) // _native.CACHE_WAYS
        if self.num_sets < 1:
            raise ValueError("cache_slots must be at least %d" % _native.CACHE_WAYS)
        slots = self.num_sets * _native.CACHE_WAYS
        self.num_slots = slots
        self.tags = torch.empty(slots, dtype=torch.int32, device=self.device)
        self.last_used = torch.empty(slots, dtype=torch.int32, device=self.device)
        self.use_count = torch.empty(slots, dtype=torch.int32, device=self.device)
        self.stage_slots = int(stage_slots)
        if self.stage_slots < 0:
            raise ValueError("stage_slots must not be negative")
        self.deferred_write_back = bool(deferred_write_back) and self.stage_slots > 0
        areas = STAGE_AREAS if self.deferred_write_back else 1
        self.rows = torch.empty(slots + areas * self.stage_slots, self.D, dtype=backing_weights.dtype,
                                device=self.device)
        self.stage_of_row = self.stage_keys = None
        if self.deferred_write_back:
            self.stage_of_row = torch.empty(self.total_rows, dtype=torch.int32, device=self.device)
            self.stage_keys = torch.empty(STAGE_AREAS * self.stage_slots, dtype=torch.int32, device=self.device)
        self.handle = _native.Cache(_ptr(self.tags), _ptr(self.last_used), _ptr(self.use_count), _ptr(self.rows),
                                    _ptr(self.backing), self.num_sets, _POLICIES[policy], self.stage_slots,
                                    _ptr(self.stage_of_row), _ptr(self.stage_keys), self.total_rows)
        if mixed is not None:
            self.handle.mixed_table_offsets = _ptr(mixed.table_offsets)
            self.handle.mixed_table_rows = _ptr(mixed.table_dim_offsets)
            self.handle.mixed_dim_offsets = _ptr(mixed.dim_offsets)
            self.handle.mixed_T = mixed.T
        # default priority, both: the link stream carries the row traffic over the host link, the
        # plan stream the decisions of a prefetched batch
        self.link_stream = torch.cuda.Stream(device=self.device)
        self.plan_stream = torch.cuda.Stream(device=self.device)
        self.side_stream = self.link_stream
        self.step = 0        # stamps the recency words; only has to grow
        self.sequence = 0    # consecutive number of the planned batches; picks the staging area
        self._next_plan_id = 0
        # Two planned batches can exist at a time: the one that forward / backward work on and the
        # one prefetched behind it; their workspaces alternate by the sequence number.
        self._ws = [None, None]
        self._cws = [None, None]
        self._slots = [None, None]
        self._queue = []       # prefetched plans that no prepare() has taken yet
        self._current = None   # the plan of the last prepare()
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_cache_init(ctypes.byref(self.handle), self._stream()))

    # ------------------------------------------------------------------ helpers
    def _stream(self):
        return ctypes.c_void_p(torch.cuda.current_stream(self.device).cuda_stream)

    def _grow(self, current, nbytes):
        if current is None or current.numel() < nbytes:
            return torch.empty(int(nbytes * 1.25) + 256, dtype=torch.uint8, device=self.device)
        return current

    @staticmethod
    def _view(ws, offset, count):
        return ws[offset:offset + 4 * count].view(torch.int32)

    @property
    def plan_id(self):
        """Names the batch that forward() and backward() currently work on (-1: none)."""
        return self._current.plan_id if self._current is not None else -1

    def _require_current(self):
        if self._current is None:
            raise RuntimeError("no batch is prepared: call prepare() first")
        return self._current

    # ----------------------------------------------------------------- planning
    def _plan(self, table_offsets, indices, offsets, ahead):
        T = table_offsets.numel()
        B = (offsets.numel() - 1) // T
        n = indices.numel()
        if self.mixed is not None and T != self.mixed.T:
            raise RuntimeError("table_offsets must be the first row of each of the cache's %d tables "
                               "(MixedTables.table_rows)" % self.mixed.T)
        which = (self.sequence + 1) % 2
        old = self._slots[which]
        if old is not None and old.state in (_Plan.PREFETCHED, _Plan.COMMITTED):
            raise RuntimeError("two batches are already prefetched and waiting for their forward; "
                               "run the forward of the first before prefetching another")
        if old is not None and old.state == _Plan.FORWARDED:
            old.state = _Plan.REPLACED  # its workspaces are taken over: a late backward must not use them
        self.step += 1
        self.sequence += 1
        self._next_plan_id += 1
        if self.mixed is not None:
            plan_layout = _native.backward_mixed_workspace_layout(n, self.dtype_code, T)
        else:
            plan_layout = _native.backward_workspace_layout(n, self.D, self.dtype_code, T)
        layout = _native.cache_workspace_layout(n, self.num_sets, self.stage_slots)
        self._ws[which] = self._grow(self._ws[which], plan_layout.total_bytes)
        self._cws[which] = self._grow(self._cws[which], layout.total_bytes)
        plan = _Plan(plan_id=self._next_plan_id, sequence=self.sequence, step=self.step, n=n, T=T, B=B,
                     plan_layout=plan_layout, layout=layout, ws=self._ws[which], cws=self._cws[which],
                     table_offsets=table_offsets, indices=indices, offsets=offsets, fill_done=None,
                     state=_Plan.PREFETCHED)
        self._slots[which] = plan
        lib = _native.load()
        args = (ctypes.byref(self.handle), self.dtype_code, self.total_rows,
                _max_table_rows(table_offsets, self.total_rows), self.D, _ptr(table_offsets), T, _ptr(indices), n,
                _ptr(offsets), B, plan.step, plan.sequence, _ptr(plan.ws), plan.ws.numel(), _ptr(plan.cws),
                plan.cws.numel())
        with torch.cuda.device(self.device):
            if not self.deferred_write_back:
                _native.check(lib.tbe_cache_prepare(*args, self._stream(),
                                                    ctypes.c_void_p(self.link_stream.cuda_stream)))
                plan.state = _Plan.COMMITTED
                return plan
            current = torch.cuda.current_stream(self.device)
            if ahead:
                # behind everything issued so far: the previous plan, the commit of the batch two back
                # and the last kernels that read this plan's workspaces
                self.plan_stream.wait_stream(current)
                decisions = self.plan_stream
            else:
                decisions = current
            _native.check(lib.tbe_cache_plan(*args, ctypes.c_void_p(decisions.cuda_stream),
                                             ctypes.c_void_p(self.link_stream.cuda_stream)))
            plan.fill_done = torch.cuda.Event()
            plan.fill_done.record(self.link_stream)
        return plan

    def _commit(self, plan):
        """The part of a plan that has to follow the update of the batch before it."""
        if plan.state != _Plan.PREFETCHED:
            return
        with torch.cuda.device(self.device):
            torch.cuda.current_stream(self.device).wait_event(plan.fill_done)
            _native.check(_native.load().tbe_cache_commit(
                ctypes.byref(self.handle), self.dtype_code, self.D, plan.T, plan.n, plan.sequence, _ptr(plan.ws),
                plan.ws.numel(), _ptr(plan.cws), plan.cws.numel(), self._stream()))
        plan.state = _Plan.COMMITTED

    def prefetch(self, table_offsets, indices, offsets):
        """Plans a batch ahead of its prepare(): sorts it, decides its slots and starts moving its
        rows over the host link, on side streams, while the kernels of the batch before it run.  The
        batches must then be prepared in the order they were prefetched.  Call it before the
        forward of the current batch for the most overlap.  The three tensors must stay unchanged
        until the batch's prepare()."""
        if not self.deferred_write_back:
            raise RuntimeError("prefetch needs deferred write-back: a cache with a staging area "
                               "(stage_slots > 0, deferred_write_back=True)")
        self._queue.append(self._plan(table_offsets, indices, offsets, ahead=True))

    def prepare(self, table_offsets, indices, offsets):
        """Sorts the batch, probes / fills the cache for its unique rows and builds the
        per-lookup slot table -- or takes over the plan that prefetch() made for this batch.
        Must precede forward() and backward() of the same batch."""
        if self._queue:
            plan = self._queue[0]
            same = (plan.indices.data_ptr() == indices.data_ptr() and plan.indices.numel() == indices.numel()
                    and plan.offsets.data_ptr() == offsets.data_ptr() and plan.offsets.numel() == offsets.numel())
            if not same:
                raise RuntimeError("another batch was prefetched: batches must be prepared in the order they "
                                   "were prefetched (its slots and rows are already decided)")
            self._queue.pop(0)
        else:
            plan = self._plan(table_offsets, indices, offsets, ahead=False)
        self._commit(plan)
        plan.state = _Plan.FORWARDED
        self._current = plan

    # ------------------------------------------------------- views of the current plan
    @property
    def lookup_slots(self):
        p = self._require_current()
        return self._view(p.cws, p.layout.lookup_slots, p.n)

    def num_unique(self):
        p = self._require_current()
        return int(self._view(p.ws, p.plan_layout.num_unique, 1)[0]) if p.n else 0

    def unique_slots(self):
        p = self._require_current()
        return self._view(p.cws, p.layout.unique_slots, self.num_unique())

    def segment_starts(self):
        """First sorted position of each unique row of the batch, then the number of lookups."""
        p = self._require_current()
        return self._view(p.ws, p.plan_layout.segment_starts, self.num_unique() + 1)

    def unique_keys(self):
        p = self._require_current()
        starts = self.segment_starts()[:-1].long()
        return self._view(p.ws, p.plan_layout.keys_sorted, p.n)[starts]

    def evicted_keys(self):
        p = self._require_current()
        return self._view(p.cws, p.layout.evicted_keys, self.num_unique())

    def stage_area_base(self):
        """First row of the staging area that the current batch stages into."""
        p = self._require_current()
        area = p.sequence % STAGE_AREAS if self.deferred_write_back else 0
        return self.num_slots + area * self.stage_slots

    def stats(self):
        """Counters of the current batch's plan (synchronises)."""
        p = self._require_current()
        values = self._view(p.cws, p.layout.stats, len(STAT_NAMES)).tolist()
        return dict(zip(STAT_NAMES, values))

    # ---------------------------------------------------------------- arithmetic
    def forward(self, table_offsets, indices, offsets, per_sample_weights=None):
        p = self._require_current()
        slots = self.lookup_slots if p.n else None
        if self.mixed is not None:
            output = torch.empty((p.B, self.mixed.total_D), dtype=self.backing.dtype, device=self.device)
            with torch.cuda.device(self.device):
                _native.check(_native.load().tbe_forward_mixed_cached(
                    ctypes.byref(self.handle), self.dtype_code, self.mixed.vector_width, self.D, self.mixed.total_D,
                    _ptr(indices), p.n, _ptr(offsets), p.B, _ptr(per_sample_weights), _ptr(slots), _ptr(output),
                    self._stream()))
            return output
        output = torch.empty((p.B, p.T, self.D), dtype=self.backing.dtype, device=self.device)
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_forward_cached(
                ctypes.byref(self.handle), self.dtype_code, self.D, _ptr(table_offsets), p.T, _ptr(indices), p.n,
                _ptr(offsets), p.B, _ptr(per_sample_weights), _ptr(slots), _ptr(output), self._stream()))
        return output

    def backward(self, optimizer, grad_output, per_sample_weights, optimizer_state, learning_rate, eps,
                 stochastic_rounding=None, plan_id=None):
        """optimizer: 'sgd', 'adagrad' (exact row-wise Adagrad) or 'approx_adagrad' (the reference's
        per-lookup row-wise Adagrad, lookups of a row applied in position order).  Updates rows where they live; returns the gradient
        w.r.t. per_sample_weights or None.  stochastic_rounding: None, or the (seed, offset) of
        the random stream that rounds updated fp16 weights (Adagrad only).  plan_id: the value of
        self.plan_id after the prepare() of the batch this gradient belongs to; a later prepare()
        has replaced that batch's plan and slots (and may have evicted its rows), so the call is
        refused instead of applying the gradient to another batch's rows."""
        p = self._current
        if p is None or (plan_id is not None and plan_id != p.plan_id) or p.state == _Plan.REPLACED:
            raise RuntimeError(
                "the row cache was prepared for another batch since this batch's forward (plan %s, now %s): "
                "a cache-fronted module holds one batch between forward and backward -- run each forward's "
                "backward before the next forward" % (plan_id, self.plan_id))
        if p.state == _Plan.DONE:
            raise RuntimeError("this batch's backward has already run; its plan serves one update")
        shape = (p.B, p.T, self.D) if self.mixed is None else (p.B, self.mixed.total_D)
        if (grad_output.dtype != self.backing.dtype or grad_output.device != self.device
                or tuple(grad_output.shape) != shape):
            raise RuntimeError("grad_output must be %s of %s on %s (got %s of %s)"
                               % (shape, self.backing.dtype, self.device, tuple(grad_output.shape), grad_output.dtype))
        if optimizer not in ("sgd", "adagrad", "approx_adagrad"):
            raise ValueError("optimizer must be 'sgd', 'adagrad' or 'approx_adagrad' (got %r)" % (optimizer,))
        p.state = _Plan.DONE
        grad_output = grad_output.contiguous()
        grad_psw = None
        if per_sample_weights is not None:
            grad_psw = torch.empty(p.n, dtype=grad_output.dtype, device=self.device)
        code = _native.OPT_SGD if optimizer == "sgd" else _native.OPT_ROWWISE_ADAGRAD
        unique = self._view(p.cws, p.layout.unique_slots, max(p.n, 1))
        if self.mixed is not None:
            if optimizer == "approx_adagrad":
                code = _native.OPT_APPROX_ROWWISE_ADAGRAD
            with torch.cuda.device(self.device):
                _native.check(_native.load().tbe_backward_mixed_cached(
                    code, _ptr(grad_output), ctypes.byref(self.handle), self.dtype_code, self.mixed.vector_width,
                    self.D, self.mixed.total_D, p.B, p.n, _ptr(p.offsets), _ptr(per_sample_weights),
                    _ptr(optimizer_state) if optimizer != "sgd" else ctypes.c_void_p(0), float(learning_rate),
                    float(eps or 0.0), _ptr(grad_psw), int(stochastic_rounding is not None),
                    stochastic_rounding[0] if stochastic_rounding else 0,
                    stochastic_rounding[1] if stochastic_rounding else 0, _ptr(p.ws), p.ws.numel(), _ptr(unique),
                    self._stream()))
            return grad_psw
        if optimizer == "approx_adagrad":
            with torch.cuda.device(self.device):
                _native.check(_native.load().tbe_backward_approx_cached(
                    _ptr(grad_output), ctypes.byref(self.handle), self.dtype_code, self.total_rows, self.D,
                    p.T, p.B, p.n, _ptr(p.offsets), _ptr(per_sample_weights), _ptr(optimizer_state),
                    float(learning_rate), float(eps or 0.0), _ptr(grad_psw), int(stochastic_rounding is not None),
                    stochastic_rounding[0] if stochastic_rounding else 0,
                    stochastic_rounding[1] if stochastic_rounding else 0, _ptr(p.ws), p.ws.numel(), _ptr(unique),
                    self._stream()))
            return grad_psw
        with torch.cuda.device(self.device):
            _native.check(_native.load().tbe_backward_cached(
                code, _ptr(grad_output), ctypes.byref(self.handle), self.dtype_code, self.total_rows, self.D,
                p.T, p.B, p.n, _ptr(per_sample_weights),
                _ptr(optimizer_state) if optimizer != "sgd" else ctypes.c_void_p(0), float(learning_rate),
                float(eps or 0.0), _ptr(grad_psw), int(stochastic_rounding is not None),
                stochastic_rounding[0] if stochastic_rounding else 0,
                stochastic_rounding[1] if stochastic_rounding else 0, _ptr(p.ws), p.ws.numel(),
                _ptr(unique), self._stream()))
        return grad_psw

    # ------------------------------------------------------------------ write-back
    def flush(self):
        """Writes every resident row (and every staged or evicted row whose write-back is still
        pending) back to the backing table.  Call it between steps: a prefetched batch is committed
        first (its slots are already decided), which takes the slots away from a batch whose
        backward has not run yet -- that backward is then refused."""
        for plan in self._queue:
            if plan.state == _Plan.PREFETCHED:
                if self._current is not None and self._current.state == _Plan.FORWARDED:
                    self._current.state = _Plan.REPLACED
                self._commit(plan)
        # planned batches whose update is still to come keep their staging areas listed: they are the
        # newest plans, consecutive in sequence
        live = 0
        for plan in sorted((p for p in self._slots if p is not None), key=lambda p: -p.sequence):
            if plan.state not in (_Plan.COMMITTED, _Plan.FORWARDED):
                break
            live += 1
        with torch.cuda.device(self.device):
            current = torch.cuda.current_stream(self.device)
            current.wait_stream(self.plan_stream)
            current.wait_stream(self.link_stream)
            _native.check(_native.load().tbe_cache_flush(ctypes.byref(self.handle), self.dtype_code, self.D, live,
                                                         self.sequence, self._stream()))

    def invalidate(self, write_back=True):
        """Empties the cache (tags, recency and frequency words back to their initial values), after
        writing the resident rows back to the backing table unless write_back is False.  Needed
        whenever the backing table is written behind the cache's back (loading a checkpoint,
        assigning to the weights): a resident row would otherwise keep serving, and later write
        back, its old value.  Any planned batch, prefetched ones included, is dropped."""
        if write_back:
            self.flush()
        for plan in self._slots:
            if plan is not None:
                plan.state = _Plan.REPLACED
        self._queue = []
        self._current = None
        with torch.cuda.device(self.device):
            current = torch.cuda.current_stream(self.device)
            current.wait_stream(self.plan_stream)
            current.wait_stream(self.link_stream)
            _native.check(_native.load().tbe_cache_init(ctypes.byref(self.handle), self._stream()))

    def resident_keys(self):
        """Sorted keys of the rows currently held (synchronises)."""
        return torch.sort(self.tags[self.tags >= 0])[0]
