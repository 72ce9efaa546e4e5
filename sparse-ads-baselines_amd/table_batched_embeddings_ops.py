"""Drop-in for the reference's table_batched_embeddings_ops.py (uniform-D part, :1-201).

`TableBatchedEmbeddingBags` keeps the reference's constructor arguments, state-dict
keys (`embedding_weights`, `table_offsets`, `optimizer_state`), flat `[sum(rows), D]`
weight layout and `forward(indices, offsets, per_sample_weights)` signature; the
optimizer is applied inside backward.  Differences, all extensions:
  * `num_embeddings` may be a list of per-table row counts;
  * SGD backward is exact (each distinct row updated once with its summed gradient);
  * EXACT_ROWWISE_ADAGRAD accepts per-sample weights;
  * APPROX_ROWWISE_ADAGRAD applies the lookups of a row one at a time in position order, so a
    batch in which rows repeat has a defined, reproducible result.
"""
import enum
import logging

import numpy as np
import torch
from torch import nn

import table_batched_embeddings
import table_batched_embeddings_cache

# The module behind the ten functions that the reference imports as `table_batched_embeddings`
# (table_batched_embeddings_ops.py:24, 53, 148): the Python binding of the C ABI by default, or the
# compiled one (table_batched_embeddings_cpp, same names and positional arguments) after
# use_extension().  What the reference's module does not have (plan-ahead, the row cache, exact SGD
# for mixed-dimension tables) always comes from the Python binding.
extension = table_batched_embeddings


def use_extension(module):
    """Routes the reference's ten extension functions through `module`
    (table_batched_embeddings or table_batched_embeddings_cpp); returns the previous one."""
    global extension
    previous, extension = extension, module
    return previous


class Optimizer(enum.Enum):
    SGD = 1
    APPROX_ROWWISE_ADAGRAD = 2
    EXACT_ROWWISE_ADAGRAD = 3


class EmbeddingLocation(enum.Enum):
    DEVICE = 0
    HOST_MAPPED = 1
    HOST_CACHED = 2  # extension: pinned host table fronted by an HBM row cache


def _launch_block(D):
    # the reference's BT_block_size heuristic (table_batched_embeddings_ops.py:38);
    # forwarded for signature compatibility, the kernels do not use it
    return int(max(256 / D, 1))


class LookupFunction(torch.autograd.Function):
    """Mirror of LookupFunction (table_batched_embeddings_ops.py:9-121)."""

    plan_ahead = False  # start the backward's sort during forward, on a side stream

    @staticmethod
    def forward(ctx, weights, table_offsets, indices, offsets, per_sample_weights, optimizer,
                optimizer_state, learning_rate, eps, stochastic_rounding):
        ctx.optimizer = optimizer
        ctx.learning_rate = learning_rate
        ctx.eps = eps
        ctx.stochastic_rounding = stochastic_rounding
        ctx.save_for_backward(weights, table_offsets, indices, offsets, per_sample_weights, optimizer_state)
        L_max = 200
        # The sort that the backward needs depends on the indices only, so it can be started here on
        # a side stream (table_batched_embeddings.plan_backward).  Measured on MI355X it does not
        # pay: the forward gather occupies every CU and a default-priority side stream only gets
        # the slots it leaves, so the step time is unchanged.  Off unless a caller opts in.
        ctx.plan = None
        if (LookupFunction.plan_ahead and any(ctx.needs_input_grad)
                and optimizer != Optimizer.APPROX_ROWWISE_ADAGRAD):
            ctx.plan = table_batched_embeddings.plan_backward(weights, table_offsets, indices, offsets)
        return extension.forward(
            weights, table_offsets, indices, offsets, per_sample_weights, L_max,
            _launch_block(weights.shape[1]), False)

    @staticmethod
    def backward(ctx, grad_output):
        (weights, table_offsets, indices, offsets, per_sample_weights, optimizer_state) = ctx.saved_tensors
        L_max = 200
        assert ctx.optimizer in (Optimizer.SGD, Optimizer.APPROX_ROWWISE_ADAGRAD,
                                 Optimizer.EXACT_ROWWISE_ADAGRAD)
        plan, ctx.plan = ctx.plan, None
        if plan is not None:
            assert ctx.optimizer != Optimizer.SGD or per_sample_weights is None
            import tbe_native
            code = tbe_native.OPT_SGD if ctx.optimizer == Optimizer.SGD else tbe_native.OPT_ROWWISE_ADAGRAD
            grad_per_sample_weight = plan.apply(code, grad_output, weights, per_sample_weights, optimizer_state,
                                                ctx.learning_rate, ctx.eps, ctx.stochastic_rounding)
        elif ctx.optimizer == Optimizer.SGD:
            assert per_sample_weights is None
            grad_per_sample_weight = extension.backward_sgd(
                grad_output, weights, table_offsets, indices, offsets, ctx.learning_rate, L_max,
                _launch_block(weights.shape[1]), False)
        elif ctx.optimizer == Optimizer.APPROX_ROWWISE_ADAGRAD:
            grad_per_sample_weight = extension.backward_approx_adagrad(
                grad_output, weights, table_offsets, indices, offsets, per_sample_weights,
                optimizer_state, ctx.learning_rate, ctx.eps, L_max, ctx.stochastic_rounding, 1)
        else:
            grad_per_sample_weight = extension.backward_exact_adagrad(
                grad_output, weights, table_offsets, indices, offsets, per_sample_weights,
                optimizer_state, ctx.learning_rate, ctx.eps, ctx.stochastic_rounding, 1)
        # The update is already applied; autograd receives an empty sparse gradient of the
        # weights' shape (table_batched_embeddings_ops.py:110-111), here in the weights' dtype.
        empty_grad = None
        if ctx.needs_input_grad[0]:
            empty_grad = torch.sparse_coo_tensor(
                torch.empty((2, 0), dtype=torch.int64, device=weights.device),
                torch.empty((0,), dtype=weights.dtype, device=weights.device),
                size=tuple(weights.shape))
        return (empty_grad, None, None, None, grad_per_sample_weight, None, None, None, None, None)


class CachedLookupFunction(torch.autograd.Function):
    """LookupFunction for tables that live in host memory behind an HBM row cache: the batch
    is planned (sorted, cut into unique rows) once, the cache is probed / filled for those
    rows, and forward and backward address every row where it lives."""

    @staticmethod
    def forward(ctx, weights, module, indices, offsets, per_sample_weights):
        cache = module.row_cache
        first_rows = module.cache_table_rows()
        cache.prepare(first_rows, indices, offsets)
        ctx.module = module
        ctx.plan_id = cache.plan_id
        ctx.save_for_backward(weights, per_sample_weights)
        return cache.forward(first_rows, indices, offsets, per_sample_weights)

    @staticmethod
    def backward(ctx, grad_output):
        weights, per_sample_weights = ctx.saved_tensors
        module = ctx.module
        if module.optimizer == Optimizer.SGD:
            assert per_sample_weights is None
            kind = "sgd"
        elif module.optimizer == Optimizer.APPROX_ROWWISE_ADAGRAD:
            kind = "approx_adagrad"
        else:
            kind = "adagrad"
        rounding = None
        if module.stochastic_rounding and kind != "sgd" and weights.dtype == torch.float16:
            rounding = table_batched_embeddings._rounding_stream(weights.device)
        grad_per_sample_weight = module.row_cache.backward(
            kind, grad_output, per_sample_weights, module.optimizer_state, module.learning_rate, module.eps,
            rounding, plan_id=ctx.plan_id)
        empty_grad = None
        if ctx.needs_input_grad[0]:
            empty_grad = torch.sparse_coo_tensor(
                torch.empty((weights.dim(), 0), dtype=torch.int64, device=weights.device),
                torch.empty((0,), dtype=weights.dtype, device=weights.device), size=tuple(weights.shape))
        return (empty_grad, None, None, None, grad_per_sample_weight)


class _CacheFronted:
    """What the two modules share when their tables sit behind a row cache: the cache keeps device
    addresses (the pinned table, and for mixed-D tables the three offset buffers), so a call that
    moves or casts them (.to(other), .half(), .double()) is refused instead of leaving the cache
    pointing at freed memory."""

    def _cache_anchors(self):
        cache = getattr(self, "row_cache", None)
        if cache is None:
            return None
        anchors = [self.embedding_weights.data_ptr(), self.embedding_weights.dtype]
        if cache.mixed is not None:
            anchors += [self.table_offsets.data_ptr(), self.table_dim_offsets.data_ptr(), self.dim_offsets.data_ptr()]
        return anchors

    def _apply(self, fn, *args, **kwargs):
        before = self._cache_anchors()
        out = super()._apply(fn, *args, **kwargs)
        if before is not None and before != self._cache_anchors():
            raise RuntimeError("a module whose tables sit behind the row cache (EmbeddingLocation.HOST_CACHED) cannot "
                               "be moved to another device or cast: the cache holds the addresses of its tensors")
        return out


class TableBatchedEmbeddingBags(_CacheFronted, nn.Module):
    """Mirror of TableBatchedEmbeddingBags (table_batched_embeddings_ops.py:135-201)."""

    def __init__(self, num_tables, num_embeddings, embedding_dim, optimizer=Optimizer.SGD,
                 learning_rate=0.01, eps=None, stochastic_rounding=False, fp16=False,
                 managed=EmbeddingLocation.DEVICE, cache_slots=None, cache_policy="lru",
                 cache_stage_slots=0, cache_deferred_write_back=True):
        super(TableBatchedEmbeddingBags, self).__init__()
        assert managed in (EmbeddingLocation.DEVICE, EmbeddingLocation.HOST_MAPPED,
                           EmbeddingLocation.HOST_CACHED)
        if isinstance(num_embeddings, (list, tuple, np.ndarray)):
            rows = [int(r) for r in num_embeddings]
            assert len(rows) == num_tables
        else:
            rows = [int(num_embeddings)] * num_tables
        total_rows = int(sum(rows))
        dtype = torch.float16 if fp16 else torch.float32
        device = torch.device("cuda", torch.cuda.current_device())
        if managed == EmbeddingLocation.DEVICE:
            logging.info("Allocating device embedding bag")
            embedding_data = torch.randn(total_rows, embedding_dim, device=device, dtype=dtype)
        elif managed == EmbeddingLocation.HOST_MAPPED:
            logging.info("Allocating host-mapped embedding bag")
            embedding_data = extension.new_managed_tensor(
                torch.empty(1, device=device, dtype=dtype), (total_rows, embedding_dim))
            embedding_data.normal_()
        else:
            logging.info("Allocating pinned host embedding bag behind an HBM row cache")
            embedding_data = extension.new_host_mapped_tensor(
                torch.empty(1, device=device, dtype=dtype), (total_rows, embedding_dim))
            embedding_data.normal_()
        self.embedding_weights = nn.Parameter(embedding_data)
        self.row_cache = None
        if managed == EmbeddingLocation.HOST_CACHED:
            assert cache_slots is not None, "HOST_CACHED needs cache_slots"
            self.row_cache = table_batched_embeddings_cache.RowCache(self.embedding_weights.data, cache_slots,
                                                                     cache_policy, cache_stage_slots,
                                                                     cache_deferred_write_back)
            # checkpoints must see the rows the cache holds ...
            self.register_state_dict_pre_hook(lambda module, prefix, keep_vars: module.flush_cache())
            # ... and a loaded checkpoint must not be shadowed (or later overwritten) by rows that
            # were resident before it was loaded
            self.register_load_state_dict_pre_hook(lambda module, *args: module.invalidate_cache())
        self.register_buffer("table_offsets",
                             torch.tensor([0] + np.cumsum(rows[:-1]).tolist()).int())
        # unused by SGD, kept so state dicts interchange (table_batched_embeddings_ops.py:177-180)
        self.register_buffer("optimizer_state", torch.zeros(total_rows).float())
        self.optimizer = optimizer
        self.learning_rate = learning_rate
        self.eps = eps
        self.stochastic_rounding = stochastic_rounding

    def cache_table_rows(self):
        """First row of each table, as the row cache's calls take it."""
        return self.table_offsets

    def flush_cache(self):
        """Writes the rows held by the HBM cache back to embedding_weights (no-op without a cache)."""
        if self.row_cache is not None:
            self.row_cache.flush()

    def invalidate_cache(self):
        """Writes the resident rows back, then empties the cache.  Call it after writing to
        embedding_weights directly (load_state_dict does so itself); no-op without a cache."""
        if self.row_cache is not None:
            self.row_cache.invalidate()

    def prefetch(self, sharded_sparse_features, sharded_offsets):
        """HOST_CACHED tables: plans the NEXT batch while the current one computes -- its sort, its
        cache slots and most of its row traffic over the host link run on side streams.  Call it
        before the current batch's forward for the most overlap; batches must then be given to
        forward() in the order they were prefetched, and the two tensors must stay unchanged until
        then.  Results are the same with and without it.  (No counterpart in the reference, whose
        host-resident tables are read over the bus on every lookup.)"""
        if self.row_cache is None:
            raise RuntimeError("prefetch is for tables behind the row cache (managed=EmbeddingLocation.HOST_CACHED)")
        self.row_cache.prefetch(self.cache_table_rows(), sharded_sparse_features, sharded_offsets)

    def forward(self, sharded_sparse_features, sharded_offsets, per_sample_weights=None):
        if self.row_cache is not None:
            return CachedLookupFunction.apply(self.embedding_weights, self, sharded_sparse_features,
                                              sharded_offsets, per_sample_weights)
        return LookupFunction.apply(
            self.embedding_weights, self.table_offsets, sharded_sparse_features, sharded_offsets,
            per_sample_weights, self.optimizer, self.optimizer_state, self.learning_rate, self.eps,
            self.stochastic_rounding)


class MixedDimLookupFunction(torch.autograd.Function):
    """Mirror of MixedDimLookupFunction (table_batched_embeddings_ops.py:204-321)."""

    @staticmethod
    def forward(ctx, weights, table_offsets, table_dim_offsets, dim_offsets, total_D, indices, offsets,
                per_sample_weights, optimizer, optimizer_state, learning_rate, eps, stochastic_rounding):
        ctx.optimizer = optimizer
        ctx.learning_rate = learning_rate
        ctx.eps = eps
        ctx.stochastic_rounding = stochastic_rounding
        ctx.total_D = total_D
        ctx.save_for_backward(weights, table_offsets, table_dim_offsets, dim_offsets, indices, offsets,
                              per_sample_weights, optimizer_state)
        return extension.forward_mixed_D(
            weights, table_offsets, dim_offsets, total_D, indices, offsets, per_sample_weights, 200, 1, False)

    @staticmethod
    def backward(ctx, grad_output):
        (weights, table_offsets, table_dim_offsets, dim_offsets, indices, offsets, per_sample_weights,
         optimizer_state) = ctx.saved_tensors
        L_max = 200
        if ctx.optimizer == Optimizer.SGD:  # extension: the reference asserts Adagrad here (:269)
            assert per_sample_weights is None
            grad_per_sample_weight = table_batched_embeddings.backward_sgd_mixed_D(
                grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, ctx.total_D, indices, offsets,
                optimizer_state, ctx.learning_rate)
        elif ctx.optimizer == Optimizer.APPROX_ROWWISE_ADAGRAD:
            grad_per_sample_weight = extension.backward_approx_adagrad_mixed_D(
                grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, ctx.total_D, indices, offsets,
                per_sample_weights, optimizer_state, ctx.learning_rate, ctx.eps, L_max, ctx.stochastic_rounding, 1)
        else:
            grad_per_sample_weight = extension.backward_exact_adagrad_mixed_D(
                grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, ctx.total_D, indices, offsets,
                per_sample_weights, optimizer_state, ctx.learning_rate, ctx.eps, ctx.stochastic_rounding, 1)
        empty_grad = None
        if ctx.needs_input_grad[0]:
            empty_grad = torch.sparse_coo_tensor(
                torch.empty((1, 0), dtype=torch.int64, device=weights.device),
                torch.empty((0,), dtype=weights.dtype, device=weights.device), size=tuple(weights.shape))
        return (empty_grad, None, None, None, None, None, None, grad_per_sample_weight, None, None, None, None,
                None)


class MixedDimTableBatchedEmbeddingBags(_CacheFronted, nn.Module):
    """Mirror of MixedDimTableBatchedEmbeddingBags (table_batched_embeddings_ops.py:324-435):
    `embeddings` is a list of (rows, dim) per table; weights are one flat 1-D parameter."""

    def __init__(self, embeddings, optimizer=Optimizer.SGD, learning_rate=0.01, eps=None,
                 stochastic_rounding=False, fp16=False, managed=EmbeddingLocation.DEVICE, cache_slots=None,
                 cache_policy="lru", cache_stage_slots=0, cache_deferred_write_back=True):
        """managed=EmbeddingLocation.HOST_CACHED (an extension, like that of TableBatchedEmbeddingBags):
        the tables live in pinned host memory behind an HBM row cache of cache_slots rows of the widest
        table's width."""
        super(MixedDimTableBatchedEmbeddingBags, self).__init__()
        assert managed in (EmbeddingLocation.DEVICE, EmbeddingLocation.HOST_MAPPED, EmbeddingLocation.HOST_CACHED)
        rows, dims = zip(*embeddings)
        assert all(d > 0 and d % 4 == 0 for d in dims), "every embedding dimension must be a multiple of 4"
        numel = sum(row * dim for (row, dim) in embeddings)
        dtype = torch.float16 if fp16 else torch.float32
        device = torch.device("cuda", torch.cuda.current_device())
        if managed == EmbeddingLocation.DEVICE:
            logging.info("Allocating device embedding bag")
            embedding_data = torch.randn(size=(numel,), device=device, dtype=dtype)
        elif managed == EmbeddingLocation.HOST_MAPPED:
            logging.info("Allocating host-mapped embedding bag")
            embedding_data = extension.new_managed_tensor(
                torch.empty(1, device=device, dtype=dtype), (numel,))
            embedding_data.normal_()
        else:
            logging.info("Allocating pinned host embedding bag behind an HBM row cache")
            embedding_data = extension.new_host_mapped_tensor(
                torch.empty(1, device=device, dtype=dtype), (numel,))
            embedding_data.normal_()
        self.embedding_weights = nn.Parameter(embedding_data)
        self.register_buffer("table_dim_offsets", torch.tensor([0] + np.cumsum(rows).tolist()).int())
        self.register_buffer("table_offsets",
                             torch.tensor([0] + np.cumsum([r * d for r, d in zip(rows, dims)]).tolist()).long())
        self.register_buffer("dim_offsets", torch.tensor([0] + np.cumsum(dims).tolist()).int())
        self.register_buffer("optimizer_state", torch.zeros(sum(rows)).float())
        self.total_D = sum(dims)
        self.optimizer = optimizer
        self.learning_rate = learning_rate
        self.eps = eps
        self.stochastic_rounding = stochastic_rounding
        self.row_cache = None
        if managed == EmbeddingLocation.HOST_CACHED:
            assert cache_slots is not None, "HOST_CACHED needs cache_slots"
            self.to(device)  # the cache keeps the addresses of the three offset buffers
            self.row_cache = table_batched_embeddings_cache.RowCache(
                self.embedding_weights.data, cache_slots, cache_policy, cache_stage_slots, cache_deferred_write_back,
                mixed=table_batched_embeddings_cache.MixedTables(self.table_offsets, self.table_dim_offsets,
                                                                 self.dim_offsets))
            # (as for TableBatchedEmbeddingBags: checkpoints see the cached rows, a loaded one is not shadowed)
            self.register_state_dict_pre_hook(lambda module, prefix, keep_vars: module.flush_cache())
            self.register_load_state_dict_pre_hook(lambda module, *args: module.invalidate_cache())

    def cache_table_rows(self):
        """First row of each table, as the row cache's calls take it."""
        return self.row_cache.mixed.table_rows

    def flush_cache(self):
        """Writes the rows held by the HBM cache back to embedding_weights (no-op without a cache)."""
        if self.row_cache is not None:
            self.row_cache.flush()

    def invalidate_cache(self):
        """Writes the resident rows back, then empties the cache (see TableBatchedEmbeddingBags)."""
        if self.row_cache is not None:
            self.row_cache.invalidate()

    def prefetch(self, sharded_sparse_features, sharded_offsets):
        """HOST_CACHED tables: plans the NEXT batch while the current one computes (see
        TableBatchedEmbeddingBags.prefetch)."""
        if self.row_cache is None:
            raise RuntimeError("prefetch is for tables behind the row cache (managed=EmbeddingLocation.HOST_CACHED)")
        self.row_cache.prefetch(self.cache_table_rows(), sharded_sparse_features, sharded_offsets)

    def forward(self, sharded_sparse_features, sharded_offsets, per_sample_weights=None):
        if self.row_cache is not None:
            return CachedLookupFunction.apply(self.embedding_weights, self, sharded_sparse_features,
                                              sharded_offsets, per_sample_weights)
        return MixedDimLookupFunction.apply(
            self.embedding_weights, self.table_offsets, self.table_dim_offsets, self.dim_offsets, self.total_D,
            sharded_sparse_features, sharded_offsets, per_sample_weights, self.optimizer, self.optimizer_state,
            self.learning_rate, self.eps, self.stochastic_rounding)

    def split_embedding_weights(self):
        """Returns a list of weights, split by table."""
        T = self.table_offsets.size(0) - 1
        return [
            self.embedding_weights.detach()[self.table_offsets[i]:self.table_offsets[i + 1]].view(
                self.table_dim_offsets[i + 1] - self.table_dim_offsets[i],
                self.dim_offsets[i + 1] - self.dim_offsets[i])
            for i in range(T)
        ]

    def split_optimizer_state(self):
        """Returns a list of optimizer states, split by table."""
        T = self.table_offsets.size(0) - 1
        return [self.optimizer_state.detach()[self.table_dim_offsets[i]:self.table_dim_offsets[i + 1]]
                for i in range(T)]

    def split_output(self, output):
        """Returns a list of outputs, split by table."""
        T = self.table_offsets.size(0) - 1
        return [output[:, self.dim_offsets[i]:self.dim_offsets[i + 1]] for i in range(T)]
