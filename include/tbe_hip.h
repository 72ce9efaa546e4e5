/*
 * tbe_hip.h -- C ABI of the MI355X (gfx950) table-batched embedding-bag library.
 *
 * Every entry point takes plain device pointers, sizes and an opaque HIP stream
 * (a hipStream_t passed as void*; NULL = the default stream).  No compute entry
 * point allocates device memory: scratch is a caller-owned workspace whose size
 * is reported by the *_workspace_* queries (tbe_backward_sgd_static uses an array
 * the library holds instead).  The exceptions are the allocators at the end of
 * this file (tbe_host_mapped_alloc, tbe_managed_alloc), the HIP events that the
 * kernel-timing aid creates between tbe_profile_begin/end, and the two events
 * tbe_cache_prepare creates once per calling thread to join its side stream.  No entry
 * point other than tbe_profile_end synchronises the host with the device.
 *
 * Return value: 0 (TBE_OK) on success, a TBE_ERR_* code otherwise; the message
 * of the last failure on the calling thread is returned by tbe_last_error().
 * This mirrors the reference's AT_ASSERT / AT_CUDA_CHECK -> RuntimeError
 * behaviour (table_batched_embeddings_cuda.cu:262-273, 314): the Python host
 * turns a non-zero code into RuntimeError.
 *
 * Layout conventions (table_batched_embeddings_cuda.cu:193-222):
 *   weights        [total_rows][D], row-major, element type `dtype`
 *   table_offsets  int32 [T]     first row of each table inside `weights`
 *   indices        int32 [N]     table-major: all bags of table 0, then table 1...
 *   offsets        int32 [T*B+1] bag (t,b) owns indices[offsets[t*B+b] : offsets[t*B+b+1]]
 *   output / grad  [B][T][D]     bag-major, element type `dtype`
 *   D % 4 == 0.
 */
#ifndef TBE_HIP_H
#define TBE_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported symbols; everything else in the library has hidden visibility. */
#define TBE_API __attribute__((visibility("default")))

/* element type of weights / outputs / gradients / per-sample weights */
enum { TBE_DTYPE_F32 = 0, TBE_DTYPE_F16 = 1, TBE_DTYPE_F64 = 2 };

/* optimizer selector of the entry points that serve several optimizers */
enum {
  TBE_OPT_SGD = 0,
  TBE_OPT_ROWWISE_ADAGRAD = 1,        /* exact: one update per distinct row with its summed gradient */
  TBE_OPT_APPROX_ROWWISE_ADAGRAD = 2  /* per lookup, see tbe_backward_approx_adagrad (tbe_backward_mixed only) */
};

enum {
  TBE_OK = 0,
  TBE_ERR_INVALID = 1,     /* a shape / pointer / dtype precondition failed */
  TBE_ERR_WORKSPACE = 2,   /* workspace pointer NULL or too small           */
  TBE_ERR_HIP = 3,         /* a HIP runtime call or kernel launch failed    */
  TBE_ERR_UNSUPPORTED = 4  /* a valid request this library does not serve   */
};

/* Message of the last error raised on this thread ("" if none). */
TBE_API const char *tbe_last_error(void);

/* ABI version; bumped whenever a signature below changes. */
TBE_API int32_t tbe_abi_version(void);

/* ---------------------------------------------------------- kernel timing
 * Benchmark aid with no counterpart in the reference (it times whole calls with
 * CUDA events, table_batched_embeddings_benchmark.py:27-37).  Between
 * tbe_profile_begin() and tbe_profile_end() every kernel launch of this library
 * is bracketed by two HIP events recorded on the launch stream.
 * tbe_profile_end() waits for those events; tbe_profile_get(i, ...) then returns
 * the kernel's short name and its duration in milliseconds, in launch order.
 */
TBE_API int tbe_profile_begin(void);
TBE_API int tbe_profile_end(void);
TBE_API int32_t tbe_profile_count(void);
TBE_API int tbe_profile_get(int32_t i, const char **name, float *milliseconds);

/* Benchmark aid with no counterpart in the reference: the memory system's rate for the row-access
 * pattern of the gather and update kernels, with none of their bookkeeping.  Lane groups of
 * row_bytes / 16 lanes visit rows[row_ids[i]] (row_bytes = 64, 128, 256 or 512; eight independent
 * rows in flight per group) in the order of row_ids.  modify = 0: the rows are read (and
 * state[row_ids[i]], if state is not NULL); modify = 1: every row is read, changed and written
 * back in place, and so is its state word -- row_ids must then hold no row twice.  `sink` is 16
 * bytes of device memory that the read-only form may write. */
TBE_API int tbe_probe_row_access(void *rows, int32_t row_bytes, const int32_t *row_ids, int64_t num_ids,
                                 float *state, int32_t modify, void *sink, void *stream);

/* ------------------------------------------------------------------ forward
 * Pooled gather-sum:  output[b][t][:] = sum_{p in bag(t,b)} (psw[p] *) weights[table_offsets[t] + indices[p]][:]
 * Replaces batched_embedding_forward_cuda (table_batched_embeddings_cuda.cu:253-316,
 * bound as "forward" in table_batched_embeddings.cpp:58).  `per_sample_weights`
 * may be NULL (unweighted); otherwise it has `dtype` elements and length N.
 * Accumulation is fp32 for F16/F32 and fp64 for F64; the result is rounded to
 * nearest-even once.  An empty bag yields zeros.  The reference's launch knobs
 * (L_max, BT_block_size, shmem) do not exist here.
 */
TBE_API int tbe_forward(const void *weights, int32_t dtype, int32_t D,
                const int32_t *table_offsets, int32_t T,
                const int32_t *indices, int64_t num_indices,
                const int32_t *offsets, int32_t B,
                const void *per_sample_weights,
                void *output, void *stream);

/* ----------------------------------------------------------------- backward
 * Byte offsets of the regions of the backward workspace.  After a backward call
 * the first five regions hold the intermediate results that the parity gates
 * inspect (all int32):
 *   keys              [N]   table_offsets[t] + indices[p]             (tbe.cu:1495); only for batches
 *                           over more than 2048 tables, whose keys are sorted in one piece -- otherwise
 *                           the backward entry points sort the indices table by table, nothing is
 *                           written here and the region is 256 bytes
 *   keys_sorted       [N]   stable ascending sort of keys             (tbe.cu:1639-1655)
 *   positions_sorted  [N]   position p of each sorted key (IndexInfo.indices_idx, tbe.cu:1217)
 *   segment_starts    [U+1] first sorted position of each unique key, then N (tbe.cu:1523-1539)
 *   num_unique        [1]   U
 */
typedef struct tbe_workspace_layout {
  uint64_t total_bytes;
  uint64_t keys;
  uint64_t grad_rows;        /* int32 [N]: b*T + t of the bag owning position p        */
  uint64_t keys_sorted;
  uint64_t positions_sorted;
  uint64_t segment_starts;
  uint64_t num_unique;       /* int32 [320]: U, then the update stage's queue counters
                              * (one 128-byte line per eighth of the sorted positions)   */
  uint64_t sort_scratch;
  uint64_t segment_scratch;
  uint64_t segment_ids;      /* int32 [N]: index of the unique row of each sorted position */
  uint64_t long_segments;    /* 16-byte records [max_long_segments]: rows reduced in several chunks */
  uint64_t chunk_segments;   /* 32-byte records [8][max_chunks / 8]: queues of occurrence chunks,
                              * one per eighth of the sorted positions                          */
  uint64_t partial_sums;     /* accumulator-typed [max_partial_rows][D]                         */
  int64_t max_long_segments;
  int64_t max_chunks;
  int64_t max_partial_rows;
} tbe_workspace_layout_t;

/* T (number of tables) sizes the sort scratch: no sort tile straddles two tables. */
TBE_API int tbe_backward_workspace_layout(int64_t num_indices, int32_t D, int32_t dtype, int32_t T,
                                  tbe_workspace_layout_t *layout);

/* Exact SGD:  weights[r][:] -= lr * sum_{p: key[p]==r} grad_output[b(p)][t(p)][:]
 * once per distinct row r, with no atomics and a fixed summation order
 * (ascending position).  Replaces batched_embedding_backward_sgd_cuda
 * (table_batched_embeddings_cuda.cu:383-435, "backward_sgd" in
 * table_batched_embeddings.cpp:59), whose per-lookup read-modify-write is only
 * correct when no row repeats (test_table_batched_embeddings.py:177-193).
 * `total_rows` is the row count of `weights`.  `max_table_rows` is an upper bound of the row
 * count of the largest table, or 0 when unknown (total_rows is then used): it fixes the number
 * of key bits sorted, as optimizer_state.numel() does at tbe.cu:1643 -- the lookups of a table
 * are consecutive, so each table's indices are sorted on their own and the bits of a row
 * inside its table suffice.  The sorted order is that of the (table, row) keys either way; an
 * index >= 2^ceil(log2(bound + 1)) is an error of the caller, like any out-of-range index.
 */
TBE_API int tbe_backward_sgd(const void *grad_output, void *weights, int32_t dtype,
                     int64_t total_rows, int64_t max_table_rows, int32_t D,
                     const int32_t *table_offsets, int32_t T,
                     const int32_t *indices, int64_t num_indices,
                     const int32_t *offsets, int32_t B,
                     float learning_rate,
                     void *workspace, uint64_t workspace_bytes, void *stream);

/* tbe_backward_sgd for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc).  It has no counterpart in the reference,
 * which allocates its sort buffers inside every backward call
 * (table_batched_embeddings_cuda.cu:1618-1647).  Same arguments, same kernels and bit-identical
 * results, but the workspace is an array of TBE_STATIC_SCRATCH_BYTES that the library's code
 * object holds on every device it runs on; the call makes no hipMalloc / hipFree and no other
 * allocating call.  A batch whose workspace (tbe_backward_workspace_layout(...).total_bytes)
 * exceeds TBE_STATIC_SCRATCH_BYTES is refused with TBE_ERR_WORKSPACE -- about 0.8 M lookups fit.
 * The first call on a device resolves the array's address there (make it outside a capture).
 * All calls on one device share the array, which keeps the previous call's contents: every
 * counter the pipeline needs at zero is cleared by its own kernels at the start of each call,
 * and two calls that overlap on one device (different streams or threads) race.  After the call
 * the array holds the intermediate results in the layout of tbe_backward_workspace_layout, as a
 * caller's workspace would.
 */
#define TBE_STATIC_SCRATCH_BYTES (32ull << 20)
TBE_API int tbe_backward_sgd_static(const void *grad_output, void *weights, int32_t dtype,
                                    int64_t total_rows, int64_t max_table_rows, int32_t D,
                                    const int32_t *table_offsets, int32_t T,
                                    const int32_t *indices, int64_t num_indices,
                                    const int32_t *offsets, int32_t B,
                                    float learning_rate, void *stream);

/* Exact row-wise Adagrad (table_batched_embeddings_cuda.cu:1589-1706 with
 * AdaGradFunctor, :437-471; "backward_exact_adagrad" in table_batched_embeddings.cpp:61):
 *   G = sum over the occurrences of row r of (psw[p] *) grad_output[b(p)][t(p)][:]
 *   state[r] += sum_d G_d^2 ;  weights[r][:] -= lr / (sqrt(state[r]) + eps) * G
 * `optimizer_state` is float [total_rows] for F16/F32 weights, double for F64.
 * When `per_sample_weights` is non-NULL, `grad_per_sample_weights` (same dtype,
 * length N) receives <weights_before_update[row(p)], grad_output[b(p)][t(p)]>,
 * the quantity the reference's weighted functor accumulates (tbe.cu:529-553);
 * the reference leaves the weighted exact case unimplemented (tbe.cu:1552, 1678).
 */
TBE_API int tbe_backward_exact_adagrad(const void *grad_output, void *weights, int32_t dtype,
                               int64_t total_rows, int64_t max_table_rows, int32_t D,
                               const int32_t *table_offsets, int32_t T,
                               const int32_t *indices, int64_t num_indices,
                               const int32_t *offsets, int32_t B,
                               const void *per_sample_weights,
                               void *optimizer_state,
                               float learning_rate, float eps,
                               void *grad_per_sample_weights,
                               void *workspace, uint64_t workspace_bytes, void *stream);

/* Approximate row-wise Adagrad: the per-lookup update of
 * batched_embedding_backward_adagrad_approx_cuda (table_batched_embeddings_cuda.cu:706-793, kernel
 * :648-704, functors :437-553; "backward_approx_adagrad" in table_batched_embeddings.cpp:60).
 * For every lookup p of bag (t, b), with g = grad_output[b][t][:] and r = its row:
 *   wss = sum_d g_d^2 (* psw[p]^2);  state[r] += wss
 *   mult = (psw[p] *) lr / (sqrt(state[r]) + eps)           (the state AFTER this lookup's addition)
 *   grad_per_sample_weights[p] = <weights[r], g>            (the row as it is at that moment)
 *   weights[r] -= mult * g                                  (stored in the weights' type each time)
 * The reference runs all bags at once with plain loads and stores, so its result is only defined
 * when no row occurs twice in the batch (all its test draws, test_table_batched_embeddings.py:244).
 * Here the lookups of a row are applied one at a time in ascending position (table-major bag
 * order, then the order inside the bag): the reference's arithmetic executed serially.  The two
 * agree whenever the reference's result is defined; when rows repeat this library returns the
 * serial result, deterministically.  (fp32 / fp64 rows without per-sample weights: nothing
 * rounds the row between its lookups and nothing reads it, so a row of many lookups is written
 * once, as row - sum_k mult_k * g_k with the sum taken in a fixed tree order -- the serial result
 * up to the rounding of the additions.)  With stochastic_rounding (fp16 only) the k-th update of a
 * row within the call draws its bits with the Philox key seed ^ (k * 0x9E3779B97F4A7C15): k = 0
 * is the stream of tbe_backward_exact_adagrad_stochastic.  Arguments as in
 * tbe_backward_exact_adagrad_stochastic.
 */
TBE_API int tbe_backward_approx_adagrad(const void *grad_output, void *weights, int32_t dtype,
                                        int64_t total_rows, int64_t max_table_rows, int32_t D,
                                        const int32_t *table_offsets, int32_t T,
                                        const int32_t *indices, int64_t num_indices,
                                        const int32_t *offsets, int32_t B,
                                        const void *per_sample_weights, void *optimizer_state,
                                        float learning_rate, float eps,
                                        void *grad_per_sample_weights,
                                        int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                        void *workspace, uint64_t workspace_bytes, void *stream);

/* The backward in two calls, so that the integer half can overlap other work.
 * tbe_plan_batch runs the stages that depend on the indices only -- gradient rows, sort, run
 * boundaries (table_batched_embeddings_cuda.cu:1618-1655 and the head test :1523-1539) -- and
 * leaves the result in `workspace`; it may run on another stream than the forward, while the
 * forward gathers.  tbe_backward_planned runs the gradient reduction and the optimizer
 * (kernel :1499-1587) on that workspace once `grad_output` exists; `stream` must be ordered
 * after the plan (e.g. by an event).  Together they equal tbe_backward_sgd /
 * tbe_backward_exact_adagrad(_stochastic); optimizer is TBE_OPT_SGD or TBE_OPT_ROWWISE_ADAGRAD.
 * A plan serves ONE tbe_backward_planned call (the update fills the queue counters that the plan
 * left at zero); plan again for the next batch or the next update.
 */
TBE_API int tbe_plan_batch(const int32_t *table_offsets, int32_t T,
                           const int32_t *indices, int64_t num_indices,
                           const int32_t *offsets, int32_t B, int64_t total_rows,
                           int64_t max_table_rows, int32_t D, int32_t dtype,
                           void *workspace, uint64_t workspace_bytes, void *stream);

TBE_API int tbe_backward_planned(int32_t optimizer, const void *grad_output, void *weights, int32_t dtype,
                                 int64_t total_rows, int32_t D, int32_t T, int32_t B, int64_t num_indices,
                                 const void *per_sample_weights, void *optimizer_state,
                                 float learning_rate, float eps, void *grad_per_sample_weights,
                                 int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                 void *workspace, uint64_t workspace_bytes, void *stream);

/* tbe_backward_exact_adagrad with fp16 stochastic rounding of the updated weights
 * (StochasticRoundingAdaGradFunctor, table_batched_embeddings_cuda.cu:618-646, and
 * stochastic_rounding_vector, :557-578: 13 random bits added to the fp32 pattern, then
 * truncation to fp16).  The reference draws its bits from cuRAND's Philox4_32_10 seeded from
 * PyTorch's generator per thread (:1685-1691); here element e of the table takes word e % 4 of
 * Philox4x32-10(counter = {e / 4, offset}, key = seed), so results are reproducible for a
 * given (seed, offset) and independent of launch geometry.  The two random streams differ,
 * so only the distribution -- not the bits -- matches the reference.  For dtypes other than
 * F16 the call equals tbe_backward_exact_adagrad.
 */
TBE_API int tbe_backward_exact_adagrad_stochastic(
    const void *grad_output, void *weights, int32_t dtype, int64_t total_rows,
    int64_t max_table_rows, int32_t D, const int32_t *table_offsets, int32_t T,
    const int32_t *indices, int64_t num_indices, const int32_t *offsets, int32_t B,
    const void *per_sample_weights, void *optimizer_state, float learning_rate, float eps,
    void *grad_per_sample_weights, uint64_t seed, uint64_t offset,
    void *workspace, uint64_t workspace_bytes, void *stream);

/* ------------------------------------------------- stages, individually callable
 * The backward entry points run exactly these stages on the caller's workspace.
 */

/* keys[p] = table_offsets[t] + indices[p]; grad_rows[p] = b*T + t
 * (linear_index_weight_offsets_kernel, table_batched_embeddings_cuda.cu:1471-1497;
 * IndexInfo.b_t = t*B + b is recoverable from grad_rows, indices_idx is p itself). */
TBE_API int tbe_linearize(const int32_t *table_offsets, int32_t T,
                  const int32_t *indices, int64_t num_indices,
                  const int32_t *offsets, int32_t B,
                  int32_t *keys, int32_t *grad_rows, void *stream);

/* Stable ascending LSD radix sort of (key, value) pairs on key bits [0, end_bit),
 * the contract of cub::DeviceRadixSort::SortPairs at
 * table_batched_embeddings_cuda.cu:1639-1655.  values_in == NULL sorts the
 * identity permutation (values_out = stable argsort).  Inputs are not modified. */
TBE_API uint64_t tbe_sort_workspace_bytes(int64_t n);
TBE_API int tbe_sort_pairs(const int32_t *keys_in, const int32_t *values_in,
                   int32_t *keys_out, int32_t *values_out,
                   int64_t n, int32_t end_bit,
                   void *workspace, uint64_t workspace_bytes, void *stream);

/* Run boundaries of a sorted key array: segment_starts[u] = first i with the
 * u-th distinct key, segment_starts[U] = n, *num_unique = U (device memory).
 * Same rule as the segment-head test at table_batched_embeddings_cuda.cu:1523-1539.
 * keys_sorted must be 16-byte aligned (it is read in 16-byte vectors). */
TBE_API uint64_t tbe_segments_workspace_bytes(int64_t n);
TBE_API int tbe_find_segments(const int32_t *keys_sorted, int64_t n,
                      int32_t *segment_starts, int32_t *num_unique,
                      void *workspace, uint64_t workspace_bytes, void *stream);

/* output[0] = 0; output[1 + t*B + b] = length of bag (t,b) given per-table bag
 * starts [T][B] and per-table totals [T]; the caller cumsums
 * (construct_offsets, table_batched_embeddings_cuda.cu:1165-1213,
 * table_batched_embeddings.cpp:67). */
TBE_API int tbe_construct_offsets(const int32_t *batch_offsets_per_table,
                          const int32_t *total_indices_per_table,
                          int32_t T, int32_t B, int32_t *output, void *stream);

/* Stage entry point for tests: out[i] = fp16 bit pattern of values[i] rounded stochastically with
 * the random word random_words[i], the element rule of stochastic_rounding_vector
 * (table_batched_embeddings_cuda.cu:564-578: the word's top 13 bits are added to the fp32 pattern,
 * the sum is converted toward zero) as every kernel here that rounds stochastically applies it. */
TBE_API int tbe_stochastic_round(const float *values, const uint32_t *random_words, uint16_t *out,
                                 int64_t n, void *stream);

/* ---------------------------------------------- per-table embedding dimension
 * The reference's MixedDim path (table_batched_embeddings_ops.py:204-435):
 *   weights            1-D; table t occupies elements [table_offsets[t], table_offsets[t+1]),
 *                      row-major [rows_t][D_t]                         int64 [T+1]
 *   table_dim_offsets  first global row id of each table (cumulative ROW counts) int32 [T+1]
 *   dim_offsets        first output column of each table, D_t % 4 == 0  int32 [T+1]
 *   output / grad      [B][total_D]
 * `fp16_vector_width` is 8 when every D_t of an fp16 table set is a multiple of 8, else 4
 * (ignored for other dtypes).
 * tbe_forward_mixed replaces batched_embedding_forward_mixed_D_cuda
 * (table_batched_embeddings_cuda.cu:945-1004, "forward_mixed_D" in table_batched_embeddings.cpp:66);
 * tbe_backward_mixed replaces batched_embedding_backward_adagrad_exact_mixed_D_cuda
 * (:1350-1469, "backward_exact_adagrad_mixed_D", .cpp:64), with TBE_OPT_APPROX_ROWWISE_ADAGRAD
 * batched_embedding_backward_adagrad_approx_mixed_D_cuda (:1076-1163, .cpp:63; semantics of
 * tbe_backward_approx_adagrad), and adds exact SGD; per-sample weights as in tbe_backward_exact_adagrad;
 * stochastic_rounding / seed / offset as in tbe_backward_exact_adagrad_stochastic;
 * max_table_rows as in tbe_backward_sgd (0 = unknown).  The
 * workspace is a backward workspace laid out by tbe_backward_mixed_workspace_layout (its partial
 * rows hold the widest row that is summed in chunks: 64 vectors).
 * grad_output may hold at most 2^31 - 1 elements (B * total_D), so that the element offset of a
 * gradient row fits 32 bits.
 */
TBE_API int tbe_forward_mixed(const void *weights, int32_t dtype, int32_t fp16_vector_width,
                              const int64_t *table_offsets, const int32_t *dim_offsets,
                              int32_t total_D, int32_t T,
                              const int32_t *indices, int64_t num_indices,
                              const int32_t *offsets, int32_t B,
                              const void *per_sample_weights, void *output, void *stream);

TBE_API int tbe_backward_mixed_workspace_layout(int64_t num_indices, int32_t dtype, int32_t T,
                                                tbe_workspace_layout_t *layout);

TBE_API int tbe_backward_mixed(int32_t optimizer, const void *grad_output, void *weights, int32_t dtype,
                               int32_t fp16_vector_width, int64_t total_rows, int64_t max_table_rows,
                               const int64_t *table_offsets, const int32_t *table_dim_offsets,
                               const int32_t *dim_offsets, int32_t total_D, int32_t T,
                               const int32_t *indices, int64_t num_indices,
                               const int32_t *offsets, int32_t B,
                               const void *per_sample_weights, void *optimizer_state,
                               float learning_rate, float eps, void *grad_per_sample_weights,
                               int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                               void *workspace, uint64_t workspace_bytes, void *stream);

/* ---------------------------------------------------------------- row cache
 * An HBM-resident set-associative row cache in front of a host-resident table
 * (pinned, device-mapped memory from tbe_host_mapped_alloc).  The reference has
 * no cache: its only host-table mechanism is managed / mapped memory read over
 * the bus on every lookup (table_batched_embeddings_cuda.cu:795-880,
 * EmbeddingLocation.HOST_MAPPED in table_batched_embeddings_ops.py:130-167).
 * Semantics are this library's own and are restated by oracle/lxu_cache_model.c.
 *
 * Geometry: num_sets sets of TBE_CACHE_WAYS = 64 slots; set = mix(key) scaled to
 * [0, num_sets) with a fixed 32-bit integer hash; one wavefront probes a set with
 * one coalesced tag load and a ballot.  All state lives in caller-owned device
 * arrays.  One call of tbe_cache_prepare per step (steps are numbered from 1):
 *   1. the batch is linearized, sorted and cut into unique rows (ascending key);
 *   2. every unique row probes its set; hits record their slot and are marked
 *      used in this step (last_used = step, use_count += 1);
 *   3. the missing rows of a set are inserted in ascending key order; the victim
 *      is the slot with the smallest (priority, way) among slots not used in this
 *      step, priority = last_used (LRU) or use_count (LFU); empty slots (priority 0)
 *      go first; if every slot of the set was used in this step the row is *staged*:
 *      it gets a row of the staging area that follows the slots in `rows` (index
 *      num_sets * 64 + s, s < stage_slots) for this step only, without a tag; when the
 *      staging area is exhausted (or stage_slots is 0) the row stays uncached for the
 *      step and is read / updated in the backing table directly;
 *   4. on the side stream, evicted rows are written back to the backing table and
 *      the inserted and the staged rows are fetched into their slots (every resident row counts
 *      as dirty: the optimizer updates each row it looks up); the side stream is
 *      joined to `stream` by an event before the call returns control of `stream`
 *      to the caller's next kernel;
 *   5. unique_slots[u] / lookup_slots[p] tell the forward and backward kernels
 *      where each row lives (slot >= 0, or -1 = backing table);
 *   6. tbe_backward_cached, after the update, copies the staged rows back to the
 *      backing table.  A staged row thus crosses the host link once in each
 *      direction per step, however many lookups hit it (an uncached row is read
 *      once per lookup in the forward and read and written once in the backward).
 * Deferred write-back (stage_of_row given) takes the row traffic out of the step, so that the plan
 * of the next step can be made, and most of its rows moved, while the current step computes
 * (tbe_cache_plan / tbe_cache_commit; tbe_cache_prepare is the two in a row).  `rows` then holds
 * THREE staging areas that take turns by the call's `sequence` number (area = sequence mod 3):
 *   - the decisions (1-3, 5) touch no row, so they may run as soon as the previous call's have;
 *   - a staged row is fetched into its staging row and stays there after the update; an inserted
 *     row is fetched into a *landing row* of the same area (its slot may still serve the step
 *     before), and tbe_cache_commit swaps slot and landing row, so the evicted row ends up in the
 *     staging area as well;
 *   - whatever a staging area holds two calls later, and no later step has fetched again from
 *     there (HBM to HBM, marked in stage_keys), goes back to the backing table in that call's fill
 *     launch, beside its fetches: both directions of the host link are busy at once, and nothing
 *     on the link waits for a step's kernels;
 *   - tbe_cache_commit, on the caller's stream after the update of the step before, does what
 *     depends on that update: fetches from the staging area of the step before, the swaps, and the
 *     rare rows that found neither slot nor staging row nor landing row (those move over the link
 *     on the caller's stream).
 * tbe_cache_flush writes back whatever is still pending.  Until then the backing table's copy of a
 * staged or evicted row is stale, like that of a cached row.
 * The resulting tags / slots are a pure function of the key sequence, so a CPU
 * model can reproduce them bit for bit (a staged row is an uncached row of the
 * model; its staging index is the rank of the miss inside its set plus the number
 * of misses of the sets before it, so it is reproducible too).
 */
#define TBE_CACHE_WAYS 64
enum { TBE_CACHE_LRU = 0, TBE_CACHE_LFU = 1 };

typedef struct tbe_cache {
  int32_t *tags;        /* [num_sets * 64] key of the row held by each slot, -1 = empty  */
  int32_t *last_used;   /* [num_sets * 64] step of the slot's last use, 0 = never        */
  int32_t *use_count;   /* [num_sets * 64] steps that used the row since it was inserted */
  void *rows;           /* [num_sets * 64 + stage_slots][D] cached rows, then the staging area
                         * (three areas, [num_sets * 64 + 3 * stage_slots][D], with deferred write-back) */
  void *backing_rows;   /* device-visible address of the backing table [total_rows][D]   */
  int64_t num_sets;
  int32_t policy;       /* TBE_CACHE_LRU or TBE_CACHE_LFU                                */
  int64_t stage_slots;  /* rows of the staging area (0 = none); num_sets * 64 + stage_slots < 2^31 */
  /* deferred write-back (all null / 0: staged rows go back right after the update) */
  int32_t *stage_of_row;  /* [total_rows] row of `rows` (a staging row) that holds the row's newest value and
                           * owes it to the backing table, -1 = none, < -1 = none, and the backing row is
                           * written on the caller's stream in the step with sequence -(value + 2)      */
  int32_t *stage_keys;    /* [3 * stage_slots] key held by each staging row, -1 = none, -(key + 2) = taken
                           * over by a later step                                                       */
  int64_t total_rows;     /* rows of the backing table                                                 */
  /* tables of different row widths (all null / 0: every row has the D elements passed to the calls).
   * backing_rows is then the 1-D weights of tbe_forward_mixed, a row's key its global row id
   * (mixed_table_rows[t] + index), a row of `rows` has the widest table's D_t elements -- the D passed
   * to the calls below -- of which a narrower row uses the first D_t, and `workspace` follows
   * tbe_backward_mixed_workspace_layout.  Forward and update: tbe_forward_mixed_cached,
   * tbe_backward_mixed_cached. */
  const int64_t *mixed_table_offsets;  /* [T + 1] first element of each table in backing_rows             */
  const int32_t *mixed_table_rows;     /* [T + 1] first global row id of each table (`table_dim_offsets`) */
  const int32_t *mixed_dim_offsets;    /* [T + 1] first output column of each table                       */
  int32_t mixed_T;
} tbe_cache_t;

/* Byte offsets into the cache workspace (separate from the backward workspace). */
typedef struct tbe_cache_workspace_layout {
  uint64_t total_bytes;
  uint64_t unique_slots;   /* int32 [U]  slot of each unique row (>= num_sets * 64: staged), -1 = backing table */
  uint64_t lookup_slots;   /* int32 [N]  the same, per lookup position                         */
  uint64_t evicted_keys;   /* int32 [U]  -2 untouched, -1 filled an empty or staging slot, >= 0 key written back */
  uint64_t miss_sets;      /* int32 [U]  set of each missing row (num_sets: the row is resident) */
  uint64_t miss_list;      /* int32 [U]  missing rows grouped by set, ascending inside a set   */
  uint64_t set_counts;     /* int32 [num_sets] misses per set                                  */
  uint64_t set_fill;       /* int32 [num_sets]  (not used)                                     */
  uint64_t set_starts;     /* int32 [num_sets + 1]                                             */
  uint64_t stats;          /* int32 [16]: unique rows, hits, misses, inserted, evicted (slots that held a row),
                            * uncached, staged; with deferred write-back also: fetched from a staging row,
                            * rows the fill launch writes to the backing table, fetches left to
                            * tbe_cache_commit, inserted rows without a landing row                */
  uint64_t fetch_source;   /* int32 [U]  deferred write-back: row of `rows` a fetched row comes from, -1 = backing
                            * table, -3 = backing table, by tbe_cache_commit                     */
  uint64_t landing;        /* int32 [U]  deferred write-back: landing row of an inserted row, -1 = none */
  uint64_t write_out;      /* int32 [stage_slots]  deferred write-back: key that each row of the released
                            * staging area owes to the backing table, -1 = none                  */
} tbe_cache_workspace_layout_t;

TBE_API int tbe_cache_workspace_layout(int64_t num_indices, int64_t num_sets, int64_t stage_slots,
                                       tbe_cache_workspace_layout_t *layout);

/* Empties the cache: tags = -1, last_used = use_count = 0 (and stage_of_row = stage_keys = -1: rows that
 * still wait in a staging area are dropped, so flush first to keep them). */
TBE_API int tbe_cache_init(const tbe_cache_t *cache, void *stream);

/* Steps 1-5 above.  `workspace` is a backward workspace (tbe_backward_workspace_layout)
 * and keeps the batch's plan for tbe_backward_cached; `cache_workspace` follows
 * tbe_cache_workspace_layout.  `side_stream` must differ from `stream`.  `step` stamps the recency
 * words and only has to grow from call to call.  `sequence` selects the staging area of deferred
 * write-back: successive calls must pass consecutive numbers (after tbe_cache_init, or a
 * tbe_cache_flush that left no staging area listed, any number may follow); it is ignored otherwise. */
TBE_API int tbe_cache_prepare(const tbe_cache_t *cache, int32_t dtype, int64_t total_rows,
                              int64_t max_table_rows, int32_t D,
                              const int32_t *table_offsets, int32_t T,
                              const int32_t *indices, int64_t num_indices,
                              const int32_t *offsets, int32_t B, int32_t step, int32_t sequence,
                              void *workspace, uint64_t workspace_bytes,
                              void *cache_workspace, uint64_t cache_workspace_bytes,
                              void *stream, void *side_stream);

/* tbe_cache_prepare in two parts, for deferred write-back only, so that a batch can be planned
 * while the batch before it still computes.  tbe_cache_plan makes the decisions on `plan_stream`
 * and then, on `link_stream`, moves the rows that do not depend on the step before;
 * tbe_cache_commit finishes the step on the stream that runs the forward and backward kernels.
 * Ordering is the caller's: a plan's kernels must follow (a) the previous call's tbe_cache_plan,
 * (b) the tbe_cache_commit of the batch two calls back and (c) the last use of the two
 * workspaces; tbe_cache_commit of a batch must follow its tbe_cache_plan on both streams, the
 * update of the batch before it, and precede its own forward.  With the calls of one cache issued
 * in batch order from one host thread on one stream, that is: make `plan_stream` wait for that
 * stream when tbe_cache_plan is called, and make that stream wait for `link_stream` before
 * tbe_cache_commit.  The workspaces of a planned batch must stay untouched until its backward. */
TBE_API int tbe_cache_plan(const tbe_cache_t *cache, int32_t dtype, int64_t total_rows,
                           int64_t max_table_rows, int32_t D,
                           const int32_t *table_offsets, int32_t T,
                           const int32_t *indices, int64_t num_indices,
                           const int32_t *offsets, int32_t B, int32_t step, int32_t sequence,
                           void *workspace, uint64_t workspace_bytes,
                           void *cache_workspace, uint64_t cache_workspace_bytes,
                           void *plan_stream, void *link_stream);
TBE_API int tbe_cache_commit(const tbe_cache_t *cache, int32_t dtype, int32_t D, int32_t T,
                             int64_t num_indices, int32_t sequence,
                             void *workspace, uint64_t workspace_bytes,
                             void *cache_workspace, uint64_t cache_workspace_bytes, void *stream);

/* tbe_forward with every row read through lookup_slots (cache slot or backing table). */
TBE_API int tbe_forward_cached(const tbe_cache_t *cache, int32_t dtype, int32_t D,
                               const int32_t *table_offsets, int32_t T,
                               const int32_t *indices, int64_t num_indices,
                               const int32_t *offsets, int32_t B,
                               const void *per_sample_weights, const int32_t *lookup_slots,
                               void *output, void *stream);

/* The fused update of tbe_backward_sgd / tbe_backward_exact_adagrad(_stochastic) on the plan
 * that tbe_cache_prepare left in `workspace`, updating each row where it lives; staged rows are
 * then copied back to the backing table.  stochastic_rounding / seed / offset as in
 * tbe_backward_exact_adagrad_stochastic: the random word of a weight depends on its place in the
 * table, not on where the row currently lives, so a cached run equals an uncached one. */
TBE_API int tbe_backward_cached(int32_t optimizer, const void *grad_output, const tbe_cache_t *cache,
                                int32_t dtype, int64_t total_rows, int32_t D, int32_t T, int32_t B,
                                int64_t num_indices, const void *per_sample_weights,
                                void *optimizer_state, float learning_rate, float eps,
                                void *grad_per_sample_weights,
                                int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                void *workspace, uint64_t workspace_bytes,
                                const int32_t *unique_slots, void *stream);

/* tbe_backward_approx_adagrad (the per-lookup row-wise Adagrad of
 * batched_embedding_backward_adagrad_approx_cuda, table_batched_embeddings_cuda.cu:706-793) on the plan
 * that tbe_cache_prepare left in `workspace`, every row updated where it lives; `offsets` are the
 * batch's bag offsets [T*B + 1] again (the plan does not keep them).  Same result, bit for bit, as the
 * uncached entry point on the backing table. */
TBE_API int tbe_backward_approx_cached(const void *grad_output, const tbe_cache_t *cache, int32_t dtype,
                                       int64_t total_rows, int32_t D, int32_t T, int32_t B,
                                       int64_t num_indices, const int32_t *offsets,
                                       const void *per_sample_weights, void *optimizer_state,
                                       float learning_rate, float eps, void *grad_per_sample_weights,
                                       int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                       void *workspace, uint64_t workspace_bytes,
                                       const int32_t *unique_slots, void *stream);

/* tbe_forward_mixed and tbe_backward_mixed (every optimizer of it) for tables of different widths
 * behind the row cache: `cache` carries the tables (mixed_* fields), D is the width of a cache row
 * (the widest table's), the other arguments are those of the uncached entry points; `offsets` are the
 * batch's bag offsets [T*B + 1] again, read by TBE_OPT_APPROX_ROWWISE_ADAGRAD only (null otherwise).  The plan comes from tbe_cache_prepare / tbe_cache_plan + tbe_cache_commit called with
 * table_offsets = mixed_table_rows, T = mixed_T and a workspace laid out by
 * tbe_backward_mixed_workspace_layout.  Same results, bit for bit, as the uncached entry points on the
 * backing table (stochastic rounding included: a weight's random word goes by its place in the table).
 * The reference has no counterpart (its mixed-D tables are device or managed memory,
 * table_batched_embeddings_ops.py:324-379). */
TBE_API int tbe_forward_mixed_cached(const tbe_cache_t *cache, int32_t dtype, int32_t fp16_vector_width, int32_t D,
                                     int32_t total_D, const int32_t *indices, int64_t num_indices,
                                     const int32_t *offsets, int32_t B, const void *per_sample_weights,
                                     const int32_t *lookup_slots, void *output, void *stream);
TBE_API int tbe_backward_mixed_cached(int32_t optimizer, const void *grad_output, const tbe_cache_t *cache,
                                      int32_t dtype, int32_t fp16_vector_width, int32_t D, int32_t total_D,
                                      int32_t B, int64_t num_indices, const int32_t *offsets,
                                      const void *per_sample_weights,
                                      void *optimizer_state, float learning_rate, float eps,
                                      void *grad_per_sample_weights, int32_t stochastic_rounding, uint64_t seed,
                                      uint64_t offset, void *workspace, uint64_t workspace_bytes,
                                      const int32_t *unique_slots, void *stream);

/* Writes every resident row, and every row waiting in a staging area, back to the backing table (the
 * cache stays valid).  `stream` must be ordered behind the streams of earlier tbe_cache_plan calls, and a
 * planned batch must have been committed.  Deferred write-back: the last `live_sequences` planned batches
 * (sequence numbers last_sequence, last_sequence - 1, ...) have not had their update yet; their staging
 * areas are written out as they are and stay listed, because that update changes their rows again.  With
 * live_sequences = 0 every staging area is empty afterwards and any sequence number may follow. */
TBE_API int tbe_cache_flush(const tbe_cache_t *cache, int32_t dtype, int32_t D, uint32_t live_sequences,
                            int32_t last_sequence, void *stream);

/* ------------------------------------------------- interleaved [E][T][D] tables
 * The older sparse_embedding_cuda kernels keep all tables in one [E][T][D] array, number bags
 * bag-major (b*T + t) and bound bag (b, t) by two consecutive entries of an offsets array that is
 * either flat [B*T+1] or [B][T+1] with offsets[b][T] == offsets[b+1][0]
 * (sparse_embedding_cuda_kernel.cu:221-284 forward_offsets, :349-462 forward / forward_fast,
 * :286-347 and :464-583 the fused updates; bound in sparse_embedding_cuda.cpp:255-322).
 * offsets_row_stride = T for the flat form (dense [B][T][L] indices: offsets[i] = i*L), T + 1 for
 * the [B][T+1] form.  The table-major kernels serve this layout through a row stride: the row of
 * a lookup in the [E*T][D] view is idx*T + t, output and gradient are [B][T][D].  No index array
 * is rewritten and nothing is allocated.
 *
 * tbe_forward_interleaved replaces sparse_embedding_cuda_forward_single / _fast_single / _offsets.
 * tbe_backward_sgd_interleaved replaces sparse_embedding_cuda_backward_update_single / _fast_single /
 * _offsets, made exact: every distinct row receives -lr * (sum of its gradients) once, where the
 * reference's `weights[ind][t][d] -= lr * g` races on repeats (sparse_embedding_cuda_kernel.cu:493-497).
 * Its workspace follows tbe_backward_interleaved_workspace_layout (at most 2048 tables): the lookups of a
 * table are not consecutive positions here, so one pass first copies the indices into table-major
 * order (kept in the layout's `keys` region); the batch is then sorted table by table and updated
 * like a table-major one, with idx*T + t as the row of a lookup.  positions_sorted refers to that
 * table-major order.
 */
TBE_API int tbe_forward_interleaved(const void *weights, int32_t dtype, int64_t E, int32_t T, int32_t D,
                                    const int32_t *indices, int64_t num_indices,
                                    const int32_t *offsets, int32_t offsets_row_stride, int32_t B,
                                    void *output, void *stream);
TBE_API int tbe_backward_interleaved_workspace_layout(int64_t num_indices, int32_t D, int32_t dtype,
                                                      int32_t T, int32_t B, tbe_workspace_layout_t *layout);
TBE_API int tbe_backward_sgd_interleaved(const void *grad_output, void *weights, int32_t dtype, int64_t E,
                                         int32_t T, int32_t D, const int32_t *indices, int64_t num_indices,
                                         const int32_t *offsets, int32_t offsets_row_stride, int32_t B,
                                         float learning_rate, void *workspace, uint64_t workspace_bytes,
                                         void *stream);

/* ------------------------------------------------------ host-resident tables
 * Pinned, device-mapped host memory (new_host_mapped_tensor,
 * table_batched_embeddings_cuda.cu:820-880) and managed memory preferring the
 * host (new_managed_tensor, :797-871).  *device_ptr is the address kernels use.
 */
TBE_API int tbe_host_mapped_alloc(uint64_t bytes, void **host_ptr, void **device_ptr);
TBE_API int tbe_host_mapped_free(void *host_ptr);
TBE_API int tbe_managed_alloc(uint64_t bytes, int32_t device, void **ptr);
TBE_API int tbe_managed_free(void *ptr);

#ifdef __cplusplus
}
#endif
#endif /* TBE_HIP_H */
