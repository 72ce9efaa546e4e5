// Fused backward entry points: linearize -> stable radix sort -> run boundaries
// -> per-row gradient reduction + optimizer, all on the caller's stream and
// workspace, with no host synchronisation.  Pipeline shape follows
// batched_embedding_backward_adagrad_exact_cuda
// (table_batched_embeddings_cuda.cu:1589-1706); SGD uses the same pipeline so
// that repeated rows are updated exactly once.

#include <math.h>

#include <mutex>

#include "tbe_stages.h"

namespace tbe {
namespace {

// Number of low key bits that can be set when keys are < total_rows.  The
// reference sorts int(log2(total_rows) + 1) bits (tbe.cu:1643), which is the
// same quantity for every total_rows >= 1.
int key_bits(int64_t total_rows) {
  int bits = 0;
  while (bits < 32 && (int64_t{1} << bits) <= total_rows) ++bits;
  return bits;
}

// Every table is sorted on its own as long as there are at most this many: each table costs the
// sort a (possibly nearly empty) tile and 20 KB of counters.  A batch over more tables than that
// sorts the linearized keys in one piece, like the reference (tbe.cu:1639-1655).
constexpr int32_t kMaxTablesSortedApart = 2048;
inline int32_t sort_tables(int32_t T) { return T <= kMaxTablesSortedApart ? T : 1; }

// interleaved_B > 0 (tables stored [E][T][D], B bags per table): the `keys` region holds the batch in
// table-major order instead -- indices [n], offsets [T*B+1], then small scratch (interleaved_regions()).
void compute_layout(int64_t n, int32_t D, int32_t dtype, int32_t T, tbe_workspace_layout_t *l,
                    int32_t interleaved_B = 0) {
  const uint64_t nn = static_cast<uint64_t>(n > 0 ? n : 1);
  const uint64_t ints = align_up(nn * 4, 256);
  // a segment enters the chunk queue when it has more than kShortSegment occurrences and owns
  // partial rows when it has more than kChunkLen
  // (one list per XCD: the segments of several chunks that start in its eighth of the sorted positions)
  l->max_long_segments = static_cast<int64_t>(kNumXcd * long_list_capacity(static_cast<int64_t>(nn)));
  l->max_chunks = static_cast<int64_t>(kNumXcd * chunk_queue_capacity(static_cast<int64_t>(nn)));
  // (a partial row's number follows from where its chunk lies, two per kChunkLen sorted positions)
  l->max_partial_rows = static_cast<int64_t>(2 * (nn / kChunkLen + 1));
  uint64_t off = 0;
  // the linearized keys are only written (and sorted in one piece) for more tables than are sorted apart
  l->keys = off;
  if (interleaved_B > 0)
    off += ints + align_up((static_cast<uint64_t>(T) * interleaved_B + 1) * 4, 256) + 2 * align_up(T * 4ull, 256) +
           align_up(static_cast<uint64_t>(T) * interleaved_chunks_per_table(interleaved_B) * 4, 256);
  else
    off += sort_tables(T) == T ? 256 : ints;
  l->grad_rows = off; off += ints;
  l->keys_sorted = off; off += ints;
  l->positions_sorted = off; off += ints;
  l->segment_starts = off; off += align_up((nn + 1) * 4, 256);
  l->num_unique = off; off += align_up(static_cast<uint64_t>(kNumCounters) * 4, 256);
  l->sort_scratch = off; off += align_up(sort_workspace_bytes(n, sort_tables(T)), 256);
  l->segment_scratch = off; off += align_up(segments_workspace_bytes(n), 256);
  l->segment_ids = off; off += ints;
  l->long_segments = off; off += align_up(static_cast<uint64_t>(l->max_long_segments) * 16, 256);
  l->chunk_segments = off; off += align_up(static_cast<uint64_t>(l->max_chunks) * 32, 256);
  l->partial_sums = off;
  off += align_up(static_cast<uint64_t>(l->max_partial_rows) * static_cast<uint64_t>(D) * acc_size(dtype), 256);
  l->total_bytes = off;
}

}  // namespace

int key_bits_for(int64_t total_rows) { return key_bits(total_rows); }

namespace {
// The pieces of the `keys` region of an interleaved-tables layout.
struct InterleavedRegions {
  int32_t *indices_tm, *offsets_tm, *totals, *bias, *chunk_sums;
};
InterleavedRegions interleaved_regions(const tbe_workspace_layout_t &l, void *workspace, int64_t n, int32_t T,
                                       int32_t B) {
  char *base = static_cast<char *>(workspace) + l.keys;
  const uint64_t nn = static_cast<uint64_t>(n > 0 ? n : 1);
  InterleavedRegions r;
  r.indices_tm = reinterpret_cast<int32_t *>(base);
  base += align_up(nn * 4, 256);
  r.offsets_tm = reinterpret_cast<int32_t *>(base);
  base += align_up((static_cast<uint64_t>(T) * B + 1) * 4, 256);
  r.totals = reinterpret_cast<int32_t *>(base);
  base += align_up(T * 4ull, 256);
  r.bias = reinterpret_cast<int32_t *>(base);
  base += align_up(T * 4ull, 256);
  r.chunk_sums = reinterpret_cast<int32_t *>(base);
  return r;
}
}  // namespace

void backward_layout(int64_t n, int32_t D, int32_t dtype, int32_t T, tbe_workspace_layout_t *l) {
  compute_layout(n, D, dtype, T, l);
}

// sort_batch: gradient rows and the sort; build_plan: also the run boundaries (and the segment of
// every sorted position), into the workspace regions of `l`.  The lookups of a table are
// consecutive, so the (table, row) order of the reference's sort (tbe.cu:1639-1655) is reached by
// sorting every table's indices on their own; the last pass adds the table's first row, and
// keys_sorted / positions_sorted come out as the sort of the linearized keys would leave them.
// The `keys` region stays unwritten, unless the batch has more than kMaxTablesSortedApart tables:
// then the linearized keys are written there and sorted in one piece.
int sort_batch(const tbe_workspace_layout_t &l, void *workspace, const int32_t *table_offsets, int32_t T,
               const int32_t *indices, int64_t n, const int32_t *offsets, int32_t B, int64_t total_rows,
               int64_t max_table_rows, hipStream_t stream, int32_t interleaved_offsets_stride) {
  char *ws = static_cast<char *>(workspace);
  int32_t *keys_sorted = reinterpret_cast<int32_t *>(ws + l.keys_sorted);
  int32_t *positions_sorted = reinterpret_cast<int32_t *>(ws + l.positions_sorted);
  int32_t *grad_rows = reinterpret_cast<int32_t *>(ws + l.grad_rows);
  if (interleaved_offsets_stride > 0) {
    // Tables stored [E][T][D], bags b*T + t: the batch is put into table-major order first (one pass
    // over the indices), then sorted table by table like any other; a key leaves the last pass as
    // idx*T + t, the row of the [E*T][D] view.  Positions are those of the table-major order.
    const InterleavedRegions r = interleaved_regions(l, workspace, n, T, B);
    const int rc = interleaved_to_table_major(indices, offsets, interleaved_offsets_stride, T, B, r.totals, r.bias,
                                              r.chunk_sums, r.offsets_tm, r.indices_tm, stream);
    if (rc) return rc;
    SortTables tables{r.offsets_tm, B, T, r.bias, grad_rows};
    tables.key_mul = T;
    return sort_pairs(r.indices_tm, nullptr, keys_sorted, positions_sorted, n, key_bits(total_rows / T),
                      ws + l.sort_scratch, stream, &tables);
  }
  if (sort_tables(T) != T) {
    int32_t *keys = reinterpret_cast<int32_t *>(ws + l.keys);
    const int rc = linearize(table_offsets, T, indices, offsets, B, keys, grad_rows, stream);
    if (rc) return rc;
    return sort_pairs(keys, nullptr, keys_sorted, positions_sorted, n, key_bits(total_rows), ws + l.sort_scratch,
                      stream, nullptr);
  }
  const int64_t largest = (max_table_rows > 0 && max_table_rows < total_rows) ? max_table_rows : total_rows;
  // (the gradient row of every position is recorded by the sort's first launch)
  const SortTables tables{offsets, B, T, table_offsets, grad_rows};
  return sort_pairs(indices, nullptr, keys_sorted, positions_sorted, n, key_bits(largest), ws + l.sort_scratch,
                    stream, &tables);
}

int build_plan(const tbe_workspace_layout_t &l, void *workspace, const int32_t *table_offsets,
               int32_t T, const int32_t *indices, int64_t n, const int32_t *offsets, int32_t B,
               int64_t total_rows, int64_t max_table_rows, hipStream_t stream,
               int32_t interleaved_offsets_stride) {
  char *ws = static_cast<char *>(workspace);
  const int rc = sort_batch(l, workspace, table_offsets, T, indices, n, offsets, B, total_rows, max_table_rows,
                            stream, interleaved_offsets_stride);
  if (rc) return rc;
  return find_segments(reinterpret_cast<int32_t *>(ws + l.keys_sorted), n,
                       reinterpret_cast<int32_t *>(ws + l.segment_starts),
                       reinterpret_cast<int32_t *>(ws + l.num_unique),
                       reinterpret_cast<int32_t *>(ws + l.segment_ids), ws + l.segment_scratch,
                       stream, /*clear_queue_counters=*/true);
}

namespace {

struct BackwardCall {
  const void *grad_output;
  void *weights;
  int32_t dtype;
  int64_t total_rows;
  int64_t max_table_rows;
  int32_t D;
  const int32_t *table_offsets;
  int32_t T;
  const int32_t *indices;
  int64_t num_indices;
  const int32_t *offsets;
  int32_t B;
  const void *psw;
  void *state;
  float lr;
  float eps;
  void *grad_psw;
  void *workspace;
  uint64_t workspace_bytes;
  hipStream_t stream;
  int optimizer;
  // cache-fronted tables: the plan already sits in the workspace, rows are resolved through slots
  bool planned;
  const int32_t *unique_slots;
  void *cache_rows;
  StochasticRounding stochastic_rounding;
  // interleaved tables [E][T][D]: entries of `offsets` per b (T or T + 1); 0 = table-major
  int32_t interleaved_offsets_stride = 0;
};

int run_backward(const char *name, const BackwardCall &c) {
  TBE_REQUIRE(c.T > 0, "%s: T must be positive (got %d)", name, c.T);
  TBE_REQUIRE(c.D > 0, "%s: D must be positive (got %d)", name, c.D);
  TBE_REQUIRE(c.B > 0, "%s: B must be positive (got %d)", name, c.B);
  TBE_REQUIRE(c.D % 4 == 0, "%s: D must be a multiple of 4 (got %d)", name, c.D);
  TBE_REQUIRE(c.dtype >= TBE_DTYPE_F32 && c.dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, c.dtype);
  TBE_REQUIRE(c.total_rows > 0 && c.total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(c.max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(c.num_indices >= 0 && c.num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(c.T) * c.B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(c.grad_output && c.weights, "%s: null pointer argument", name);
  TBE_REQUIRE(c.planned || ((c.table_offsets || c.interleaved_offsets_stride > 0) && c.offsets),
              "%s: null pointer argument", name);
  TBE_REQUIRE(c.planned || c.indices || c.num_indices == 0, "%s: indices is null but num_indices > 0", name);
  TBE_REQUIRE(c.optimizer == kOptSgd || c.state, "%s: optimizer_state is null", name);
  TBE_REQUIRE((c.psw == nullptr) == (c.grad_psw == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  if (c.num_indices == 0) return TBE_OK;

  tbe_workspace_layout_t l;
  compute_layout(c.num_indices, c.D, c.dtype, c.T, &l, c.interleaved_offsets_stride > 0 ? c.B : 0);
  if (!c.workspace || c.workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)c.workspace_bytes);
  char *ws = static_cast<char *>(c.workspace);
  int32_t *grad_rows = reinterpret_cast<int32_t *>(ws + l.grad_rows);
  int32_t *keys_sorted = reinterpret_cast<int32_t *>(ws + l.keys_sorted);
  int32_t *positions_sorted = reinterpret_cast<int32_t *>(ws + l.positions_sorted);
  int32_t *segment_starts = reinterpret_cast<int32_t *>(ws + l.segment_starts);
  int32_t *counters = reinterpret_cast<int32_t *>(ws + l.num_unique);

  if (!c.planned) {
    const int rc = build_plan(l, c.workspace, c.table_offsets, c.T, c.indices, c.num_indices,
                              c.offsets, c.B, c.total_rows, c.max_table_rows, c.stream,
                              c.interleaved_offsets_stride);
    if (rc) return rc;
  }

  UpdateArgs a;
  a.grad_output = c.grad_output;
  a.weights = c.weights;
  a.optimizer_state = c.state;
  a.per_sample_weights = c.psw;
  a.grad_per_sample_weights = c.grad_psw;
  a.keys_sorted = keys_sorted;
  a.positions_sorted = positions_sorted;
  a.grad_rows = grad_rows;
  a.segment_starts = segment_starts;
  a.counters = counters;
  a.segment_ids = reinterpret_cast<int32_t *>(ws + l.segment_ids);
  a.long_segments = ws + l.long_segments;
  a.chunk_segments = ws + l.chunk_segments;
  a.partial_sums = ws + l.partial_sums;
  a.unique_slots = c.unique_slots;
  a.cache_rows = c.cache_rows;
  a.num_indices = c.num_indices;
  a.max_long = l.max_long_segments;
  a.max_chunks = l.max_chunks;
  a.dtype = c.dtype;
  a.D = c.D;
  a.optimizer = c.optimizer;
  a.learning_rate = c.lr;
  a.eps = c.eps;
  a.stochastic_rounding = c.stochastic_rounding;
  return segment_update(a, c.stream);
}

}  // namespace
}  // namespace tbe

extern "C" int tbe_backward_workspace_layout(int64_t num_indices, int32_t D, int32_t dtype,
                                             int32_t T, tbe_workspace_layout_t *layout) {
  using namespace tbe;
  TBE_REQUIRE(layout, "tbe_backward_workspace_layout: null layout");
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX,
              "tbe_backward_workspace_layout: num_indices out of range");
  TBE_REQUIRE(D > 0 && D % 4 == 0, "tbe_backward_workspace_layout: D must be a positive multiple of 4 (got %d)", D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64,
              "tbe_backward_workspace_layout: bad dtype %d", dtype);
  TBE_REQUIRE(T > 0, "tbe_backward_workspace_layout: T must be positive (got %d)", T);
  compute_layout(num_indices, D, dtype, T, layout);
  return TBE_OK;
}

extern "C" int tbe_backward_interleaved_workspace_layout(int64_t num_indices, int32_t D, int32_t dtype, int32_t T,
                                                         int32_t B, tbe_workspace_layout_t *layout) {
  using namespace tbe;
  const char *name = "tbe_backward_interleaved_workspace_layout";
  TBE_REQUIRE(layout, "%s: null layout", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(T > 0 && B > 0 && static_cast<int64_t>(T) * B < INT32_MAX, "%s: bad T or B (got %d, %d)", name, T, B);
  compute_layout(num_indices, D, dtype, T, layout, B);
  return TBE_OK;
}

extern "C" int tbe_backward_sgd_interleaved(const void *grad_output, void *weights, int32_t dtype, int64_t E,
                                            int32_t T, int32_t D, const int32_t *indices, int64_t num_indices,
                                            const int32_t *offsets, int32_t offsets_row_stride, int32_t B,
                                            float learning_rate, void *workspace, uint64_t workspace_bytes,
                                            void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_sgd_interleaved";
  TBE_REQUIRE(E > 0 && T > 0 && E * T < INT32_MAX, "%s: E * T must fit a 32-bit row number", name);
  TBE_REQUIRE(offsets_row_stride == T || offsets_row_stride == T + 1,
              "%s: offsets_row_stride must be T (flat offsets) or T + 1 ([B][T+1] offsets), got %d", name,
              offsets_row_stride);
  if (T > kMaxTablesSortedApart)
    return fail(TBE_ERR_UNSUPPORTED, "%s: at most %d interleaved tables (got %d)", name, kMaxTablesSortedApart, T);
  // T tables of E rows: row idx*T + t of the [E*T][D] view, gradient row b*T + t of [B*T][D]
  BackwardCall c{grad_output, weights, dtype, E * T, 0, D, nullptr, T, indices, num_indices, offsets, B, nullptr,
                 nullptr, learning_rate, 0.0f, nullptr, workspace, workspace_bytes,
                 static_cast<hipStream_t>(stream), kOptSgd, false, nullptr, nullptr, StochasticRounding{0, 0, 0}};
  c.interleaved_offsets_stride = offsets_row_stride;
  return run_backward(name, c);
}

extern "C" int tbe_backward_sgd(const void *grad_output, void *weights, int32_t dtype,
                                int64_t total_rows, int64_t max_table_rows, int32_t D, const int32_t *table_offsets,
                                int32_t T, const int32_t *indices, int64_t num_indices,
                                const int32_t *offsets, int32_t B, float learning_rate,
                                void *workspace, uint64_t workspace_bytes, void *stream) {
  tbe::BackwardCall c{grad_output, weights, dtype, total_rows, max_table_rows, D, table_offsets, T, indices,
                      num_indices, offsets, B, nullptr, nullptr, learning_rate, 0.0f, nullptr,
                      workspace, workspace_bytes, static_cast<hipStream_t>(stream), tbe::kOptSgd,
                      false, nullptr, nullptr, tbe::StochasticRounding{0, 0, 0}};
  return tbe::run_backward("tbe_backward_sgd", c);
}

// ------------------------------------------------------------ library-held scratch
// tbe_backward_sgd_static runs tbe_backward_sgd's pipeline on this array instead of a caller's
// workspace, for callers that may not allocate.  The array belongs to the code object: every
// device the library runs on holds its own copy, at its own address, until the process ends.
// In host code the array's name is only a handle for hipGetSymbolAddress; the address kernels
// and layouts use is the one that call returns for the current device.
static __device__ __align__(256) unsigned char scratch[TBE_STATIC_SCRATCH_BYTES];

namespace tbe {
namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void *g_scratch_address[kMaxDevices] = {};  // per device, resolved on the first call there

// Device address of `scratch` on the current device.
int static_scratch(const char *name, void **address) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "%s: hipGetDevice: %s", name, hipGetErrorString(e));
  if (device < 0 || device >= kMaxDevices)
    return fail(TBE_ERR_UNSUPPORTED, "%s: device %d is beyond the %d devices tracked", name, device, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_address[device]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return fail(TBE_ERR_HIP, "%s: hipGetSymbolAddress(scratch) on device %d: %s", name, device,
                  hipGetErrorString(e));
    g_scratch_address[device] = p;
  }
  *address = g_scratch_address[device];
  return TBE_OK;
}
}  // namespace
}  // namespace tbe

extern "C" int tbe_backward_sgd_static(const void *grad_output, void *weights, int32_t dtype,
                                       int64_t total_rows, int64_t max_table_rows, int32_t D,
                                       const int32_t *table_offsets, int32_t T,
                                       const int32_t *indices, int64_t num_indices,
                                       const int32_t *offsets, int32_t B, float learning_rate,
                                       void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_sgd_static";
  // the layout query's own preconditions, so that a bad shape is reported as such and not as a size
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(T > 0, "%s: T must be positive (got %d)", name, T);
  tbe_workspace_layout_t l;
  compute_layout(num_indices, D, dtype, T, &l);
  if (l.total_bytes > TBE_STATIC_SCRATCH_BYTES)
    return fail(TBE_ERR_WORKSPACE,
                "%s: %lld lookups of %d tables need %llu bytes of scratch, the library holds %llu; "
                "use tbe_backward_sgd with a workspace of the caller's",
                name, (long long)num_indices, T, (unsigned long long)l.total_bytes,
                (unsigned long long)TBE_STATIC_SCRATCH_BYTES);
  void *address = nullptr;
  if (int rc = static_scratch(name, &address)) return rc;
  BackwardCall c{grad_output, weights, dtype, total_rows, max_table_rows, D, table_offsets, T, indices,
                 num_indices, offsets, B, nullptr, nullptr, learning_rate, 0.0f, nullptr,
                 address, TBE_STATIC_SCRATCH_BYTES, static_cast<hipStream_t>(stream), kOptSgd,
                 false, nullptr, nullptr, StochasticRounding{0, 0, 0}};
  return run_backward(name, c);
}

extern "C" int tbe_backward_exact_adagrad(const void *grad_output, void *weights, int32_t dtype,
                                          int64_t total_rows, int64_t max_table_rows, int32_t D,
                                          const int32_t *table_offsets, int32_t T,
                                          const int32_t *indices, int64_t num_indices,
                                          const int32_t *offsets, int32_t B,
                                          const void *per_sample_weights, void *optimizer_state,
                                          float learning_rate, float eps,
                                          void *grad_per_sample_weights, void *workspace,
                                          uint64_t workspace_bytes, void *stream) {
  tbe::BackwardCall c{grad_output, weights, dtype, total_rows, max_table_rows, D, table_offsets, T, indices,
                      num_indices, offsets, B, per_sample_weights, optimizer_state, learning_rate,
                      eps, grad_per_sample_weights, workspace, workspace_bytes,
                      static_cast<hipStream_t>(stream), tbe::kOptAdagrad, false, nullptr, nullptr,
                      tbe::StochasticRounding{0, 0, 0}};
  return tbe::run_backward("tbe_backward_exact_adagrad", c);
}

extern "C" int tbe_backward_exact_adagrad_stochastic(
    const void *grad_output, void *weights, int32_t dtype, int64_t total_rows,
    int64_t max_table_rows, int32_t D, const int32_t *table_offsets, int32_t T,
    const int32_t *indices, int64_t num_indices, const int32_t *offsets, int32_t B,
    const void *per_sample_weights, void *optimizer_state, float learning_rate, float eps,
    void *grad_per_sample_weights, uint64_t seed, uint64_t offset,
    void *workspace, uint64_t workspace_bytes, void *stream) {
  tbe::BackwardCall c{grad_output, weights, dtype, total_rows, max_table_rows, D, table_offsets, T, indices,
                      num_indices, offsets, B, per_sample_weights, optimizer_state, learning_rate,
                      eps, grad_per_sample_weights, workspace, workspace_bytes,
                      static_cast<hipStream_t>(stream), tbe::kOptAdagrad, false, nullptr, nullptr,
                      tbe::StochasticRounding{seed, offset, dtype == TBE_DTYPE_F16 ? 1 : 0}};
  return tbe::run_backward("tbe_backward_exact_adagrad_stochastic", c);
}

extern "C" int tbe_backward_cached(int32_t optimizer, const void *grad_output,
                                   const tbe_cache_t *cache, int32_t dtype, int64_t total_rows,
                                   int32_t D, int32_t T, int32_t B, int64_t num_indices,
                                   const void *per_sample_weights, void *optimizer_state,
                                   float learning_rate, float eps, void *grad_per_sample_weights,
                                   int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                   void *workspace, uint64_t workspace_bytes,
                                   const int32_t *unique_slots, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(cache && cache->rows && cache->backing_rows, "tbe_backward_cached: null cache");
  TBE_REQUIRE(optimizer == TBE_OPT_SGD || optimizer == TBE_OPT_ROWWISE_ADAGRAD,
              "tbe_backward_cached: bad optimizer %d", optimizer);
  TBE_REQUIRE(unique_slots || num_indices == 0, "tbe_backward_cached: null unique_slots");
  TBE_REQUIRE(optimizer != TBE_OPT_SGD || !per_sample_weights,
              "tbe_backward_cached: SGD takes no per-sample weights");
  BackwardCall c{grad_output, cache->backing_rows, dtype, total_rows, 0, D, nullptr, T, nullptr,
                 num_indices, nullptr, B, per_sample_weights, optimizer_state, learning_rate, eps,
                 grad_per_sample_weights, workspace, workspace_bytes,
                 static_cast<hipStream_t>(stream),
                 optimizer == TBE_OPT_SGD ? kOptSgd : kOptAdagrad, true, unique_slots, cache->rows,
                 StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0}};
  if (int rc = run_backward("tbe_backward_cached", c)) return rc;
  if (cache->stage_slots <= 0 || num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, D, dtype, T, &l);
  const char *ws = static_cast<const char *>(workspace);
  return cache_unstage(cache, dtype, D, reinterpret_cast<const int32_t *>(ws + l.keys_sorted),
                       reinterpret_cast<const int32_t *>(ws + l.segment_starts),
                       reinterpret_cast<const int32_t *>(ws + l.num_unique), unique_slots, num_indices,
                       static_cast<hipStream_t>(stream));
}

extern "C" int tbe_plan_batch(const int32_t *table_offsets, int32_t T, const int32_t *indices,
                              int64_t num_indices, const int32_t *offsets, int32_t B,
                              int64_t total_rows, int64_t max_table_rows, int32_t D,
                              int32_t dtype, void *workspace, uint64_t workspace_bytes,
                              void *stream) {
  using namespace tbe;
  const char *name = "tbe_plan_batch";
  TBE_REQUIRE(T > 0 && B > 0, "%s: T and B must be positive (got %d, %d)", name, T, B);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(table_offsets && offsets && (indices || num_indices == 0), "%s: null pointer argument", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  compute_layout(num_indices, D, dtype, T, &l);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  return build_plan(l, workspace, table_offsets, T, indices, num_indices, offsets, B, total_rows,
                    max_table_rows, static_cast<hipStream_t>(stream));
}

extern "C" int tbe_backward_planned(int32_t optimizer, const void *grad_output, void *weights,
                                    int32_t dtype, int64_t total_rows, int32_t D, int32_t T,
                                    int32_t B, int64_t num_indices,
                                    const void *per_sample_weights, void *optimizer_state,
                                    float learning_rate, float eps, void *grad_per_sample_weights,
                                    int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                    void *workspace, uint64_t workspace_bytes, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(optimizer == TBE_OPT_SGD || optimizer == TBE_OPT_ROWWISE_ADAGRAD,
              "tbe_backward_planned: bad optimizer %d", optimizer);
  TBE_REQUIRE(optimizer != TBE_OPT_SGD || !per_sample_weights,
              "tbe_backward_planned: SGD takes no per-sample weights");
  BackwardCall c{grad_output, weights, dtype, total_rows, 0, D, nullptr, T, nullptr, num_indices,
                 nullptr, B, per_sample_weights, optimizer_state, learning_rate, eps,
                 grad_per_sample_weights, workspace, workspace_bytes,
                 static_cast<hipStream_t>(stream),
                 optimizer == TBE_OPT_SGD ? kOptSgd : kOptAdagrad, true, nullptr, nullptr,
                 StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0}};
  return run_backward("tbe_backward_planned", c);
}
