// Host-side launchers of the backward stages, shared between the stage entry
// points and the fused backward entry points.
#pragma once

#include "tbe_common.h"

namespace tbe {

int linearize(const int32_t *table_offsets, int32_t T, const int32_t *indices,
              const int32_t *offsets, int32_t B, int32_t *keys, int32_t *grad_rows,
              hipStream_t stream);

// Pairs that come table by table (positions [offsets[t*B], offsets[(t+1)*B]) belong to table t)
// can be sorted per table: keys are then rows inside a table, end_bit covers the largest table,
// and key_bias[t] (nullable) is added to the keys of table t in the output.
struct SortTables {
  const int32_t *offsets;   // [T*B+1] bag offsets
  int32_t bags_per_table;   // B
  int32_t num_tables;       // T
  const int32_t *key_bias;  // [T] first row of every table
  // nullable, [n] out: the gradient row b*T + t of every position (what linearize() records),
  // written by the sort's set-up launch instead of a launch of its own
  int32_t *grad_rows = nullptr;
  int32_t key_mul = 1;      // a key leaves the last pass as key * key_mul + key_bias[t]
};

// Tables stored interleaved, [E][T][D] with bags b*T + t bounded by offsets[b * stride + t] and the
// entry after it: puts the batch into table-major order (indices_tm [n], offsets_tm [T*B+1]) and
// writes bias[t] = t; totals [T] and chunk_sums [T * interleaved_chunks_per_table(B)] are scratch.
inline int64_t interleaved_chunks_per_table(int32_t B) { return (static_cast<int64_t>(B) + kBlockThreads - 1) / kBlockThreads; }
int interleaved_to_table_major(const int32_t *indices, const int32_t *offsets, int32_t offsets_stride,
                               int32_t T, int32_t B, int32_t *totals, int32_t *bias, int32_t *chunk_sums,
                               int32_t *offsets_tm, int32_t *indices_tm, hipStream_t stream);

uint64_t sort_workspace_bytes(int64_t n, int32_t num_tables);
// device_count (nullable): the number of pairs, read on the device (at most n; with tables == nullptr).
int sort_pairs(const int32_t *keys_in, const int32_t *values_in, int32_t *keys_out,
               int32_t *values_out, int64_t n, int32_t end_bit, void *workspace,
               hipStream_t stream, const SortTables *tables, const int32_t *device_count = nullptr);

uint64_t segments_workspace_bytes(int64_t n);
// segment_ids (nullable): receives, for every sorted position, the index of its segment.
// clear_queue_counters: num_unique points at the 4-word counter block of a backward workspace;
// words 1..3 (the update stage's queue counters) are set to zero as well.
int find_segments(const int32_t *keys_sorted, int64_t n, int32_t *segment_starts,
                  int32_t *num_unique, int32_t *segment_ids, void *workspace, hipStream_t stream,
                  bool clear_queue_counters = false);

// Segments of more than kShortSegment occurrences leave the lane-group path and are reduced by
// whole wavefronts in chunks of at most kChunkLen occurrences.  (Measured, fused forward + backward
// of 5.2 M lookups: 64 tables of 100 k fp32 rows of 128, Zipf 1.05 / 32 tables of 1 M fp16 rows of
// 64, Zipf 1.2, weighted Adagrad -- threshold 16: 1.118 / 0.540 ms, 32: 1.118 / 0.532, 64: 1.114 /
// 0.525, 128: 1.105 / 0.522, 256: 1.102 / 0.525.)  The approximate (per-lookup) update, whose
// lane groups walk a row's occurrences one after the other, hands rows over from
// kApproxShortSegment occurrences on.
constexpr int kShortSegment = 128;
constexpr int kApproxShortSegment = 16;
// (tables of different row widths: rows of more than kMixedShort occurrences are summed in chunks)
constexpr int kMixedShort = 8;
constexpr int kChunkLen = 256;
// Integers kept next to the number of unique rows (all zeroed when the segments are found): [1], [2]
// queue lengths of the kernels that keep one queue (mixed-D tables, the approximate update), and from
// word 64 on one 128-byte line per XCD: [0] chunk records (or rows) queued by the XCD's workgroups,
// [1] its segments of several chunks.  A line of its own, because the workgroups of an XCD queue
// with one 64-bit atomic add on those two words, and atomic adds on one line queue up behind each
// other (with all counters of the chip on one line, a skewed batch spent 26 us of a 180 us kernel
// waiting for them).
constexpr int kXcdCounterBase = 64;
constexpr int kXcdCounterStride = 32;
constexpr int kNumCounters = kXcdCounterBase + 8 * kXcdCounterStride;
__host__ __device__ constexpr int xcd_counter(int xcd) { return kXcdCounterBase + kXcdCounterStride * xcd; }
constexpr int kApproxHuge = 256;   // occurrences from which on the approximate update walks a row before the others
constexpr int kApproxCoopD = 128;  // widest row that a whole workgroup walks (fp16 rows of more than kApproxHuge occurrences)
// The short-row kernel's workgroups of XCD x own the segments that start in the x-th eighth of
// the sorted positions (rounded up to whole workgroups: fewer than 1200 positions more) and queue
// their chunk records in a region of their own.  Segments are consecutive, so only the last
// segment that starts in an eighth can reach beyond it: the records of one XCD are bounded by
// those of its eighth plus those of one segment of any length.
inline int64_t chunk_queue_capacity(int64_t n) {
  const int64_t eighth = (n + 7) / 8 + 2048;
  // (sized for the smallest of the thresholds: the approximate update of fp32 rows and the update of
  // tables of different row widths queue their chunk records here too)
  return eighth / (kMixedShort + 1) + eighth / kChunkLen + n / kChunkLen + 8;
}

// Room of one XCD's list of segments of several chunks (more than kChunkLen occurrences each) that
// start in its eighth of the sorted positions (and, for tables of different row widths, the up to
// 63 rows that share a strip of 64 unique rows with the last row of the eighth).
inline int64_t long_list_capacity(int64_t n) { return ((n + 7) / 8 + 2048) / (kChunkLen + 1) + 2 + 64; }
// The partial row of chunk k of a segment [begin, end) of several chunks.  Every chunk but a segment's
// last is kChunkLen positions long, so no two of them begin in the same window of kChunkLen positions;
// and segments of several chunks end more than kChunkLen positions apart, so no two last chunks end in
// the same window: two rows per window, no counter.
__host__ __device__ inline int partial_row_of_chunk(int begin, int end, int k, int num_chunks) {
  return k == num_chunks - 1 ? 2 * ((end - 1) / kChunkLen) + 1 : 2 * ((begin + k * kChunkLen) / kChunkLen);
}

// Room of one XCD's queue of rows that the approximate update's short-row kernel leaves to the
// wavefront-per-row kernel: the rows of more than kApproxShortSegment occurrences that start in the
// XCD's eighth of the sorted positions (an eighth is rounded up to whole workgroups of tiles).
inline int64_t approx_long_queue_capacity(int64_t n) { return (n / 8 + 8192) / (kApproxShortSegment + 1) + 2; }
// (behind the eight queues: the rows of more than kApproxHuge occurrences, at most n / 257 + 1)

enum { kOptSgd = 0, kOptAdagrad = 1 };

struct UpdateArgs {
  const void *grad_output;
  void *weights;
  void *optimizer_state;        // null for SGD
  const void *per_sample_weights;  // null when unweighted
  void *grad_per_sample_weights;
  const int32_t *keys_sorted;
  const int32_t *positions_sorted;
  const int32_t *grad_rows;
  const int32_t *segment_starts;
  int32_t *counters;            // [0] = U (input), [1] = #long records, [2] = #chunk records, [3] = #partial rows
  const int32_t *segment_ids;   // [N] segment of every sorted position
  void *long_segments;          // 16-byte records [8][max_long / 8]: segments cut into several chunks, one list per XCD
  void *chunk_segments;         // 32-byte records [8][max_chunks / 8]: one chunk queue per XCD
  void *partial_sums;           // acc [max_partial][D]
  const int32_t *unique_slots;  // cache-fronted tables: slot of each unique row (-1 = not resident)
  void *cache_rows;             // cache-fronted tables: [slots][D] rows in HBM
  int64_t num_indices;
  int64_t max_long;
  int64_t max_chunks;
  int32_t dtype;
  int32_t D;
  int32_t optimizer;
  float learning_rate;
  float eps;
  StochasticRounding stochastic_rounding;  // fp16 weights only
};

int segment_update(const UpdateArgs &args, hipStream_t stream);
// The approximate row-wise Adagrad for rows of at most kApproxShortSegment occurrences, with the
// position-balanced tiles of the exact update (rows no wider than 64 vectors: approx_short_serves);
// longer rows are appended to `queue` as unique-row numbers, their count in args.counters[1].
bool approx_short_serves(int32_t dtype, int32_t D);
int segment_update_approx_short(const UpdateArgs &args, int32_t *queue, hipStream_t stream);
// fp32 / fp64 rows without per-sample weights: the approximate update of a row is a weighted sum
// of its gradient rows, so its long rows are summed in chunks like the exact update's.  Then
// segment_update_approx_short() is called with a null queue (the rows go to the chunk queues of
// its UpdateArgs) and, once the lookups' state addends are known, segment_update_approx_sum_long().
bool approx_sums_long_rows(int32_t dtype, int32_t D, bool weighted);
int segment_update_approx_sum_long(const UpdateArgs &args, const void *lookup_wss, hipStream_t stream);

int key_bits_for(int64_t total_rows);
void backward_layout(int64_t n, int32_t D, int32_t dtype, int32_t T, tbe_workspace_layout_t *layout);
// max_table_rows: an upper bound of the rows of the largest table (0 = unknown, total_rows is
// used); it sets how many key bits are sorted.
// grad_rows, keys_sorted and positions_sorted of the layout (table_offsets: first row of every table)
// interleaved_offsets_stride > 0: tables stored [E][T][D] (table_offsets unused), `offsets` rows of
// that many entries; the layout is then the one of backward_interleaved_layout().
int sort_batch(const tbe_workspace_layout_t &layout, void *workspace, const int32_t *table_offsets, int32_t T,
               const int32_t *indices, int64_t n, const int32_t *offsets, int32_t B, int64_t total_rows,
               int64_t max_table_rows, hipStream_t stream, int32_t interleaved_offsets_stride = 0);
int build_plan(const tbe_workspace_layout_t &layout, void *workspace, const int32_t *table_offsets,
               int32_t T, const int32_t *indices, int64_t n, const int32_t *offsets, int32_t B,
               int64_t total_rows, int64_t max_table_rows, hipStream_t stream,
               int32_t interleaved_offsets_stride = 0);

// Tables of different row widths in one flat weight array (the reference's MixedDim layout,
// table_batched_embeddings_ops.py:204-435).
struct MixedTables {
  const int64_t *table_offsets;      // [T+1] first element of each table
  const int32_t *table_dim_offsets;  // [T+1] first row id of each table
  const int32_t *dim_offsets;        // [T+1] first output column of each table
  int32_t total_D;
  int32_t T;
  // b = grow / T for a gradient row number grow = b*T + t < 2^31 as a multiplication and a shift:
  // magic = ceil(2^(31 + s) / T) with s = ceil(log2 T) fits 32 bits and gives the exact quotient
  uint32_t bag_magic = 0;
  int32_t bag_shift = 0;
};
// Row width the workspace of mixed-D tables is laid out for: its partial rows hold 64 vectors, the
// widest row that is summed in chunks (8 elements a vector at most for fp16).
inline int32_t mixed_layout_dim(int32_t dtype) {
  return kWave * (dtype == TBE_DTYPE_F16 ? 8 : dtype == TBE_DTYPE_F32 ? 4 : 2);
}
inline void set_bag_division(MixedTables &mt) {
  int log2_T = 0;
  while ((int64_t{1} << log2_T) < mt.T) ++log2_T;
  mt.bag_shift = 31 + log2_T;
  mt.bag_magic = static_cast<uint32_t>(((uint64_t{1} << mt.bag_shift) + static_cast<uint64_t>(mt.T) - 1) /
                                       static_cast<uint64_t>(mt.T));
}
// The approximate row-wise Adagrad update (one lookup at a time per row, in position order) on a
// workspace that holds the batch's plan.  Uniform tables: D > 0 and the mixed_* pointers null;
// mixed-D tables: D = 0, and the strip kernel of tbe_backward_mixed has already applied the rows
// of few occurrences and filled the two queues above.  unique_slots / cache_rows (tables behind the
// row cache; slot_D: the width of a cache row, for mixed-D tables): every row is updated where it
// lives, as in segment_update.
int approx_update(const void *grad_output, void *weights, void *state, const void *psw, void *grad_psw,
                  int32_t dtype, int32_t fp16_vector_width, int32_t D, int64_t n, float lr, float eps,
                  const int64_t *mixed_table_offsets, const int32_t *table_dim_offsets,
                  const int32_t *dim_offsets, int32_t total_D, int32_t T, const int32_t *offsets, int32_t B,
                  StochasticRounding sr, const tbe_workspace_layout_t &l, void *workspace, hipStream_t stream,
                  const int32_t *unique_slots = nullptr, void *cache_rows = nullptr, int32_t slot_D = 0);

// Where the approximate update of mixed-D tables keeps its two queues of unique-row indices inside
// the backward workspace: rows of at most 64 vectors with more occurrences than the strip kernel
// applies itself (counted in counters[1]; the queue approx_update's wavefront-per-row kernel
// drains), and rows wider than 64 vectors (counters[2]).
inline int32_t *approx_mixed_long_queue(const tbe_workspace_layout_t &l, void *workspace) {
  return reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + l.chunk_segments);
}
// (behind the first queue's room, n / (kMixedShort + 1) + 1 rows: the fp16 rows of more than kApproxHuge
// occurrences and at most kApproxCoopD elements, which a workgroup walks; counted in counters[xcd_counter(0)])
inline int64_t approx_mixed_huge_offset(int64_t n) { return n / (kMixedShort + 1) + 1; }
inline int32_t *approx_mixed_wide_queue(const tbe_workspace_layout_t &l, void *workspace) {
  return reinterpret_cast<int32_t *>(static_cast<char *>(workspace) + l.segment_ids);
}

// Copies the rows that tbe_cache_prepare staged for this step back to the backing table.
int cache_unstage(const tbe_cache_t *cache, int32_t dtype, int32_t D, const int32_t *keys_sorted,
                  const int32_t *segment_starts, const int32_t *counters,
                  const int32_t *unique_slots, int64_t num_indices, hipStream_t stream);

}  // namespace tbe
