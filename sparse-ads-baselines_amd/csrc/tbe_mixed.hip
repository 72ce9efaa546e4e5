// Tables with per-table embedding dimension (mixed D), for gfx950.
//
// Layout of the reference's MixedDim classes (table_batched_embeddings_ops.py:324-379):
//   weights            1-D, table t occupies elements [table_offsets[t], table_offsets[t+1]),
//                      row-major [rows_t][D_t]                     (int64 [T+1])
//   table_dim_offsets  first global row id of each table             (int32 [T+1]; the name is the
//                      reference's: it is a cumulative sum of ROW counts)
//   dim_offsets        first output column of each table             (int32 [T+1]), D_t % 4 == 0
//   output / grad      [B][total_D], table t in columns [dim_offsets[t], dim_offsets[t+1])
// Kernels follow batched_embedding_forward_kernel_mixed_D_1
// (table_batched_embeddings_cuda.cu:882-943), linear_index_weight_offsets_mixed_D_kernel
// (:1220-1247) and batched_embedding_backward_adagrad_exact_kernel_mixed_D_1 (:1249-1348).
//
// Forward: one wavefront owns a bag and its lanes stride over the row's 16-byte vectors, so any
// D_t works.  Backward: rows of a few occurrences are updated by lane groups in strips of 64
// unique rows (update_mixed_kernel); rows of more occurrences are summed in chunks by whole
// wavefronts, with the chunk records, per-XCD queues and partial rows of the uniform tables'
// update (update_chunks_mixed_kernel, update_long_finish_mixed_kernel); rows wider than 64
// vectors are walked by one wavefront each.  The integer stages (sort, segments) are shared.

#include <algorithm>
#include <type_traits>

#include "tbe_queues.h"
#include "tbe_rowwise.h"
#include "tbe_stages.h"

namespace tbe {
namespace {

template <typename A> __device__ __forceinline__ A mixed_multiplier(A state_new, float lr, float eps);
template <> __device__ __forceinline__ float mixed_multiplier<float>(float s, float lr, float eps) {
  return static_cast<float>(static_cast<double>(lr) * (1.0 / static_cast<double>(sqrtf(s) + eps)));
}
template <> __device__ __forceinline__ double mixed_multiplier<double>(double s, float lr, float eps) {
  return static_cast<double>(lr) * (1.0 / (sqrt(s) + static_cast<double>(eps)));
}

// One wavefront per bag.  A table's rows are `chunks` = D_t / VEC vectors; for rows of at most
// 64 vectors the lanes form 64 / group_lanes lane groups (group_lanes = chunks rounded up to a
// power of two: group and column of a lane are a shift and a mask whatever the width), the
// groups split the bag's rows and are combined by a butterfly at the end -- a table of 32
// columns keeps all 64 lanes busy with 8 rows per load instruction instead of 8 lanes with one.
// Wider rows are walked in blocks of 64 vectors, one row per load.
// CACHED: every lookup carries a location (lookup_slots[p]); a non-negative value is a row of the
// HBM row cache (at cache_rows + slot * slot_D, slot_D the widest table's width), a negative one
// means the row is read from the table.
template <typename T, int VEC, bool WEIGHTED, int UNROLL, bool CACHED>
__global__ __launch_bounds__(kBlockThreads) void forward_mixed_kernel(
    const T *__restrict__ weights, const int64_t *__restrict__ table_offsets,
    const int32_t *__restrict__ dim_offsets, const int32_t *__restrict__ indices,
    const int32_t *__restrict__ offsets, const T *__restrict__ psw, T *__restrict__ output, int B,
    int total_D, int num_bags, int64_t blocks_per_xcd, const int32_t *__restrict__ lookup_slots,
    const T *__restrict__ cache_rows, int slot_D) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t bag64 = xcd_contiguous(blockIdx.x, blocks_per_xcd) * kWavesPerBlock + (threadIdx.x >> 6);
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const int t = bag / B;
  const int b = bag - t * B;
  const int dim_start = dim_offsets[t];
  const int D = dim_offsets[t + 1] - dim_start;
  const int chunks = D / VEC;
  const T *table = weights + table_offsets[t];
  const int start = offsets[bag];
  const int end = offsets[bag + 1];
  T *out_row = output + static_cast<int64_t>(b) * total_D + dim_start;
  if (chunks <= 0) return;  // a table without columns has no output

  if (chunks <= kWave) {
    const int group_shift = chunks > 1 ? 32 - __builtin_clz(chunks - 1) : 0;
    const int group_lanes = 1 << group_shift;
    const int groups = kWave >> group_shift;
    const int r = lane >> group_shift;
    const int c = lane & (group_lanes - 1);
    const bool active = c < chunks;
    // a lane beside the row's columns loads the row's last vector and drops it
    const int64_t col_element = static_cast<int64_t>(min(c, chunks - 1)) * VEC;
    const T *col = table + col_element;
    V acc;
    acc.zero();
    for (int base = start; base < end; base += kWave) {
      const int n = min(kWave, end - base);
      int my_idx = 0, my_slot = -1;
      T my_w_raw = T(0);
      if (lane < n) {
        my_idx = __builtin_nontemporal_load(indices + base + lane);
        if constexpr (CACHED) my_slot = __builtin_nontemporal_load(lookup_slots + base + lane);
        if constexpr (WEIGHTED) my_w_raw = psw[base + lane];
      }
      const A my_w = WEIGHTED ? to_acc(my_w_raw) : A(0);
      // `count` rows per lane group at a time; the loads of a step are straight-line code (every
      // lane loads; a lane past the batch's end loads the batch's first row again and drops it)
      // so they are issued back to back.  The step sizes 8, 4, 2, 1 follow the rows that are left,
      // so that a bag of one row costs one load instruction, not eight.
      int j0 = 0;
      auto step = [&](auto count) {
        constexpr int kCount = decltype(count)::value;
        R raw[kCount];
        A w[kCount];
        bool ok[kCount];
#pragma unroll
        for (int u = 0; u < kCount; ++u) {
          const int j = j0 + u * groups + r;
          ok[u] = active && j < n;
          const int src = j < n ? j : 0;
          const int64_t idx = shfl_idx(my_idx, src);
          if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, src);
          const T *row = col + idx * D;
          if constexpr (CACHED) {
            const int slot = shfl_idx(my_slot, src);
            if (slot >= 0) row = cache_rows + static_cast<int64_t>(slot) * slot_D + col_element;
          }
          raw[u] = V::load_raw(row);
        }
#pragma unroll
        for (int u = 0; u < kCount; ++u) {
          V x;
          x.unpack(raw[u]);
#pragma unroll
          for (int i = 0; i < VEC; ++i) {
            const A term = WEIGHTED ? x.v[i] * w[u] : x.v[i];
            acc.v[i] += ok[u] ? term : A(0);
          }
        }
        j0 += kCount * groups;
      };
      while (n - j0 >= groups * UNROLL) step(std::integral_constant<int, UNROLL>{});
      if (n - j0 >= groups * 4) step(std::integral_constant<int, 4>{});
      if (n - j0 >= groups * 2) step(std::integral_constant<int, 2>{});
      while (j0 < n) step(std::integral_constant<int, 1>{});
    }
    // combine the groups (butterfly over the group index: every group ends with the sum)
    for (int m = kWave >> 1; m >= group_lanes; m >>= 1) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc.v[i] += shfl_x(acc.v[i], m);
    }
    if (r == 0 && active) acc.store(out_row + static_cast<int64_t>(c) * VEC);
    return;
  }

  for (int cb = 0; cb < chunks; cb += kWave) {
    const int c = cb + lane;
    const bool ok_c = c < chunks;
    const T *col = table + static_cast<int64_t>(c) * VEC;
    V acc;
    acc.zero();
    for (int base = start; base < end; base += kWave) {
      const int n = min(kWave, end - base);
      int my_idx = 0, my_slot = -1;
      A my_w = A(0);
      if (lane < n) {
        my_idx = indices[base + lane];
        if constexpr (CACHED) my_slot = lookup_slots[base + lane];
        if constexpr (WEIGHTED) my_w = to_acc(psw[base + lane]);
      }
      for (int j0 = 0; j0 < n; j0 += 4) {
        R raw[4];
        A w[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int j = min(j0 + u, n - 1);
          const int64_t idx = shfl_idx(my_idx, j);
          if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, j);
          const T *row = col + idx * D;
          if constexpr (CACHED) {
            const int slot = shfl_idx(my_slot, j);
            if (slot >= 0) row = cache_rows + static_cast<int64_t>(slot) * slot_D + static_cast<int64_t>(c) * VEC;
          }
          if (ok_c && j0 + u < n) raw[u] = V::load_raw(row);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          if (ok_c && j0 + u < n) {
            V x;
            x.unpack(raw[u]);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WEIGHTED) acc.v[i] += x.v[i] * w[u];
              else acc.v[i] += x.v[i];
            }
          }
        }
      }
    }
    if (ok_c) acc.store(out_row + static_cast<int64_t>(c) * VEC);
  }
}

// Everything a wavefront needs to know about one unique row.
struct MixedRow {
  int seg_begin, seg_end;  // sorted positions of its occurrences
  int32_t key;             // global row id (index of its optimizer state)
  int dim_start, D;        // first gradient column and width of its table
  int64_t row_element;     // element offset of the row in `weights` (its place in the table: what the
                           // random words of stochastic rounding go by)
  void *where;             // the row's first element where it is stored: in `weights`, or in a row of the cache
};

// Fills in where the u-th unique row is stored.
template <bool CACHED, typename T>
__device__ __forceinline__ void locate_row(MixedRow &row, T *weights, const int32_t *__restrict__ unique_slots, int64_t u,
                                           T *cache_rows, int slot_D) {
  row.where = weights + row.row_element;
  if constexpr (CACHED) {
    const int slot = unique_slots[u];
    if (slot >= 0) row.where = cache_rows + static_cast<int64_t>(slot) * slot_D;
  }
}

// Narrow rows (at most 64 vectors): `chunks` = D / VEC consecutive lanes form a lane group, the
// 64 / chunks groups split the occurrences of a 64-position batch (the batch's positions,
// gradient rows and weights are fetched with one load per lane, then up to UNROLL independent
// gradient rows per group are in flight).  A wavefront takes the batches first_batch,
// first_batch + batch_stride, ...; the positions of a batch are requested two batches ahead and
// its gradient row ids and weights one batch ahead, so a batch waits for gradient rows only.
// The groups are combined into group 0 in a fixed tree.  Returns with G (valid in group 0) and
// w_old (valid in every group when WEIGHTED, else in group 0).
template <typename T, int VEC, bool WEIGHTED, int UNROLL>
__device__ __forceinline__ void mixed_accumulate_narrow(
    const T *__restrict__ grad_output, const T *__restrict__ psw,
    T *__restrict__ grad_psw, int num_tables, int total_D,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows, int lane,
    const MixedRow &row, int first_batch, int batch_stride, RowVec<T, VEC> &w_old, RowVec<T, VEC> &G) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;
  // a lane group is the row's vector count rounded up to a power of two (its surplus lanes idle),
  // so that group and column of a lane are a shift and a mask whatever the table's width
  const int chunks = row.D / VEC;
  const int group_shift = chunks > 1 ? 32 - __builtin_clz(chunks - 1) : 0;
  const int group_lanes = 1 << group_shift;
  const int groups = kWave >> group_shift;
  const int r = lane >> group_shift;
  const int c = lane & (group_lanes - 1);
  const bool active = c < chunks;
  const int64_t col = static_cast<int64_t>(c) * VEC;
  const int64_t safe_col = active ? col : 0;
  const T *wrow = static_cast<const T *>(row.where);
  const T *gcol = grad_output + row.dim_start;
  w_old.zero();
  if (active && (WEIGHTED || r == 0)) w_old.load(wrow + col);
  G.zero();
  const int step = batch_stride * kWave;
  // lanes past the row's end ask for its first position: any valid index will do
  auto position_at = [&](int64_t i) { return positions_sorted[i < row.seg_end ? i : row.seg_begin]; };
  int base = row.seg_begin + first_batch * kWave;
  int pos_now = position_at(base + lane);
  int pos_next = position_at(static_cast<int64_t>(base) + step + lane);
  int grow_now = grad_rows[pos_now];
  A w_now = A(1);
  if constexpr (WEIGHTED) w_now = to_acc(psw[pos_now]);
  for (; base < row.seg_end; base += min(step, row.seg_end - base)) {
    const int n = min(kWave, row.seg_end - base);
    const int my_pos = pos_now;
    const int my_bag = grow_now / num_tables;
    const A my_w = w_now;
    pos_now = pos_next;
    pos_next = position_at(static_cast<int64_t>(base) + 2 * step + lane);
    grow_now = grad_rows[pos_now];
    if constexpr (WEIGHTED) w_now = to_acc(psw[pos_now]);
    // Straight-line code: every lane loads (a lane without an occurrence or beside the row's
    // columns loads what occurrence 0 / column 0 loads and drops it), so that the UNROLL loads
    // of a step are issued back to back.
    for (int j0 = 0; j0 < n; j0 += groups * UNROLL) {
      R raw[UNROLL];
      bool ok[UNROLL];
      int src[UNROLL];
#pragma unroll
      for (int k = 0; k < UNROLL; ++k) {
        const int j = j0 + k * groups + r;
        ok[k] = active && j < n;
        src[k] = j < n ? j : 0;
      }
#pragma unroll
      for (int k = 0; k < UNROLL; ++k) {
        const int64_t bag = shfl_idx(my_bag, src[k]);
        raw[k] = V::load_raw(gcol + bag * total_D + safe_col);
      }
#pragma unroll
      for (int k = 0; k < UNROLL; ++k) {
        A pw = A(1);
        int pos = 0;
        if constexpr (WEIGHTED) {
          pw = shfl_idx(my_w, src[k]);
          pos = shfl_idx(my_pos, src[k]);
        }
        V x;
        x.unpack(raw[k]);
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = ok[k] ? x.v[i] : A(0);
        if constexpr (WEIGHTED) {
          A dot = A(0);
#pragma unroll
          for (int i = 0; i < VEC; ++i) dot += w_old.v[i] * x.v[i];
          for (int m = group_lanes >> 1; m > 0; m >>= 1) dot += shfl_x(dot, m);  // idle lanes add 0
          if (ok[k] && c == 0) grad_psw[pos] = from_acc<T, A>(dot);
#pragma unroll
          for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * pw;
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i];
        }
      }
    }
  }
  // combine the groups (butterfly over the group index: every group ends with the sum)
  for (int m = kWave >> 1; m >= group_lanes; m >>= 1) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) G.v[i] += shfl_x(G.v[i], m);
  }
}

// Optimizer step of a narrow row whose gradient sum G sits in lane group 0.
template <typename T, int VEC, int OPT>
__device__ __forceinline__ void mixed_apply_narrow(typename AccOf<T>::type *__restrict__ state,
                                                   float lr, float eps, const StochasticRounding &sr,
                                                   int lane, const MixedRow &row,
                                                   typename AccOf<T>::type state_old,
                                                   const RowVec<T, VEC> &w_old, const RowVec<T, VEC> &G) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  const int chunks = row.D / VEC;
  const bool first_group = lane < chunks;
  A mult = static_cast<A>(lr);
  if constexpr (OPT == kOptAdagrad) {
    A local = A(0);
    if (first_group) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) local += G.v[i] * G.v[i];
    }
    const A gss = group_sum<kWave, A>(local, kWave, 0);
    const A s_new = state_old + gss;
    if (lane == 0) state[row.key] = s_new;
    mult = mixed_multiplier<A>(s_new, lr, eps);
  }
  if (first_group) {
    V w;
#pragma unroll
    for (int i = 0; i < VEC; ++i) w.v[i] = w_old.v[i] - G.v[i] * mult;
    const int64_t col = static_cast<int64_t>(lane) * VEC;
    store_row<T, VEC, false>(static_cast<T *>(row.where) + col, w, sr, row.row_element + col);
  }
}

// Rows wider than 64 vectors, one wavefront: the passes of the reference's exact kernel (sum of
// squares first, then the update), one column block of 64 vectors at a time.
template <typename T, int VEC, int OPT, bool WEIGHTED>
__device__ __forceinline__ void mixed_update_wide(
    const T *__restrict__ grad_output, typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, int num_tables, int total_D,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows, float lr,
    float eps, const StochasticRounding &sr, int lane, const MixedRow &row,
    typename AccOf<T>::type state_old) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  const int seg_begin = row.seg_begin, seg_end = row.seg_end;
  const int32_t key = row.key;
  const int64_t row_element = row.row_element;
  const int chunks = row.D / VEC;
  T *wrow = static_cast<T *>(row.where);
  const T *gcol = grad_output + row.dim_start;
  if constexpr (WEIGHTED) {
    for (int i = seg_begin; i < seg_end; ++i) {
      const int pos = positions_sorted[i];
      const T *grow = gcol + static_cast<int64_t>(grad_rows[pos] / num_tables) * total_D;
      A dot = A(0);
      for (int cb = lane; cb < chunks; cb += kWave) {
        V w, g;
        w.load(wrow + static_cast<int64_t>(cb) * VEC);
        g.load(grow + static_cast<int64_t>(cb) * VEC);
#pragma unroll
        for (int k = 0; k < VEC; ++k) dot += w.v[k] * g.v[k];
      }
      dot = group_sum<kWave, A>(dot, kWave, 0);
      if (lane == 0) grad_psw[pos] = from_acc<T, A>(dot);
    }
  }

  A mult = static_cast<A>(lr);
  if constexpr (OPT == kOptAdagrad) {
    A local = A(0);
    for (int cb = lane; cb < chunks; cb += kWave) {
      V G;
      G.zero();
      for (int i = seg_begin; i < seg_end; ++i) {
        const int pos = positions_sorted[i];
        V g;
        g.load(gcol + static_cast<int64_t>(grad_rows[pos] / num_tables) * total_D + static_cast<int64_t>(cb) * VEC);
        A pw = A(1);
        if constexpr (WEIGHTED) pw = to_acc(psw[pos]);
#pragma unroll
        for (int k = 0; k < VEC; ++k) G.v[k] += WEIGHTED ? g.v[k] * pw : g.v[k];
      }
#pragma unroll
      for (int k = 0; k < VEC; ++k) local += G.v[k] * G.v[k];
    }
    const A gss = group_sum<kWave, A>(local, kWave, 0);
    const A s_new = state_old + gss;
    if (lane == 0) state[key] = s_new;
    mult = mixed_multiplier<A>(s_new, lr, eps);
  }

  for (int cb = lane; cb < chunks; cb += kWave) {
    V G;
    G.zero();
    for (int i = seg_begin; i < seg_end; ++i) {
      const int pos = positions_sorted[i];
      V g;
      g.load(gcol + static_cast<int64_t>(grad_rows[pos] / num_tables) * total_D + static_cast<int64_t>(cb) * VEC);
      A pw = A(1);
      if constexpr (WEIGHTED) pw = to_acc(psw[pos]);
#pragma unroll
      for (int k = 0; k < VEC; ++k) G.v[k] += WEIGHTED ? g.v[k] * pw : g.v[k];
    }
    V w;
    w.load(wrow + static_cast<int64_t>(cb) * VEC);
#pragma unroll
    for (int k = 0; k < VEC; ++k) w.v[k] = w.v[k] - G.v[k] * mult;
    store_row<T, VEC, false>(wrow + static_cast<int64_t>(cb) * VEC, w, sr, row_element + static_cast<int64_t>(cb) * VEC);
  }
}

// Short rows.  A wavefront takes strips of 64 consecutive unique rows.
//
// First, one row per lane: what a row needs before its gradient rows can be requested -- segment
// bounds, key, positions, bag and table of each occurrence (from the gradient row ids b*T+t),
// the table's width and offsets, optimizer state -- is fetched for the 64 rows at once, so the
// dependent loads are paid per strip.  Rows of more than kMixedShort occurrences (the hot rows,
// which are neighbours in key order) and rows wider than 64 vectors are not reduced here: the
// former leave chunk records for update_chunks_mixed_kernel -- one wavefront per chunk of at most
// kChunkLen occurrences -- so that they spread over the machine, the latter their row numbers.
// The other rows leave a 32-byte record in LDS (in row order), and every occurrence of theirs
// leaves the element offset of its gradient row (and its position, for per-sample weights).
//
// Then, one row per lane *group*, 64 / group_lanes rows at a time, so the instruction stream is
// shared by several rows.  The group size fits the widest row of the strip (a strip spans a table
// boundary now and then).  Each group adds its row's occurrences in order.  The packed row and
// the first kMixedAhead packed gradient rows of an iteration are requested one iteration ahead.
//
// bag_magic / bag_shift: b = (grow * bag_magic) >> bag_shift for every gradient row id
// grow = b*T+t < 2^31 (division by the invariant T).
// Empty statement that reads and "rewrites" the registers of x: what was loaded into x has
// arrived when it is passed.
template <typename X> __device__ __forceinline__ void register_fence(X &x) {
  static_assert(sizeof(X) % 4 == 0, "whole registers");
  uint32_t words[sizeof(X) / 4];
  __builtin_memcpy(words, &x, sizeof(X));
#pragma unroll
  for (size_t i = 0; i < sizeof(X) / 4; ++i) asm volatile("" : "+v"(words[i]));
  __builtin_memcpy(&x, words, sizeof(X));
}

// Workgroups per compute unit the strip kernel is compiled for: as many as its registers allow
// without spilling (per-sample weights, 8-element vectors, fp64 and the per-lookup form each need more).
constexpr int mixed_strip_blocks(bool weighted, bool wide_vectors, bool approx, bool fp64) {
  const int heavy = (weighted ? 1 : 0) + (wide_vectors ? 1 : 0) + (approx ? 1 : 0) + (fp64 && (weighted || approx) ? 1 : 0);
  return heavy == 0 ? 5 : heavy == 1 ? 4 : 3;
}
constexpr int kMixedAhead = 4;
// APPROX (row-wise Adagrad only): the approximate update's per-lookup form -- every occurrence adds
// its bag's ||grad||^2 (times its squared weight) to the row's state and moves the row by its own
// multiplier, one occurrence after the other in position order, the row rounded to the weights'
// type every time (the arithmetic of approx_adagrad_kernel).  Rows of more than kMixedShort
// occurrences then go to a queue of row numbers (`queued_rows`, counters[1]) whatever their length.
// CACHED: the tables are fronted by the row cache; unique_slots[u] >= 0 is the row of `cache_rows`
// (slot_D elements each) that holds the u-th unique row, and the list records of the rows of several
// chunks carry the row's number u instead of its table.
template <typename T, int VEC, int OPT, bool WEIGHTED, bool APPROX = false, bool CACHED = false>
__global__ __launch_bounds__(kBlockThreads, mixed_strip_blocks(WEIGHTED, VEC == 8, APPROX, sizeof(T) == 8)) void update_mixed_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int64_t *__restrict__ table_offsets,
    const int32_t *__restrict__ table_dim_offsets, const int32_t *__restrict__ dim_offsets,
    int num_tables, uint32_t bag_magic, int bag_shift, int total_D,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ segment_starts,
    int32_t *__restrict__ counters, int32_t *__restrict__ wide_rows,
    int32_t *__restrict__ queued_rows, ChunkRecord *__restrict__ chunk_records,
    LongRecord *__restrict__ long_records, int64_t max_chunks, int64_t max_long, int positions_per_xcd,
    float lr, float eps, StochasticRounding sr, int approx_huge_offset = 0,
    const int32_t *__restrict__ unique_slots = nullptr,
    T *__restrict__ cache_rows = nullptr, int slot_D = 0) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;
  static_assert(sizeof(A) == 4 || sizeof(A) == 8, "optimizer state is float or double");
  // a row's record: {occurrences, first slot, key, D}, {where the row is stored (64 bits), state}.
  // Where: its first element in `weights`; CACHED: or, complemented, its first element in `cache_rows`,
  // and s_element holds its first element in `weights` (its place in the table) beside the record.
  __shared__ int4 s_row[kWavesPerBlock][kWave][2];
  __shared__ int64_t s_element[kWavesPerBlock][CACHED ? kWave : 1];
  auto stored_at = [&](int64_t where) -> T * {
    if constexpr (CACHED) {
      if (where < 0) return cache_rows + ~where;
    }
    return weights + where;
  };
  // occurrences of a strip's short rows: at most 64 rows of kMixedShort occurrences
  __shared__ int s_goff[kWavesPerBlock][kWave * kMixedShort];
  __shared__ int s_pos[kWavesPerBlock][WEIGHTED ? kWave * kMixedShort : 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + wave;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  const int64_t num_strips = (static_cast<int64_t>(U) + kWave - 1) / kWave;
  auto bag_of = [&](int grow) {
    return static_cast<int>((static_cast<uint64_t>(static_cast<uint32_t>(grow)) * bag_magic) >> bag_shift);
  };

  for (int64_t strip = wave_id; strip < num_strips; strip += stride) {
    const int64_t u0 = strip * kWave;
    const int rows_here = static_cast<int>(min(static_cast<int64_t>(kWave), U - u0));
    // lane j holds the bookkeeping of row u0 + j (clamped: lanes past the end repeat the last row)
    const int64_t my_u = u0 + min(lane, rows_here - 1);
    const int l_begin = segment_starts[my_u];
    const int l_end = segment_starts[my_u + 1];
    const int32_t l_key = keys_sorted[l_begin];
    // the first kMixedShort occurrences (the last one again, past the row's end)
    int l_pos[kMixedShort], l_bag[kMixedShort];
#pragma unroll
    for (int i = 0; i < kMixedShort; ++i) l_pos[i] = positions_sorted[min(l_begin + i, l_end - 1)];
#pragma unroll
    for (int i = 0; i < kMixedShort; ++i) l_bag[i] = grad_rows[l_pos[i]];
    const int bag0 = bag_of(l_bag[0]);
    const int l_table = l_bag[0] - bag0 * num_tables;
#pragma unroll
    for (int i = 1; i < kMixedShort; ++i) l_bag[i] = bag_of(l_bag[i]);
    l_bag[0] = bag0;
    const int l_dim_start = dim_offsets[l_table];
    const int l_D = dim_offsets[l_table + 1] - l_dim_start;
    const int64_t l_row_element =
        table_offsets[l_table] + static_cast<int64_t>(l_key - table_dim_offsets[l_table]) * l_D;
    A l_state = A(0);
    if constexpr (OPT == kOptAdagrad) l_state = state[l_key];
    int64_t l_where = l_row_element;
    if constexpr (CACHED) {
      const int slot = unique_slots[my_u];
      if (slot >= 0) l_where = ~(static_cast<int64_t>(slot) * slot_D);
    }

    // Rows that are not reduced here.  Rows wider than 64 vectors go to a queue of row numbers
    // whatever their length (`wide_rows`, counters[2]; one atomic per strip).
    const bool is_wide = l_D / VEC > kWave;
    const bool is_long = lane < rows_here && (l_end - l_begin > kMixedShort || is_wide);
    const unsigned long long long_mask = __ballot(is_long);
    const unsigned long long wide_mask = __ballot(is_long && is_wide);
    if (wide_mask) {
      int first_slot = 0;
      if (lane == 0) first_slot = atomicAdd(&counters[2], __popcll(wide_mask));
      first_slot = shfl_idx(first_slot, 0);
      if (is_long && is_wide)
        wide_rows[first_slot + __popcll(wide_mask & ((1ull << lane) - 1ull))] = static_cast<int32_t>(my_u);
    }
    const unsigned long long queued_mask = long_mask & ~wide_mask;
    if constexpr (APPROX) {
      // the per-lookup form walks a row of many occurrences in one piece: its number goes to
      // `queued_rows` (counters[1]) -- or, an fp16 row of more than kApproxHuge occurrences that a
      // workgroup can walk, to the list behind that queue (counters[xcd_counter(0)])
      bool is_huge = false;
      if constexpr (sizeof(T) == 2) is_huge = is_long && !is_wide && l_end - l_begin > kApproxHuge && l_D <= kApproxCoopD;
      const unsigned long long huge_mask = __ballot(is_huge);
      const unsigned long long plain_mask = queued_mask & ~huge_mask;
      if (plain_mask) {
        int first_slot = 0;
        if (lane == 0) first_slot = atomicAdd(&counters[1], __popcll(plain_mask));
        first_slot = shfl_idx(first_slot, 0);
        if (is_long && !is_wide && !is_huge)
          queued_rows[first_slot + __popcll(plain_mask & ((1ull << lane) - 1ull))] = static_cast<int32_t>(my_u);
      }
      if (huge_mask) {
        int first_slot = 0;
        if (lane == 0) first_slot = atomicAdd(&counters[xcd_counter(0)], __popcll(huge_mask));
        first_slot = shfl_idx(first_slot, 0);
        if (is_huge)
          queued_rows[approx_huge_offset + first_slot + __popcll(huge_mask & ((1ull << lane) - 1ull))] =
              static_cast<int32_t>(my_u);
      }
    } else if (queued_mask) {
      // The exact update sums such a row in chunks of at most kChunkLen occurrences, like the uniform
      // tables' update: chunk records (and, for a row of several chunks, a list entry) in the queue
      // of the XCD whose eighth of the sorted positions the strip's first such row starts in, so
      // that update_chunks_mixed_kernel finds a table's hot rows -- and their gradient rows in L2 --
      // on one XCD.  One atomic add per strip takes the queue slots and list entries of all its
      // rows (atomic adds on one counter are served one after the other: one per row cost 40 us
      // with 27 k such rows); a row's share follows from a prefix sum over the lanes.  The records
      // of one row after the other are then written by the whole wavefront.
      const bool chunked = is_long && !is_wide;
      const int my_nch = chunked ? (l_end - l_begin + kChunkLen - 1) / kChunkLen : 0;
      // (fewer than 2^23 chunks and at most 64 rows in all: both sums fit one word)
      const int my_share = my_nch | (my_nch > 1 ? 1 << 24 : 0);
      int before = my_share;
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const int y = __shfl_up(before, d, kWave);
        if (lane >= d) before += y;
      }
      const int strip_total = shfl_idx(before, kWave - 1);
      before -= my_share;
      const int first_lane = __ffsll(static_cast<long long>(queued_mask)) - 1;
      const int queue_index = min(shfl_idx(l_begin, first_lane) / positions_per_xcd, kNumXcd - 1);
      unsigned long long taken = 0ull;
      if (lane == 0)
        taken = atomicAdd(reinterpret_cast<unsigned long long *>(counters + xcd_counter(queue_index)),
                          static_cast<unsigned long long>(strip_total & 0xffffff) |
                              (static_cast<unsigned long long>(strip_total >> 24) << 32));
      const int first_chunk_of_strip = shfl_idx(static_cast<int>(taken & 0xffffffffull), 0);
      const int first_entry_of_strip = shfl_idx(static_cast<int>(taken >> 32), 0);
      const int my_first_chunk = first_chunk_of_strip + (before & 0xffffff);
      if (my_nch > 1)
        long_records[queue_index * (max_long / kNumXcd) + first_entry_of_strip + (before >> 24)] =
            LongRecord{CACHED ? static_cast<int32_t>(my_u) : l_table, l_key, l_begin, l_end};
      ChunkRecord *queue = chunk_records + queue_index * (max_chunks / kNumXcd);
      for (unsigned long long rest = queued_mask; rest != 0ull; rest &= rest - 1ull) {
        const int src = __ffsll(static_cast<long long>(rest)) - 1;
        const int seg_begin = shfl_idx(l_begin, src), seg_end = shfl_idx(l_end, src);
        const int first_chunk = shfl_idx(my_first_chunk, src);
        const int nch = (seg_end - seg_begin + kChunkLen - 1) / kChunkLen;
        ChunkRecord rec;
        rec.key = shfl_idx(l_key, src);
        rec.u = static_cast<int32_t>(u0) + src;
        rec.pad[0] = shfl_idx(l_table, src);
        rec.pad[1] = rec.pad[2] = 0;
        for (int k = lane; k < nch; k += kWave) {
          rec.begin = seg_begin + k * kChunkLen;
          rec.end = min(seg_end, rec.begin + kChunkLen);
          rec.partial = nch > 1 ? partial_row_of_chunk(seg_begin, seg_end, k, nch) : -1;
          queue[first_chunk + k] = rec;
        }
      }
    }
    const unsigned long long todo = ~long_mask & (rows_here == kWave ? ~0ull : ((1ull << rows_here) - 1ull));
    if (todo == 0ull) continue;

    // records and occurrences to LDS; the k-th short row of the strip gets record k, the lanes
    // without a short row fill the records behind them with empty rows
    const bool is_short = (todo >> lane) & 1ull;
    const unsigned long long below = (1ull << lane) - 1ull;
    const int num_short = __popcll(todo);
    const int my_rank = is_short ? __popcll(todo & below) : num_short + __popcll(~todo & below);
    const int my_len = is_short ? l_end - l_begin : 0;
    int my_offset = my_len;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const int y = __shfl_up(my_offset, d, kWave);
      if (lane >= d) my_offset += y;
    }
    my_offset -= my_len;  // exclusive prefix: first occurrence slot of the row
    int st_lo = 0, st_hi = 0;
    if constexpr (sizeof(A) == 4) {
      st_lo = __builtin_bit_cast(int, l_state);
    } else {
      const long long bits = __builtin_bit_cast(long long, l_state);
      st_lo = static_cast<int>(bits);
      st_hi = static_cast<int>(bits >> 32);
    }
    s_row[wave][my_rank][0] = make_int4(my_len, my_offset, l_key, is_short ? l_D : 0);
    s_row[wave][my_rank][1] = make_int4(static_cast<int>(l_where), static_cast<int>(l_where >> 32), st_lo, st_hi);
    if constexpr (CACHED) s_element[wave][my_rank] = l_row_element;
#pragma unroll
    for (int i = 0; i < kMixedShort; ++i) {
      if (i < my_len) {
        s_goff[wave][my_offset + i] = l_bag[i] * total_D + l_dim_start;
        if constexpr (WEIGHTED) s_pos[wave][my_offset + i] = l_pos[i];
      }
    }
    int strip_D = is_short ? l_D : 0;
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) strip_D = max(strip_D, __shfl_xor(strip_D, m, kWave));
    __builtin_amdgcn_wave_barrier();

    const int max_chunks = strip_D / VEC;
    const int group_shift = max_chunks > 1 ? 32 - __builtin_clz(max_chunks - 1) : 0;
    const int group_lanes = 1 << group_shift;
    const int groups = kWave >> group_shift;
    const int r = lane >> group_shift;
    const int c = lane & (group_lanes - 1);
    const int col = c * VEC;

    // Two sets of requested data take turns, so that nothing is copied from one to the other.
    struct Fetched {
      R w;
      R raw[kMixedAhead];
      A pw[kMixedAhead];
    };
    auto request = [&](int k0, Fetched &f) {
      const int4 d0 = s_row[wave][k0 + r][0];
      const int4 d1 = s_row[wave][k0 + r][1];
      const int len = d0.x, slot0 = d0.y;
      const bool active = col < d0.w;
      const int64_t where =
          (static_cast<int64_t>(d1.y) << 32) | static_cast<int64_t>(static_cast<uint32_t>(d1.x));
      if (active) f.w = V::load_raw_streaming(stored_at(where) + col);
#pragma unroll
      for (int u = 0; u < kMixedAhead; ++u) {
        if (__ballot(u < len) == 0ull) break;
        if (u < len && active) {
          f.raw[u] = V::load_raw(grad_output + static_cast<int64_t>(s_goff[wave][slot0 + u]) + col);
          if constexpr (WEIGHTED) f.pw[u] = to_acc(psw[s_pos[wave][slot0 + u]]);
        }
      }
    };
    // The compiler has to finish the loads of f here: placed before the next request, it keeps the
    // wait for f from also waiting for that request.
    auto landed = [&](Fetched &f) {
      register_fence(f.w);
#pragma unroll
      for (int u = 0; u < kMixedAhead; ++u) {
        register_fence(f.raw[u]);
        if constexpr (WEIGHTED) register_fence(f.pw[u]);
      }
    };
    auto consume = [&](int k0, Fetched &f) {
      const int4 d0 = s_row[wave][k0 + r][0];
      const int4 d1 = s_row[wave][k0 + r][1];
      const int len = d0.x, slot0 = d0.y;
      const int32_t key = d0.z;
      const bool active = col < d0.w;
      const int64_t where =
          (static_cast<int64_t>(d1.y) << 32) | static_cast<int64_t>(static_cast<uint32_t>(d1.x));
      int64_t row_element = where;
      if constexpr (CACHED) row_element = s_element[wave][k0 + r];
      A state_old;
      if constexpr (sizeof(A) == 4) {
        state_old = __builtin_bit_cast(A, d1.z);
      } else {
        state_old = __builtin_bit_cast(
            A, (static_cast<long long>(d1.w) << 32) | static_cast<long long>(static_cast<uint32_t>(d1.z)));
      }
      V w_old, G, x;
      w_old.unpack(f.w);
      if constexpr (WEIGHTED) {  // lanes beside the row must not bring stale values into the dot products
#pragma unroll
        for (int i = 0; i < VEC; ++i) w_old.v[i] = active ? w_old.v[i] : A(0);
      }
      G.zero();
      A running = state_old;  // APPROX: the row's state after the occurrences applied so far
      auto add = [&](int u, const R &packed, A weight) {
        x.unpack(packed);
        const bool ok = u < len && active;
#pragma unroll
        for (int i = 0; i < VEC; ++i) x.v[i] = ok ? x.v[i] : A(0);
        if constexpr (APPROX) {
          // w_old is the row as the earlier occurrences left it
          A gss = A(0);
#pragma unroll
          for (int i = 0; i < VEC; ++i) gss += x.v[i] * x.v[i];
          for (int m = group_lanes >> 1; m > 0; m >>= 1) gss += shfl_x(gss, m);
          A mult = A(0);
          if (u < len) {
            if constexpr (!WEIGHTED) weight = A(1);
            running = running + (WEIGHTED ? gss * weight * weight : gss);
            mult = approx_multiplier<A>(running, weight, WEIGHTED, lr, eps);
          }
          if constexpr (WEIGHTED) {
            A dot = A(0);
#pragma unroll
            for (int i = 0; i < VEC; ++i) dot += w_old.v[i] * x.v[i];
            for (int m = group_lanes >> 1; m > 0; m >>= 1) dot += shfl_x(dot, m);
            if (u < len && c == 0) grad_psw[s_pos[wave][slot0 + u]] = from_acc<T, A>(dot);
          }
#pragma unroll
          for (int i = 0; i < VEC; ++i) w_old.v[i] = w_old.v[i] - x.v[i] * mult;
          round_trip<T, VEC>(w_old, rounding_of_update(sr, u), row_element + col);
        } else if constexpr (WEIGHTED) {
          weight = ok ? weight : A(1);
          A dot = A(0);
#pragma unroll
          for (int i = 0; i < VEC; ++i) dot += w_old.v[i] * x.v[i];
          for (int m = group_lanes >> 1; m > 0; m >>= 1) dot += shfl_x(dot, m);
          if (u < len && c == 0) grad_psw[s_pos[wave][slot0 + u]] = from_acc<T, A>(dot);
#pragma unroll
          for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * weight;
        } else {
#pragma unroll
          for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i];
        }
      };
#pragma unroll
      for (int u = 0; u < kMixedAhead; ++u) {
        if (__ballot(u < len) == 0ull) break;
        add(u, f.raw[u], f.pw[u]);
      }
      // occurrences kMixedAhead.. of the longer rows are fetched here
      for (int i0 = kMixedAhead; __ballot(i0 < len) != 0ull; i0 += kMixedAhead) {
        R raw[kMixedAhead];
        A pw[kMixedAhead];
#pragma unroll
        for (int u = 0; u < kMixedAhead; ++u) {
          pw[u] = A(1);
          if (i0 + u < len && active) {
            raw[u] = V::load_raw(grad_output + static_cast<int64_t>(s_goff[wave][slot0 + i0 + u]) + col);
            if constexpr (WEIGHTED) pw[u] = to_acc(psw[s_pos[wave][slot0 + i0 + u]]);
          }
        }
#pragma unroll
        for (int u = 0; u < kMixedAhead; ++u) add(i0 + u, raw[u], pw[u]);
      }
      if constexpr (APPROX) {
        if (len > 0 && c == 0) state[key] = running;
        // (fp16: the last occurrence already rounded the row to the stored type)
        if (len > 0 && active) w_old.store_streaming(stored_at(where) + col);
        return;
      }
      A mult = static_cast<A>(lr);
      if constexpr (OPT == kOptAdagrad) {
        A gss = A(0);
#pragma unroll
        for (int i = 0; i < VEC; ++i) gss += G.v[i] * G.v[i];
        for (int m = group_lanes >> 1; m > 0; m >>= 1) gss += shfl_x(gss, m);
        const A s_new = state_old + gss;
        if (len > 0 && c == 0) state[key] = s_new;
        mult = mixed_multiplier<A>(s_new, lr, eps);
      }
      if (active) {
        V w;
#pragma unroll
        for (int i = 0; i < VEC; ++i) w.v[i] = w_old.v[i] - G.v[i] * mult;
        store_row<T, VEC, true>(stored_at(where) + col, w, sr, row_element + col);
      }
    };
    Fetched fa{}, fb{};
    request(0, fa);
    for (int k0 = 0; k0 < num_short; k0 += 2 * groups) {
      landed(fa);
      if (k0 + groups < num_short) request(k0 + groups, fb);
      consume(k0, fa);
      if (k0 + groups < num_short) {
        landed(fb);
        if (k0 + 2 * groups < num_short) request(k0 + 2 * groups, fa);
        consume(k0 + groups, fb);
      }
    }
  }
}

// ------------------------------------------------ exact update: rows of many occurrences
__device__ __forceinline__ int bag_of_grad_row(int grow, const MixedTables &mt) {
  return static_cast<int>((static_cast<uint64_t>(static_cast<uint32_t>(grow)) * mt.bag_magic) >> mt.bag_shift);
}

// The chunk records of mixed-D tables: update_chunks_kernel's walk over the eight queues, each record
// reduced with its own table's row width.  A chunk that is a whole segment is applied to its row
// at once; a chunk of a longer segment stores its sum as a partial row of 64 vectors.
template <typename T, int VEC, int OPT, bool WEIGHTED, int UNROLL, bool CACHED>
__global__ __launch_bounds__(kBlockThreads) void update_chunks_mixed_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ counters,
    const ChunkRecord *__restrict__ chunk_records, int64_t max_chunks, const int32_t *__restrict__ wide_rows,
    typename AccOf<T>::type *__restrict__ partial_sums, float lr, float eps, StochasticRounding sr,
    MixedTables mt, const int32_t *__restrict__ unique_slots, T *__restrict__ cache_rows, int slot_D) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  const int lane = threadIdx.x & (kWave - 1);
  const int xcd = blockIdx.x % kNumXcd;
  const int64_t queue_capacity = max_chunks / kNumXcd;
  // an XCD drains its own queue up to one and a half times the average queue length, the rest is
  // dealt to the wavefronts of all XCDs (see update_chunks_kernel)
  int queue_len[kNumXcd];
  int64_t total = 0;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) {
    queue_len[x] = counters[xcd_counter(x)];
    total += queue_len[x];
  }
  const int fair = static_cast<int>(total / kNumXcd + total / 16 + 1);
  int64_t shared_total = 0;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) shared_total += max(0, queue_len[x] - fair);
  const int own = min(queue_len[xcd], fair);
  int64_t q = static_cast<int64_t>(blockIdx.x / kNumXcd) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x / kNumXcd) * kWavesPerBlock;
  int64_t g = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t shared_stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  while (true) {
    const ChunkRecord *next;
    if (q < own) {
      next = chunk_records + xcd * queue_capacity + q;
      q += stride;
    } else if (g < shared_total) {
      int64_t before = 0;
      int x = 0;
      while (g >= before + max(0, queue_len[x] - fair)) {
        before += max(0, queue_len[x] - fair);
        ++x;
      }
      next = chunk_records + x * queue_capacity + fair + (g - before);
      g += shared_stride;
    } else {
      break;
    }
    const ChunkRecord rec = *next;
    const int t = rec.pad[0];
    MixedRow row;
    row.seg_begin = rec.begin;
    row.seg_end = rec.end;
    row.key = rec.key;
    row.dim_start = mt.dim_offsets[t];
    row.D = mt.dim_offsets[t + 1] - row.dim_start;
    row.row_element = mt.table_offsets[t] + static_cast<int64_t>(rec.key - mt.table_dim_offsets[t]) * row.D;
    locate_row<CACHED>(row, weights, unique_slots, rec.u, cache_rows, slot_D);
    A state_old = A(0);
    if constexpr (OPT == kOptAdagrad) {
      if (rec.partial < 0) state_old = state[rec.key];
    }
    V w_old, G;
    mixed_accumulate_narrow<T, VEC, WEIGHTED, UNROLL>(grad_output, psw, grad_psw, mt.T, mt.total_D,
                                                      positions_sorted, grad_rows, lane, row, 0, 1, w_old, G);
    if (rec.partial >= 0) {
      if (lane < row.D / VEC) {
        A *dst = partial_sums + static_cast<int64_t>(rec.partial) * (kWave * VEC) + static_cast<int64_t>(lane) * VEC;
#pragma unroll
        for (int i = 0; i < VEC; ++i) dst[i] = G.v[i];
      }
    } else {
      mixed_apply_narrow<T, VEC, OPT>(state, lr, eps, sr, lane, row, state_old, w_old, G);
    }
  }
  // the rows wider than 64 vectors, a wavefront each (their number: counters[2])
  const int num_wide = counters[2];
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6); i < num_wide; i += shared_stride) {
    const int u = wide_rows[i];
    MixedRow row;
    row.seg_begin = segment_starts[u];
    row.seg_end = segment_starts[u + 1];
    row.key = keys_sorted[row.seg_begin];
    const int grow = grad_rows[positions_sorted[row.seg_begin]];
    const int t = grow - bag_of_grad_row(grow, mt) * mt.T;
    row.dim_start = mt.dim_offsets[t];
    row.D = mt.dim_offsets[t + 1] - row.dim_start;
    row.row_element = mt.table_offsets[t] + static_cast<int64_t>(row.key - mt.table_dim_offsets[t]) * row.D;
    locate_row<CACHED>(row, weights, unique_slots, u, cache_rows, slot_D);
    A state_old = A(0);
    if constexpr (OPT == kOptAdagrad) state_old = state[row.key];
    mixed_update_wide<T, VEC, OPT, WEIGHTED>(grad_output, state, psw, grad_psw, mt.T, mt.total_D,
                                             positions_sorted, grad_rows, lr, eps, sr, lane, row, state_old);
  }
}

// The rows of several chunks of mixed-D tables: one wavefront per row adds its partial rows in
// chunk order (lane group r takes partial rows r, r + groups, ..., the groups are combined in a
// fixed tree) and applies the optimizer.  The list records carry the row's table in `u` -- or,
// CACHED, the row's number, and the table follows from the gradient row of its first occurrence.
template <typename T, int VEC, int OPT, bool CACHED>
__global__ __launch_bounds__(kBlockThreads) void update_long_finish_mixed_kernel(
    T *__restrict__ weights, typename AccOf<T>::type *__restrict__ state,
    const int32_t *__restrict__ counters, const LongRecord *__restrict__ long_records,
    const typename AccOf<T>::type *__restrict__ partial_sums, float lr, float eps, StochasticRounding sr,
    int64_t max_long, MixedTables mt, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ unique_slots, T *__restrict__ cache_rows,
    int slot_D) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  const int lane = threadIdx.x & (kWave - 1);
  const LongLists lists = long_lists(counters, max_long);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t slot = wave_id; slot < lists.total; slot += stride) {
    const LongRecord rec = long_record_at(long_records, lists, slot);
    int t = rec.u;
    if constexpr (CACHED) {
      const int grow = grad_rows[positions_sorted[rec.begin]];
      t = grow - bag_of_grad_row(grow, mt) * mt.T;
    }
    MixedRow row;
    row.seg_begin = rec.begin;
    row.seg_end = rec.end;
    row.key = rec.key;
    row.dim_start = mt.dim_offsets[t];
    row.D = mt.dim_offsets[t + 1] - row.dim_start;
    row.row_element = mt.table_offsets[t] + static_cast<int64_t>(rec.key - mt.table_dim_offsets[t]) * row.D;
    locate_row<CACHED>(row, weights, unique_slots, rec.u, cache_rows, slot_D);
    const int chunks = row.D / VEC;
    const int group_shift = chunks > 1 ? 32 - __builtin_clz(chunks - 1) : 0;
    const int group_lanes = 1 << group_shift;
    const int groups = kWave >> group_shift;
    const int r = lane >> group_shift;
    const int c = lane & (group_lanes - 1);
    const bool active = c < chunks;
    const int64_t col = active ? static_cast<int64_t>(c) * VEC : 0;
    const int num_chunks = (rec.end - rec.begin + kChunkLen - 1) / kChunkLen;
    V w_old;
    w_old.zero();
    if (lane < chunks) w_old.load(static_cast<const T *>(row.where) + col);
    A state_old = A(0);
    if constexpr (OPT == kOptAdagrad) state_old = state[rec.key];
    V G;
    G.zero();
    constexpr int kAhead = 8;
    for (int k0 = r; k0 < num_chunks; k0 += groups * kAhead) {
      A part[kAhead][VEC];
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        const int k = min(k0 + a * groups, num_chunks - 1);  // clamped: no branch per load
        const A *src = partial_sums +
                       static_cast<int64_t>(partial_row_of_chunk(rec.begin, rec.end, k, num_chunks)) * (kWave * VEC) + col;
#pragma unroll
        for (int i = 0; i < VEC; ++i) part[a][i] = src[i];
      }
#pragma unroll
      for (int a = 0; a < kAhead; ++a) {
        const bool real = active && k0 + a * groups < num_chunks;
#pragma unroll
        for (int i = 0; i < VEC; ++i) G.v[i] += real ? part[a][i] : A(0);
      }
    }
    for (int m = kWave >> 1; m >= group_lanes; m >>= 1) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) G.v[i] += shfl_x(G.v[i], m);
    }
    mixed_apply_narrow<T, VEC, OPT>(state, lr, eps, sr, lane, row, state_old, w_old, G);
  }
}

struct MixedArgs {
  const void *grad_output;
  void *weights;
  int32_t dtype;
  int32_t vec;  // elements per 16-byte (or 8-byte) vector, valid for every table
  const int64_t *table_offsets;
  const int32_t *table_dim_offsets;
  const int32_t *dim_offsets;
  int32_t total_D;
  int32_t T;
  const int32_t *indices;
  int64_t n;
  const int32_t *offsets;
  int32_t B;
  const void *psw;
  void *output;
  void *state;
  void *grad_psw;
  float lr, eps;
  int optimizer;
  StochasticRounding sr;
  // tables fronted by the row cache (null otherwise): where every lookup / every unique row lives,
  // the cache's rows and their width
  const int32_t *lookup_slots;
  const int32_t *unique_slots;
  void *cache_rows;
  int32_t slot_D;
};

template <typename T, int VEC>
void launch_forward_mixed(const MixedArgs &a, hipStream_t stream) {
  const int num_bags = a.T * a.B;
  const int64_t per_xcd = ceil_div(ceil_div(num_bags, kWavesPerBlock), kNumXcd);
  const dim3 grid(static_cast<unsigned>(per_xcd * kNumXcd)), block(kBlockThreads);
  const T *w = static_cast<const T *>(a.weights);
  const T *p = static_cast<const T *>(a.psw);
  T *o = static_cast<T *>(a.output);
  const T *cr = static_cast<const T *>(a.cache_rows);
#define TBE_FORWARD_MIXED(WEIGHTED, CACHED)                                                                     \
  TBE_LAUNCH("forward_mixed", stream, (forward_mixed_kernel<T, VEC, WEIGHTED, 8, CACHED>), grid, block, w,      \
             a.table_offsets, a.dim_offsets, a.indices, a.offsets, p, o, a.B, a.total_D, num_bags, per_xcd,     \
             a.lookup_slots, cr, a.slot_D)
  if (a.lookup_slots) {
    if (a.psw) TBE_FORWARD_MIXED(true, true);
    else TBE_FORWARD_MIXED(false, true);
  } else {
    if (a.psw) TBE_FORWARD_MIXED(true, false);
    else TBE_FORWARD_MIXED(false, false);
  }
#undef TBE_FORWARD_MIXED
}

// The exact update: the strip kernel for the rows of few occurrences, then one wavefront per chunk
// record (and per row wider than 64 vectors), then the rows of several chunks.
template <typename T, int VEC, int OPT, bool WEIGHTED, bool CACHED>
void launch_update_mixed(const MixedArgs &a, const tbe_workspace_layout_t &l, char *ws, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  T *cr = static_cast<T *>(a.cache_rows);
  auto i32 = [&](uint64_t off) { return reinterpret_cast<int32_t *>(ws + off); };
  const T *go = static_cast<const T *>(a.grad_output);
  T *w = static_cast<T *>(a.weights);
  A *st = static_cast<A *>(a.state);
  const T *psw = static_cast<const T *>(a.psw);
  T *gpsw = static_cast<T *>(a.grad_psw);
  A *partial = reinterpret_cast<A *>(ws + l.partial_sums);
  LongRecord *long_records = reinterpret_cast<LongRecord *>(ws + l.long_segments);
  ChunkRecord *chunk_records = reinterpret_cast<ChunkRecord *>(ws + l.chunk_segments);
  const int64_t max_chunks = static_cast<int64_t>(l.max_chunks);
  const int64_t max_long = static_cast<int64_t>(l.max_long_segments);
  // numbers of the rows wider than 64 vectors (at most one per lookup; the exact update of
  // these tables does not use the segment of every position)
  int32_t *wide_rows = i32(l.segment_ids);
  MixedTables mt{a.table_offsets, a.table_dim_offsets, a.dim_offsets, a.total_D, a.T};
  set_bag_division(mt);
  const dim3 block(kBlockThreads);
  const int64_t want = ceil_div(ceil_div(a.n, kWave), kWavesPerBlock);
  const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 32))));
  TBE_LAUNCH("update_mixed", stream, (update_mixed_kernel<T, VEC, OPT, WEIGHTED, false, CACHED>), grid, block,
             go, w, st, psw, gpsw, a.table_offsets, a.table_dim_offsets, a.dim_offsets, a.T, mt.bag_magic, mt.bag_shift,
             a.total_D, i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),
             i32(l.num_unique), wide_rows, static_cast<int32_t *>(nullptr), chunk_records, long_records, max_chunks,
             max_long, static_cast<int>(ceil_div(a.n, kNumXcd)), a.lr, a.eps, a.sr, 0, a.unique_slots, cr, a.slot_D);

  const bool small = ceil_div(a.n, tile_positions(0)) < kSmallBatchTiles;
  const int64_t want_chunks = ceil_div(max_chunks, kWavesPerBlock);
  // a multiple of the XCD count, so that every XCD gets as many workgroups (few for a small batch)
  const dim3 grid_chunks(static_cast<unsigned>(
      kNumXcd * std::max<int64_t>(1, std::min<int64_t>(ceil_div(want_chunks, kNumXcd), small ? 64 : 1024))));
  TBE_LAUNCH("update_chunks_mixed", stream,
             (update_chunks_mixed_kernel<T, VEC, OPT, WEIGHTED, (WEIGHTED && VEC == 8) ? 4 : 8, CACHED>), grid_chunks,
             block, go, w, st, psw, gpsw, i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows),
             i32(l.segment_starts), i32(l.num_unique), chunk_records, max_chunks, wide_rows, partial, a.lr, a.eps, a.sr,
             mt, a.unique_slots, cr, a.slot_D);

  const int64_t want_long = ceil_div(max_long, kWavesPerBlock);
  const dim3 grid_finish(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_long, 256 * 4))));
  TBE_LAUNCH("update_long_finish_mixed", stream, (update_long_finish_mixed_kernel<T, VEC, OPT, CACHED>), grid_finish,
             block, w, st, i32(l.num_unique), long_records, partial, a.lr, a.eps, a.sr, max_long, mt,
             i32(l.positions_sorted), i32(l.grad_rows), a.unique_slots, cr, a.slot_D);
}

// The approximate update's strip kernel: rows of at most 64 vectors and kMixedShort occurrences
// are applied, the others queued for approx_update.
template <typename T, int VEC, bool WEIGHTED, bool CACHED>
void launch_update_mixed_approx(const MixedArgs &a, const tbe_workspace_layout_t &l, char *ws, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  auto i32 = [&](uint64_t off) { return reinterpret_cast<int32_t *>(ws + off); };
  const int64_t want = ceil_div(ceil_div(a.n, kWave), kWavesPerBlock);
  const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 32))));
  int log2_T = 0;
  while ((int64_t{1} << log2_T) < a.T) ++log2_T;
  const int bag_shift = 31 + log2_T;
  const uint32_t bag_magic =
      static_cast<uint32_t>(((uint64_t{1} << bag_shift) + static_cast<uint64_t>(a.T) - 1) / static_cast<uint64_t>(a.T));
  TBE_LAUNCH("update_mixed_approx", stream, (update_mixed_kernel<T, VEC, kOptAdagrad, WEIGHTED, true, CACHED>), grid,
             dim3(kBlockThreads), static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights),
             static_cast<A *>(a.state), static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw),
             a.table_offsets, a.table_dim_offsets, a.dim_offsets, a.T, bag_magic, bag_shift, a.total_D,
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),
             i32(l.num_unique), approx_mixed_wide_queue(l, ws), approx_mixed_long_queue(l, ws),
             static_cast<ChunkRecord *>(nullptr), static_cast<LongRecord *>(nullptr), int64_t{0}, int64_t{0}, 1, a.lr,
             a.eps, a.sr, static_cast<int>(approx_mixed_huge_offset(a.n)), a.unique_slots,
             static_cast<T *>(a.cache_rows), a.slot_D);
}

template <typename T, int VEC>
void launch_update_mixed_approx_variant(const MixedArgs &a, const tbe_workspace_layout_t &l, char *ws,
                                        hipStream_t stream) {
  if (a.unique_slots) {
    if (a.psw) launch_update_mixed_approx<T, VEC, true, true>(a, l, ws, stream);
    else launch_update_mixed_approx<T, VEC, false, true>(a, l, ws, stream);
  } else {
    if (a.psw) launch_update_mixed_approx<T, VEC, true, false>(a, l, ws, stream);
    else launch_update_mixed_approx<T, VEC, false, false>(a, l, ws, stream);
  }
}

template <typename T, int VEC>
void launch_update_mixed_variant(const MixedArgs &a, const tbe_workspace_layout_t &l, char *ws,
                                 hipStream_t stream) {
  const bool weighted = a.psw != nullptr;
  if (a.unique_slots) {
    if (a.optimizer == kOptSgd) {
      if (weighted) launch_update_mixed<T, VEC, kOptSgd, true, true>(a, l, ws, stream);
      else launch_update_mixed<T, VEC, kOptSgd, false, true>(a, l, ws, stream);
    } else {
      if (weighted) launch_update_mixed<T, VEC, kOptAdagrad, true, true>(a, l, ws, stream);
      else launch_update_mixed<T, VEC, kOptAdagrad, false, true>(a, l, ws, stream);
    }
    return;
  }
  if (a.optimizer == kOptSgd) {
    if (weighted) launch_update_mixed<T, VEC, kOptSgd, true, false>(a, l, ws, stream);
    else launch_update_mixed<T, VEC, kOptSgd, false, false>(a, l, ws, stream);
  } else {
    if (weighted) launch_update_mixed<T, VEC, kOptAdagrad, true, false>(a, l, ws, stream);
    else launch_update_mixed<T, VEC, kOptAdagrad, false, false>(a, l, ws, stream);
  }
}

int validate_mixed(const char *name, const MixedArgs &a) {
  TBE_REQUIRE(a.T > 0, "%s: T must be positive (got %d)", name, a.T);
  TBE_REQUIRE(a.B > 0, "%s: B must be positive (got %d)", name, a.B);
  TBE_REQUIRE(a.total_D > 0 && a.total_D % 4 == 0, "%s: total_D must be a positive multiple of 4 (got %d)", name,
              a.total_D);
  TBE_REQUIRE(a.dtype >= TBE_DTYPE_F32 && a.dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, a.dtype);
  TBE_REQUIRE(a.dtype != TBE_DTYPE_F16 || a.vec == 4 || a.vec == 8, "%s: fp16 vector width must be 4 or 8", name);
  TBE_REQUIRE(a.n >= 0 && a.n < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(a.T) * a.B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(a.weights && a.table_offsets && a.dim_offsets && a.offsets, "%s: null pointer argument", name);
  TBE_REQUIRE(a.indices || a.n == 0, "%s: indices is null but num_indices > 0", name);
  return TBE_OK;
}

}  // namespace
}  // namespace tbe

extern "C" int tbe_forward_mixed(const void *weights, int32_t dtype, int32_t fp16_vector_width,
                                 const int64_t *table_offsets, const int32_t *dim_offsets,
                                 int32_t total_D, int32_t T, const int32_t *indices,
                                 int64_t num_indices, const int32_t *offsets, int32_t B,
                                 const void *per_sample_weights, void *output, void *stream) {
  using namespace tbe;
  MixedArgs a{};
  a.weights = const_cast<void *>(weights);
  a.dtype = dtype;
  a.vec = fp16_vector_width;
  a.table_offsets = table_offsets;
  a.dim_offsets = dim_offsets;
  a.total_D = total_D;
  a.T = T;
  a.indices = indices;
  a.n = num_indices;
  a.offsets = offsets;
  a.B = B;
  a.psw = per_sample_weights;
  a.output = output;
  if (int rc = validate_mixed("tbe_forward_mixed", a)) return rc;
  TBE_REQUIRE(output, "tbe_forward_mixed: null output");
  hipStream_t s = static_cast<hipStream_t>(stream);
  switch (dtype) {
    case TBE_DTYPE_F32: launch_forward_mixed<float, 4>(a, s); break;
    case TBE_DTYPE_F16:
      if (a.vec == 8) launch_forward_mixed<__half, 8>(a, s);
      else launch_forward_mixed<__half, 4>(a, s);
      break;
    default: launch_forward_mixed<double, 2>(a, s); break;
  }
  return check_launch("tbe_forward_mixed");
}

extern "C" int tbe_backward_mixed_workspace_layout(int64_t num_indices, int32_t dtype, int32_t T,
                                                   tbe_workspace_layout_t *layout) {
  using namespace tbe;
  const char *name = "tbe_backward_mixed_workspace_layout";
  TBE_REQUIRE(layout, "%s: null layout", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(T > 0, "%s: T must be positive (got %d)", name, T);
  backward_layout(num_indices, mixed_layout_dim(dtype), dtype, T, layout);
  return TBE_OK;
}

extern "C" int tbe_backward_mixed(int32_t optimizer, const void *grad_output, void *weights,
                                  int32_t dtype, int32_t fp16_vector_width, int64_t total_rows,
                                  int64_t max_table_rows, const int64_t *table_offsets, const int32_t *table_dim_offsets,
                                  const int32_t *dim_offsets, int32_t total_D, int32_t T,
                                  const int32_t *indices, int64_t num_indices,
                                  const int32_t *offsets, int32_t B,
                                  const void *per_sample_weights, void *optimizer_state,
                                  float learning_rate, float eps, void *grad_per_sample_weights,
                                  int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                  void *workspace, uint64_t workspace_bytes, void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_mixed";
  MixedArgs a{};
  a.grad_output = grad_output;
  a.weights = weights;
  a.dtype = dtype;
  a.vec = fp16_vector_width;
  a.table_offsets = table_offsets;
  a.table_dim_offsets = table_dim_offsets;
  a.dim_offsets = dim_offsets;
  a.total_D = total_D;
  a.T = T;
  a.indices = indices;
  a.n = num_indices;
  a.offsets = offsets;
  a.B = B;
  a.psw = per_sample_weights;
  a.state = optimizer_state;
  a.grad_psw = grad_per_sample_weights;
  a.lr = learning_rate;
  a.eps = eps;
  a.sr = StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0};
  TBE_REQUIRE(optimizer == TBE_OPT_SGD || optimizer == TBE_OPT_ROWWISE_ADAGRAD ||
                  optimizer == TBE_OPT_APPROX_ROWWISE_ADAGRAD,
              "%s: bad optimizer %d", name, optimizer);
  a.optimizer = optimizer == TBE_OPT_SGD ? kOptSgd : kOptAdagrad;
  if (int rc = validate_mixed(name, a)) return rc;
  TBE_REQUIRE(grad_output && table_dim_offsets, "%s: null pointer argument", name);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(static_cast<int64_t>(B) * total_D < INT32_MAX, "%s: grad_output of B*total_D = %lld elements is too large",
              name, static_cast<long long>(B) * total_D);
  TBE_REQUIRE(a.optimizer == kOptSgd || optimizer_state, "%s: optimizer_state is null", name);
  TBE_REQUIRE((per_sample_weights == nullptr) == (grad_per_sample_weights == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, mixed_layout_dim(dtype), dtype, T, &l);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *ws = static_cast<char *>(workspace);
  auto i32 = [&](uint64_t off) { return reinterpret_cast<int32_t *>(ws + off); };
  // every table's indices are sorted on their own; the last pass adds the table's first row id.
  // The sort's first launch also records the gradient row b*T + t of every position.
  int rc = sort_batch(l, workspace, table_dim_offsets, T, indices, num_indices, offsets, B, total_rows,
                      max_table_rows, s);
  if (rc) return rc;
  rc = find_segments(i32(l.keys_sorted), num_indices, i32(l.segment_starts), i32(l.num_unique), nullptr,
                     ws + l.segment_scratch, s, /*clear_queue_counters=*/true);
  if (rc) return rc;
  if (optimizer == TBE_OPT_APPROX_ROWWISE_ADAGRAD) {
    switch (dtype) {
      case TBE_DTYPE_F32: launch_update_mixed_approx_variant<float, 4>(a, l, ws, s); break;
      case TBE_DTYPE_F16:
        if (a.vec == 8) launch_update_mixed_approx_variant<__half, 8>(a, l, ws, s);
        else launch_update_mixed_approx_variant<__half, 4>(a, l, ws, s);
        break;
      default: launch_update_mixed_approx_variant<double, 2>(a, l, ws, s); break;
    }
    return approx_update(grad_output, weights, optimizer_state, per_sample_weights, grad_per_sample_weights,
                         dtype, dtype == TBE_DTYPE_F16 ? a.vec : (dtype == TBE_DTYPE_F32 ? 4 : 2), 0, num_indices,
                         learning_rate, eps, table_offsets, table_dim_offsets, dim_offsets, total_D, T, offsets, B, a.sr, l,
                         workspace, s);
  }
  switch (dtype) {
    case TBE_DTYPE_F32: launch_update_mixed_variant<float, 4>(a, l, ws, s); break;
    case TBE_DTYPE_F16:
      if (a.vec == 8) launch_update_mixed_variant<__half, 8>(a, l, ws, s);
      else launch_update_mixed_variant<__half, 4>(a, l, ws, s);
      break;
    default: launch_update_mixed_variant<double, 2>(a, l, ws, s); break;
  }
  return check_launch(name);
}

namespace tbe {
namespace {

int validate_mixed_cache(const char *name, const tbe_cache_t *cache, int32_t D, int32_t total_D) {
  TBE_REQUIRE(cache && cache->rows && cache->backing_rows, "%s: null cache", name);
  TBE_REQUIRE(cache->mixed_table_offsets && cache->mixed_table_rows && cache->mixed_dim_offsets && cache->mixed_T > 0,
              "%s: the cache does not describe tables of different widths (mixed_* fields)", name);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D, the width of a cache row, must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(D <= total_D, "%s: a cache row of %d elements is wider than all tables together (%d)", name, D, total_D);
  return TBE_OK;
}

}  // namespace
}  // namespace tbe

extern "C" int tbe_forward_mixed_cached(const tbe_cache_t *cache, int32_t dtype, int32_t fp16_vector_width, int32_t D,
                                        int32_t total_D, const int32_t *indices, int64_t num_indices,
                                        const int32_t *offsets, int32_t B, const void *per_sample_weights,
                                        const int32_t *lookup_slots, void *output, void *stream) {
  using namespace tbe;
  const char *name = "tbe_forward_mixed_cached";
  if (int rc = validate_mixed_cache(name, cache, D, total_D)) return rc;
  MixedArgs a{};
  a.weights = cache->backing_rows;
  a.dtype = dtype;
  a.vec = fp16_vector_width;
  a.table_offsets = cache->mixed_table_offsets;
  a.dim_offsets = cache->mixed_dim_offsets;
  a.total_D = total_D;
  a.T = cache->mixed_T;
  a.indices = indices;
  a.n = num_indices;
  a.offsets = offsets;
  a.B = B;
  a.psw = per_sample_weights;
  a.output = output;
  a.lookup_slots = lookup_slots;
  a.cache_rows = cache->rows;
  a.slot_D = D;
  if (int rc = validate_mixed(name, a)) return rc;
  TBE_REQUIRE(output, "%s: null output", name);
  TBE_REQUIRE(lookup_slots || num_indices == 0, "%s: null lookup_slots", name);
  hipStream_t s = static_cast<hipStream_t>(stream);  // (a batch without lookups reads no row: all zeros)
  switch (dtype) {
    case TBE_DTYPE_F32: launch_forward_mixed<float, 4>(a, s); break;
    case TBE_DTYPE_F16:
      if (a.vec == 8) launch_forward_mixed<__half, 8>(a, s);
      else launch_forward_mixed<__half, 4>(a, s);
      break;
    default: launch_forward_mixed<double, 2>(a, s); break;
  }
  return check_launch(name);
}

extern "C" int tbe_backward_mixed_cached(int32_t optimizer, const void *grad_output, const tbe_cache_t *cache,
                                         int32_t dtype, int32_t fp16_vector_width, int32_t D, int32_t total_D,
                                         int32_t B, int64_t num_indices, const int32_t *offsets,
                                         const void *per_sample_weights,
                                         void *optimizer_state, float learning_rate, float eps,
                                         void *grad_per_sample_weights, int32_t stochastic_rounding, uint64_t seed,
                                         uint64_t offset, void *workspace, uint64_t workspace_bytes,
                                         const int32_t *unique_slots, void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_mixed_cached";
  if (int rc = validate_mixed_cache(name, cache, D, total_D)) return rc;
  TBE_REQUIRE(optimizer == TBE_OPT_SGD || optimizer == TBE_OPT_ROWWISE_ADAGRAD ||
                  optimizer == TBE_OPT_APPROX_ROWWISE_ADAGRAD,
              "%s: bad optimizer %d", name, optimizer);
  TBE_REQUIRE(optimizer != TBE_OPT_APPROX_ROWWISE_ADAGRAD || offsets,
              "%s: the approximate update needs the batch's bag offsets", name);
  MixedArgs a{};
  a.grad_output = grad_output;
  a.weights = cache->backing_rows;
  a.dtype = dtype;
  a.vec = fp16_vector_width;
  a.table_offsets = cache->mixed_table_offsets;
  a.table_dim_offsets = cache->mixed_table_rows;
  a.dim_offsets = cache->mixed_dim_offsets;
  a.total_D = total_D;
  a.T = cache->mixed_T;
  a.n = num_indices;
  a.offsets = offsets;
  a.B = B;
  a.psw = per_sample_weights;
  a.state = optimizer_state;
  a.grad_psw = grad_per_sample_weights;
  a.lr = learning_rate;
  a.eps = eps;
  a.sr = StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0};
  a.optimizer = optimizer == TBE_OPT_SGD ? kOptSgd : kOptAdagrad;
  a.unique_slots = unique_slots;
  a.cache_rows = cache->rows;
  a.slot_D = D;
  TBE_REQUIRE(a.T > 0 && B > 0, "%s: T and B must be positive (got %d, %d)", name, a.T, B);
  TBE_REQUIRE(total_D > 0 && total_D % 4 == 0, "%s: total_D must be a positive multiple of 4 (got %d)", name, total_D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(dtype != TBE_DTYPE_F16 || a.vec == 4 || a.vec == 8, "%s: fp16 vector width must be 4 or 8", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(B) * total_D < INT32_MAX, "%s: grad_output of B*total_D = %lld elements is too large",
              name, static_cast<long long>(B) * total_D);
  TBE_REQUIRE(grad_output, "%s: null grad_output", name);
  TBE_REQUIRE(a.optimizer == kOptSgd || optimizer_state, "%s: optimizer_state is null", name);
  TBE_REQUIRE((per_sample_weights == nullptr) == (grad_per_sample_weights == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  TBE_REQUIRE(unique_slots || num_indices == 0, "%s: null unique_slots", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, mixed_layout_dim(dtype), dtype, a.T, &l);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *ws = static_cast<char *>(workspace);
  if (optimizer == TBE_OPT_APPROX_ROWWISE_ADAGRAD) {
    switch (dtype) {
      case TBE_DTYPE_F32: launch_update_mixed_approx_variant<float, 4>(a, l, ws, s); break;
      case TBE_DTYPE_F16:
        if (a.vec == 8) launch_update_mixed_approx_variant<__half, 8>(a, l, ws, s);
        else launch_update_mixed_approx_variant<__half, 4>(a, l, ws, s);
        break;
      default: launch_update_mixed_approx_variant<double, 2>(a, l, ws, s); break;
    }
    if (int rc = approx_update(grad_output, a.weights, optimizer_state, per_sample_weights, grad_per_sample_weights,
                               dtype, dtype == TBE_DTYPE_F16 ? a.vec : (dtype == TBE_DTYPE_F32 ? 4 : 2), 0, num_indices,
                               learning_rate, eps, a.table_offsets, a.table_dim_offsets, a.dim_offsets, total_D, a.T,
                               offsets, B, a.sr, l, workspace, s, unique_slots, cache->rows, D))
      return rc;
  } else {
    switch (dtype) {
      case TBE_DTYPE_F32: launch_update_mixed_variant<float, 4>(a, l, ws, s); break;
      case TBE_DTYPE_F16:
        if (a.vec == 8) launch_update_mixed_variant<__half, 8>(a, l, ws, s);
        else launch_update_mixed_variant<__half, 4>(a, l, ws, s);
        break;
      default: launch_update_mixed_variant<double, 2>(a, l, ws, s); break;
    }
  }
  if (int rc = check_launch(name)) return rc;
  return cache_unstage(cache, dtype, D, reinterpret_cast<const int32_t *>(ws + l.keys_sorted),
                       reinterpret_cast<const int32_t *>(ws + l.segment_starts),
                       reinterpret_cast<const int32_t *>(ws + l.num_unique), unique_slots, num_indices, s);
}
