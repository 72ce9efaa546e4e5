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
// One wavefront owns a bag (forward) or a unique row (backward) and its lanes stride over the
// row's 16-byte vectors, so any D_t works; these kernels are the general path and are not
// tuned per width like the uniform-D ones.  The integer stages (sort, segments) are shared.

#include <algorithm>

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

template <typename T, int VEC, bool WEIGHTED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void forward_mixed_kernel(
    const T *__restrict__ weights, const int64_t *__restrict__ table_offsets,
    const int32_t *__restrict__ dim_offsets, const int32_t *__restrict__ indices,
    const int32_t *__restrict__ offsets, const T *__restrict__ psw, T *__restrict__ output, int B,
    int total_D, int num_bags, int64_t blocks_per_xcd) {
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

  for (int cb = 0; cb < chunks; cb += kWave) {
    const int c = cb + lane;
    const bool ok_c = c < chunks;
    const T *col = table + static_cast<int64_t>(c) * VEC;
    V acc;
    acc.zero();
    for (int base = start; base < end; base += kWave) {
      const int n = min(kWave, end - base);
      int my_idx = 0;
      A my_w = A(0);
      if (lane < n) {
        my_idx = indices[base + lane];
        if constexpr (WEIGHTED) my_w = to_acc(psw[base + lane]);
      }
      for (int j0 = 0; j0 < n; j0 += UNROLL) {
        R raw[UNROLL];
        A w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int j = min(j0 + u, n - 1);
          const int64_t idx = shfl_idx(my_idx, j);
          if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, j);
          if (ok_c && j0 + u < n) raw[u] = V::load_raw(col + idx * D);
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
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

// keys[p] = table_dim_offsets[t] + indices[p] (skipped when `keys` is null); grad_rows[p] = b * T + t.
__global__ __launch_bounds__(kBlockThreads) void linearize_mixed_kernel(
    const int32_t *__restrict__ table_dim_offsets, const int32_t *__restrict__ indices,
    const int32_t *__restrict__ offsets, int B, int num_tables, int num_bags,
    int32_t *__restrict__ keys, int32_t *__restrict__ grad_rows) {
  constexpr int kLanes = 16;
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t bag64 = gid / kLanes;
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const int t = bag / B;
  const int b = bag - t * B;
  const int32_t grow = b * num_tables + t;
  const int end = offsets[bag + 1];
  if (keys) {
    const int32_t row0 = table_dim_offsets[t];
    for (int p = offsets[bag] + static_cast<int>(gid % kLanes); p < end; p += kLanes) {
      keys[p] = row0 + indices[p];
      grad_rows[p] = grow;
    }
  } else {
    for (int p = offsets[bag] + static_cast<int>(gid % kLanes); p < end; p += kLanes) grad_rows[p] = grow;
  }
}

// Everything a wavefront needs to know about one unique row.
struct MixedRow {
  int seg_begin, seg_end;  // sorted positions of its occurrences
  int32_t key;             // global row id (index of its optimizer state)
  int dim_start, D;        // first gradient column and width of its table
  int64_t row_element;     // element offset of the row in `weights`
};

// Narrow rows (at most 64 vectors): `chunks` = D / VEC consecutive lanes form a lane group, the
// 64 / chunks groups split the occurrences of a 64-position batch (the batch's positions,
// gradient rows and weights are fetched with one load per lane, then UNROLL independent
// gradient rows per group are in flight).  A wavefront takes the batches first_batch,
// first_batch + batch_stride, ...; its groups are combined into group 0 in a fixed tree.
// Returns with G (valid in group 0) and w_old (valid in every group when WEIGHTED, else in
// group 0).  pre_w / pre_g (have_pre): the packed row and the packed gradient row of the first
// occurrence, requested by the caller ahead of time; first_* (have_first): position, bag and
// weight of the first occurrence.
template <typename T, int VEC, bool WEIGHTED, int UNROLL>
__device__ __forceinline__ void mixed_accumulate_narrow(
    const T *__restrict__ grad_output, const T *__restrict__ weights, const T *__restrict__ psw,
    T *__restrict__ grad_psw, int num_tables, int total_D,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows, int lane,
    const MixedRow &row, int first_batch, int batch_stride, bool have_first, int first_pos,
    int first_bag, typename AccOf<T>::type first_w, bool have_pre,
    const typename RowVec<T, VEC>::R &pre_w, const typename RowVec<T, VEC>::R &pre_g,
    RowVec<T, VEC> &w_old, RowVec<T, VEC> &G) {
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
  const T *wrow = weights + row.row_element;
  const T *gcol = grad_output + row.dim_start;
  w_old.zero();
  if (have_pre) {
    if (active && (WEIGHTED || r == 0)) w_old.unpack(pre_w);
  } else if (active && (WEIGHTED || r == 0)) {
    w_old.load(wrow + col);
  }
  G.zero();
  for (int base = row.seg_begin + first_batch * kWave; base < row.seg_end; base += batch_stride * kWave) {
    const int n = min(kWave, row.seg_end - base);
    const bool first_batch_of_row = base == row.seg_begin;
    int my_pos = first_pos, my_bag = first_bag;
    A my_w = first_w;
    if (!have_first || n > 1 || !first_batch_of_row) {
      if (lane < n) {
        my_pos = positions_sorted[base + lane];
        my_bag = grad_rows[my_pos] / num_tables;
        if constexpr (WEIGHTED) my_w = to_acc(psw[my_pos]);
      }
    }
    for (int j0 = 0; j0 < n; j0 += groups * UNROLL) {
      R raw[UNROLL];
      bool ok[UNROLL];
      int src[UNROLL];
#pragma unroll
      for (int k = 0; k < UNROLL; ++k) {
        const int j = j0 + k * groups + r;
        ok[k] = active && j < n;
        src[k] = ok[k] ? j : 0;
        const int64_t bag = shfl_idx(my_bag, src[k]);
        if (ok[k]) {
          if (k == 0 && have_pre && first_batch_of_row && j == 0) raw[k] = pre_g;
          else raw[k] = V::load_raw(gcol + bag * total_D + col);
        }
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
        x.zero();
        if (ok[k]) x.unpack(raw[k]);
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
__device__ __forceinline__ void mixed_apply_narrow(T *__restrict__ weights,
                                                   typename AccOf<T>::type *__restrict__ state,
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
    const int64_t element = row.row_element + static_cast<int64_t>(lane) * VEC;
    store_row<T, VEC, false>(weights + element, w, sr, element);
  }
}

// Rows wider than 64 vectors, one wavefront: the passes of the reference's exact kernel (sum of
// squares first, then the update), one column block of 64 vectors at a time.
template <typename T, int VEC, int OPT, bool WEIGHTED>
__device__ __forceinline__ void mixed_update_wide(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
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
  T *wrow = weights + row_element;
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

// Short rows.  A wavefront takes strips of 64 consecutive unique rows.  What a row needs before
// its first gradient row can be requested -- segment bounds, key, first position, table (from
// the gradient row id b*T+t of the first occurrence), the table's width and offsets, optimizer
// state -- is fetched for the 64 rows at once, one row per lane, so the dependent loads are paid
// per strip; the rows and first gradient rows of four rows are requested before the first of them
// is reduced, so a row with one occurrence (the common case) waits for no load of its own.
// Rows of more than kShortSegment occurrences (the hot rows, which are neighbours in key order)
// are not reduced here: their indices go to two queues that update_mixed_long_kernel drains --
// one wavefront per row of at most kChunkLen occurrences, one workgroup of 16 wavefronts per
// longer row -- so that they spread over the machine.
template <typename T, int VEC, int OPT, bool WEIGHTED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void update_mixed_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int64_t *__restrict__ table_offsets,
    const int32_t *__restrict__ table_dim_offsets, const int32_t *__restrict__ dim_offsets,
    int num_tables, int total_D, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, int32_t *__restrict__ counters,
    int32_t *__restrict__ long_rows, int32_t *__restrict__ huge_rows, float lr, float eps,
    StochasticRounding sr) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  const int64_t num_strips = (static_cast<int64_t>(U) + kWave - 1) / kWave;

  for (int64_t strip = wave_id; strip < num_strips; strip += stride) {
    const int64_t u0 = strip * kWave;
    const int rows_here = static_cast<int>(min(static_cast<int64_t>(kWave), U - u0));
    // lane j holds the bookkeeping of row u0 + j (clamped: lanes past the end repeat the last row)
    const int64_t my_u = u0 + min(lane, rows_here - 1);
    const int l_begin = segment_starts[my_u];
    const int l_end = segment_starts[my_u + 1];
    const int32_t l_key = keys_sorted[l_begin];
    const int l_pos0 = positions_sorted[l_begin];
    const int l_grow0 = grad_rows[l_pos0];
    const int l_bag0 = l_grow0 / num_tables;
    const int l_table = l_grow0 - l_bag0 * num_tables;
    const int l_dim_start = dim_offsets[l_table];
    const int l_D = dim_offsets[l_table + 1] - l_dim_start;
    const int64_t l_row_element =
        table_offsets[l_table] + static_cast<int64_t>(l_key - table_dim_offsets[l_table]) * l_D;
    A l_state = A(0);
    if constexpr (OPT == kOptAdagrad) l_state = state[l_key];
    A l_w0 = A(1);
    if constexpr (WEIGHTED) l_w0 = to_acc(psw[l_pos0]);

    // hand the longer rows of the strip to their queues (one atomic per strip and queue)
    const bool is_long = lane < rows_here && l_end - l_begin > kShortSegment;
    const bool is_huge = is_long && l_end - l_begin > kChunkLen;
    const unsigned long long long_mask = __ballot(is_long);
    const unsigned long long huge_mask = __ballot(is_huge);
    const unsigned long long medium_mask = long_mask & ~huge_mask;
    if (medium_mask) {
      int first_slot = 0;
      if (lane == 0) first_slot = atomicAdd(&counters[2], __popcll(medium_mask));
      first_slot = shfl_idx(first_slot, 0);
      if (is_long && !is_huge)
        long_rows[first_slot + __popcll(medium_mask & ((1ull << lane) - 1ull))] = static_cast<int32_t>(my_u);
    }
    if (huge_mask) {
      int first_slot = 0;
      if (lane == 0) first_slot = atomicAdd(&counters[1], __popcll(huge_mask));
      first_slot = shfl_idx(first_slot, 0);
      if (is_huge) huge_rows[first_slot + __popcll(huge_mask & ((1ull << lane) - 1ull))] = static_cast<int32_t>(my_u);
    }

    // The bookkeeping of row j, read from lane j into scalar registers (j is the same in every lane).
    auto lane_i32 = [](int v, int j) { return __builtin_amdgcn_readlane(v, j); };
    auto lane_i64 = [&](int64_t v, int j) {
      const unsigned int lo = static_cast<unsigned int>(__builtin_amdgcn_readlane(static_cast<int>(v), j));
      const int hi = __builtin_amdgcn_readlane(static_cast<int>(v >> 32), j);
      return (static_cast<int64_t>(hi) << 32) | lo;
    };
    auto row_of = [&](int j) {
      return MixedRow{lane_i32(l_begin, j), lane_i32(l_end, j), lane_i32(l_key, j), lane_i32(l_dim_start, j),
                      lane_i32(l_D, j), lane_i64(l_row_element, j)};
    };
    // requests the packed row and the packed first gradient row of row j (narrow rows only)
    auto request = [&](int j, const MixedRow &row, R &w, R &g) {
      const int chunks = row.D / VEC;
      if (chunks > kWave) return false;
      const int group_shift = chunks > 1 ? 32 - __builtin_clz(chunks - 1) : 0;
      const int r = lane >> group_shift;
      const int c = lane & ((1 << group_shift) - 1);
      const int64_t col = static_cast<int64_t>(c) * VEC;
      const int64_t bag = lane_i32(l_bag0, j);
      if (c < chunks && (WEIGHTED || r == 0)) w = V::load_raw(weights + row.row_element + col);
      if (c < chunks && r == 0) g = V::load_raw(grad_output + row.dim_start + bag * total_D + col);
      return true;
    };

    // Short rows in blocks of kAhead: the loads of the whole block are requested before its first
    // row is reduced, so kAhead rows' worth of memory traffic is in flight per wavefront.
    constexpr int kAhead = 4;
    unsigned long long todo = ~long_mask & (rows_here == kWave ? ~0ull : ((1ull << rows_here) - 1ull));
    while (todo) {
      int index[kAhead];
      MixedRow rows[kAhead];
      R pre_w[kAhead], pre_g[kAhead];
      bool have_pre[kAhead];
#pragma unroll
      for (int p = 0; p < kAhead; ++p) {
        index[p] = -1;
        have_pre[p] = false;
        if (todo) {
          index[p] = __ffsll(static_cast<long long>(todo)) - 1;
          todo &= todo - 1;
          rows[p] = row_of(index[p]);
          have_pre[p] = request(index[p], rows[p], pre_w[p], pre_g[p]);
        }
      }
#pragma unroll
      for (int p = 0; p < kAhead; ++p) {
        if (index[p] < 0) continue;
        const int j = index[p];
        const A state_old = __builtin_bit_cast(A, [&] {
          if constexpr (sizeof(A) == 4) return lane_i32(__builtin_bit_cast(int, l_state), j);
          else return lane_i64(__builtin_bit_cast(int64_t, l_state), j);
        }());
        if (have_pre[p] && rows[p].seg_end - rows[p].seg_begin == 1) {
          // one occurrence, already requested: no batch to fetch, nothing to combine
          const int chunks = rows[p].D / VEC;
          V w_old, G;
          w_old.zero();
          G.zero();
          if (lane < chunks) {
            w_old.unpack(pre_w[p]);
            G.unpack(pre_g[p]);
          }
          if constexpr (WEIGHTED) {
            A dot = A(0);
#pragma unroll
            for (int i = 0; i < VEC; ++i) dot += w_old.v[i] * G.v[i];
            dot = group_sum<kWave, A>(dot, kWave, 0);  // lanes outside the row add 0
            if (lane == 0) grad_psw[lane_i32(l_pos0, j)] = from_acc<T, A>(dot);
            const A pw = shfl_idx(l_w0, j);
#pragma unroll
            for (int i = 0; i < VEC; ++i) G.v[i] *= pw;
          }
          mixed_apply_narrow<T, VEC, OPT>(weights, state, lr, eps, sr, lane, rows[p], state_old, w_old, G);
        } else if (rows[p].D / VEC <= kWave) {
          V w_old, G;
          mixed_accumulate_narrow<T, VEC, WEIGHTED, UNROLL>(
              grad_output, weights, psw, grad_psw, num_tables, total_D, positions_sorted, grad_rows, lane, rows[p], 0,
              1, true, lane_i32(l_pos0, j), lane_i32(l_bag0, j), shfl_idx(l_w0, j), have_pre[p], pre_w[p], pre_g[p],
              w_old, G);
          mixed_apply_narrow<T, VEC, OPT>(weights, state, lr, eps, sr, lane, rows[p], state_old, w_old, G);
        } else {
          mixed_update_wide<T, VEC, OPT, WEIGHTED>(grad_output, weights, state, psw, grad_psw, num_tables, total_D,
                                                   positions_sorted, grad_rows, lr, eps, sr, lane, rows[p], state_old);
        }
      }
    }
  }
}

// Queued rows: WAVES wavefronts per row (1, or kHugeWaves for the rows of more than kChunkLen
// occurrences).  The wavefronts of a row take its 64-position batches round-robin; their sums
// meet in LDS and the row's first wavefront adds them in wavefront order and applies the
// optimizer.  A row wider than 64 vectors is left to its first wavefront.  `queue_counter` is
// the index of the queue's length in `counters`.
constexpr int kHugeWaves = 16;
template <typename T, int VEC, int OPT, bool WEIGHTED, int UNROLL, int WAVES>
__global__ __launch_bounds__((WAVES > 1 ? WAVES : kWavesPerBlock) * kWave) void update_mixed_long_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int64_t *__restrict__ table_offsets,
    const int32_t *__restrict__ table_dim_offsets, const int32_t *__restrict__ dim_offsets,
    int num_tables, int total_D, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ counters,
    int queue_counter, const int32_t *__restrict__ queue, float lr, float eps, StochasticRounding sr) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;
  constexpr int kRowsPerBlock = WAVES > 1 ? 1 : kWavesPerBlock;
  __shared__ A s_partial[WAVES > 1 ? WAVES : 1][WAVES > 1 ? kWave * VEC : 1];
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int wave_in_row = WAVES > 1 ? wave : 0;
  const int num_queued = counters[queue_counter];
  for (int64_t q = static_cast<int64_t>(blockIdx.x) * kRowsPerBlock + (WAVES > 1 ? 0 : wave); q < num_queued;
       q += static_cast<int64_t>(gridDim.x) * kRowsPerBlock) {
    const int u = queue[q];
    MixedRow row;
    row.seg_begin = segment_starts[u];
    row.seg_end = segment_starts[u + 1];
    row.key = keys_sorted[row.seg_begin];
    const int table = grad_rows[positions_sorted[row.seg_begin]] % num_tables;
    row.dim_start = dim_offsets[table];
    row.D = dim_offsets[table + 1] - row.dim_start;
    row.row_element = table_offsets[table] + static_cast<int64_t>(row.key - table_dim_offsets[table]) * row.D;
    A state_old = A(0);
    if constexpr (OPT == kOptAdagrad) state_old = state[row.key];
    const int chunks = row.D / VEC;
    if (chunks > kWave) {
      if (wave_in_row == 0)
        mixed_update_wide<T, VEC, OPT, WEIGHTED>(grad_output, weights, state, psw, grad_psw, num_tables, total_D,
                                                 positions_sorted, grad_rows, lr, eps, sr, lane, row, state_old);
      continue;
    }
    V w_old, G;
    const R none{};
    mixed_accumulate_narrow<T, VEC, WEIGHTED, UNROLL>(grad_output, weights, psw, grad_psw, num_tables, total_D,
                                                      positions_sorted, grad_rows, lane, row, wave_in_row, WAVES,
                                                      false, 0, 0, A(1), false, none, none, w_old, G);
    if constexpr (WAVES > 1) {
      __syncthreads();  // the previous row's partial sums have been read
      if (lane < chunks) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) s_partial[wave][lane * VEC + i] = G.v[i];
      }
      __syncthreads();
      if (wave == 0 && lane < chunks) {
        for (int w = 1; w < WAVES; ++w) {
#pragma unroll
          for (int i = 0; i < VEC; ++i) G.v[i] += s_partial[w][lane * VEC + i];
        }
      }
    }
    if (wave_in_row == 0)
      mixed_apply_narrow<T, VEC, OPT>(weights, state, lr, eps, sr, lane, row, state_old, w_old, G);
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
};

template <typename T, int VEC>
void launch_forward_mixed(const MixedArgs &a, hipStream_t stream) {
  const int num_bags = a.T * a.B;
  const int64_t per_xcd = ceil_div(ceil_div(num_bags, kWavesPerBlock), kNumXcd);
  const dim3 grid(static_cast<unsigned>(per_xcd * kNumXcd)), block(kBlockThreads);
  const T *w = static_cast<const T *>(a.weights);
  const T *p = static_cast<const T *>(a.psw);
  T *o = static_cast<T *>(a.output);
  if (a.psw)
    TBE_LAUNCH("forward_mixed", stream, (forward_mixed_kernel<T, VEC, true, 4>), grid, block, w,
               a.table_offsets, a.dim_offsets, a.indices, a.offsets, p, o, a.B, a.total_D, num_bags, per_xcd);
  else
    TBE_LAUNCH("forward_mixed", stream, (forward_mixed_kernel<T, VEC, false, 4>), grid, block, w,
               a.table_offsets, a.dim_offsets, a.indices, a.offsets, p, o, a.B, a.total_D, num_bags, per_xcd);
}

template <typename T, int VEC, int OPT, bool WEIGHTED>
void launch_update_mixed(const MixedArgs &a, const tbe_workspace_layout_t &l, char *ws, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  auto i32 = [&](uint64_t off) { return reinterpret_cast<int32_t *>(ws + off); };
  const T *go = static_cast<const T *>(a.grad_output);
  T *w = static_cast<T *>(a.weights);
  A *st = static_cast<A *>(a.state);
  const T *psw = static_cast<const T *>(a.psw);
  T *gpsw = static_cast<T *>(a.grad_psw);
  // queues of row indices: rows of 17..256 occurrences (at most n / 17 of them) and longer rows (n / 257)
  int32_t *long_rows = i32(l.chunk_segments);
  int32_t *huge_rows = i32(l.long_segments);
  const int64_t want = ceil_div(ceil_div(a.n, kWave), kWavesPerBlock);
  const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 32))));
  TBE_LAUNCH("update_mixed", stream, (update_mixed_kernel<T, VEC, OPT, WEIGHTED, 4>), grid, dim3(kBlockThreads),
             go, w, st, psw, gpsw, a.table_offsets, a.table_dim_offsets, a.dim_offsets, a.T, a.total_D,
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),
             i32(l.num_unique), long_rows, huge_rows, a.lr, a.eps, a.sr);
  const int64_t want_long = ceil_div(a.n / (kShortSegment + 1) + 1, kWavesPerBlock);
  const dim3 grid_long(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_long, 256 * 8))));
  TBE_LAUNCH("update_mixed_long", stream, (update_mixed_long_kernel<T, VEC, OPT, WEIGHTED, 4, 1>), grid_long,
             dim3(kBlockThreads), go, w, st, psw, gpsw, a.table_offsets, a.table_dim_offsets, a.dim_offsets, a.T,
             a.total_D, i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),
             i32(l.num_unique), 2, long_rows, a.lr, a.eps, a.sr);
  const int64_t want_huge = a.n / (kChunkLen + 1) + 1;
  const dim3 grid_huge(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_huge, 256 * 2))));
  TBE_LAUNCH("update_mixed_huge", stream, (update_mixed_long_kernel<T, VEC, OPT, WEIGHTED, 4, kHugeWaves>),
             grid_huge, dim3(kHugeWaves * kWave), go, w, st, psw, gpsw, a.table_offsets, a.table_dim_offsets,
             a.dim_offsets, a.T, a.total_D, i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows),
             i32(l.segment_starts), i32(l.num_unique), 1, huge_rows, a.lr, a.eps, a.sr);
}

template <typename T, int VEC>
void launch_update_mixed_variant(const MixedArgs &a, const tbe_workspace_layout_t &l, char *ws,
                                 hipStream_t stream) {
  const bool weighted = a.psw != nullptr;
  if (a.optimizer == kOptSgd) {
    if (weighted) launch_update_mixed<T, VEC, kOptSgd, true>(a, l, ws, stream);
    else launch_update_mixed<T, VEC, kOptSgd, false>(a, l, ws, stream);
  } else {
    if (weighted) launch_update_mixed<T, VEC, kOptAdagrad, true>(a, l, ws, stream);
    else launch_update_mixed<T, VEC, kOptAdagrad, false>(a, l, ws, stream);
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
  TBE_REQUIRE(optimizer == TBE_OPT_SGD || optimizer == TBE_OPT_ROWWISE_ADAGRAD, "%s: bad optimizer %d", name,
              optimizer);
  a.optimizer = optimizer == TBE_OPT_SGD ? kOptSgd : kOptAdagrad;
  if (int rc = validate_mixed(name, a)) return rc;
  TBE_REQUIRE(grad_output && table_dim_offsets, "%s: null pointer argument", name);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(a.optimizer == kOptSgd || optimizer_state, "%s: optimizer_state is null", name);
  TBE_REQUIRE((per_sample_weights == nullptr) == (grad_per_sample_weights == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, 4, dtype, T, &l);  // no partial rows are used: size them for D = 4
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  char *ws = static_cast<char *>(workspace);
  auto i32 = [&](uint64_t off) { return reinterpret_cast<int32_t *>(ws + off); };
  const int64_t num_bags = static_cast<int64_t>(T) * B;
  TBE_LAUNCH("linearize_mixed", s, linearize_mixed_kernel,
             dim3(static_cast<unsigned>(ceil_div(num_bags * 16, kBlockThreads))), dim3(kBlockThreads),
             table_dim_offsets, indices, offsets, B, T, static_cast<int>(num_bags), nullptr, i32(l.grad_rows));
  // every table's indices are sorted on their own; the last pass adds the table's first row id
  const int64_t largest = (max_table_rows > 0 && max_table_rows < total_rows) ? max_table_rows : total_rows;
  const SortTables tables{offsets, B, T, table_dim_offsets};
  int rc = sort_pairs(indices, nullptr, i32(l.keys_sorted), i32(l.positions_sorted), num_indices,
                      key_bits_for(largest), ws + l.sort_scratch, s, &tables);
  if (rc) return rc;
  rc = find_segments(i32(l.keys_sorted), num_indices, i32(l.segment_starts), i32(l.num_unique), nullptr,
                     ws + l.segment_scratch, s, /*clear_queue_counters=*/true);
  if (rc) return rc;
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
