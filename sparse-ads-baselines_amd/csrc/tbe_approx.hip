// Approximate row-wise Adagrad for gfx950: the reference's per-lookup update
// (batched_embedding_backward_adagrad_approx_kernel_1, table_batched_embeddings_cuda.cu:648-704,
// with AdaGradFunctor / WeightedAdaGradFunctor, :437-471, :483-553; mixed-D twin :1006-1074),
// made deterministic.
//
// The reference gives every bag a warp that, for each of the bag's lookups, adds the bag's
// ||grad||^2 to the row's state with a plain load and store, derives one multiplier per lookup
// from the state it found, and subtracts multiplier * grad from the row.  Bags run concurrently,
// so a row that occurs in two bags is raced for; the result is defined only when no row repeats.
// Here the same per-lookup arithmetic runs ONE LOOKUP AT A TIME per row, in position order:
// the batch is sorted by (table, row) as for the exact update, and the lane group that owns a
// row walks its occurrences in ascending position,
//     wss  = ||grad_output[b][t]||^2 (* psw[p]^2)
//     s   += wss;  mult = (psw[p] *) lr * (1.0 / (sqrt(s) + eps))
//     grad_psw[p] = <row, grad_output[b][t]>          (weighted; the row as it is at that moment)
//     row -= mult * grad_output[b][t]                 (rounded to the weights' type every time)
// Rows are independent, so this is the reference's kernel executed serially in position order:
// identical to it when no row repeats, and the serial outcome when rows do.  No atomics, fixed
// order, bit-identical reruns.
//
// Geometry: `group` lanes (a power of two, the row's vector count rounded up, at most 64) own
// one row; a wavefront holds 64 / group rows.  A row of at most `group` vectors stays in
// registers from its first to its last occurrence; wider rows (and the mixed-D tables, which use
// the whole wavefront per row) are read and written per occurrence in column blocks.  Gradient
// rows of up to 8 occurrences are requested together.
//
// A row with more than kApproxLong occurrences would keep one lane group busy for a long serial
// walk (three dependent loads per 8 occurrences, a double-precision division per occurrence).
// Such rows are queued and get a wavefront each (approx_adagrad_long_kernel), which takes 64
// occurrences at a time: bookkeeping one occurrence per lane, ||grad||^2 by all lane groups in
// parallel, the running state by a wavefront prefix sum and the 64 multipliers side by side;
// only `row -= mult * grad` (and its rounding) remains a serial chain, fed by prefetched rows.

#include <algorithm>

#include "tbe_rowwise.h"
#include "tbe_stages.h"

namespace tbe {
namespace {

// Value of `v` in lane `src`, for a lane number that is the same in every lane (a scalar read
// instead of a trip through LDS).
__device__ __forceinline__ int broadcast_lane(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ float broadcast_lane(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ __forceinline__ int64_t broadcast_lane(int64_t v, int src) {
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), src));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v >> 32), src));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}
__device__ __forceinline__ double broadcast_lane(double v, int src) {
  return __longlong_as_double(broadcast_lane(static_cast<int64_t>(__double_as_longlong(v)), src));
}

// Sum over the `group` lanes (a power of two) around the caller; every lane gets the result.
template <typename A> __device__ __forceinline__ A group_sum_pow2(A v, int group) {
  for (int m = group >> 1; m > 0; m >>= 1) v += shfl_x(v, m);
  return v;
}

struct MixedTables {
  const int64_t *table_offsets;      // [T+1] first element of each table
  const int32_t *table_dim_offsets;  // [T+1] first row id of each table
  const int32_t *dim_offsets;        // [T+1] first output column of each table
  int32_t total_D;
  int32_t T;
};

constexpr int kBatch = 8;  // occurrences whose gradient rows are requested together
constexpr int kApproxLong = 64;  // a register-held row with more occurrences gets a wavefront of its own

// Geometry of the row behind a unique key and of its gradient rows.
struct RowPlace {
  int row_D;            // elements in the row
  int64_t row_element;  // first element of the row inside `weights`
  int64_t grad_stride;  // elements between consecutive gradient rows ...
  int grad_column;      // ... and the first column of this table inside one
};

template <bool MIXED>
__device__ __forceinline__ RowPlace place_row(int64_t key, int first_grad_row, int D, const MixedTables &mt) {
  RowPlace p{D, key * D, D, 0};
  if constexpr (MIXED) {
    const int table = first_grad_row % mt.T;
    const int column0 = mt.dim_offsets[table];
    p.row_D = mt.dim_offsets[table + 1] - column0;
    p.row_element = mt.table_offsets[table] + (key - mt.table_dim_offsets[table]) * p.row_D;
    p.grad_column = column0;
    p.grad_stride = mt.total_D;
  }
  return p;
}

template <bool MIXED>
__device__ __forceinline__ int64_t grad_row_offset(int grad_row, const RowPlace &p, const MixedTables &mt) {
  if constexpr (MIXED) return static_cast<int64_t>(grad_row / mt.T) * p.grad_stride + p.grad_column;
  else return static_cast<int64_t>(grad_row) * p.grad_stride;
}

template <typename T, int VEC, bool WEIGHTED, bool MIXED>
__global__ __launch_bounds__(kBlockThreads) void approx_adagrad_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw, T *__restrict__ grad_psw,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ segment_starts,
    int32_t *__restrict__ counters, int32_t *__restrict__ long_queue, int D, int group, float lr,
    float eps, MixedTables mt, StochasticRounding sr) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int r = lane / group;
  const int c = lane - r * group;
  const int group_base = r * group;
  const int groups = kWave / group;
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t wave_stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  const int batch = group < kBatch ? group : kBatch;  // one lane of the group fetches one occurrence's bookkeeping

  // A wavefront takes strips of 64 unique rows.  First one row per LANE: segment bounds, key,
  // state, position / gradient row / weight of the first occurrence -- the dependent loads are
  // paid once per strip, 64 wide.  Then one row per lane GROUP, handed out by lane shuffles.
  // (Every lane of the wavefront runs the same trip counts: the shuffles need all of them.)
  for (int64_t strip = wave_id * kWave; strip < U; strip += wave_stride * kWave) {
    const int rows_here = static_cast<int>(min(static_cast<int64_t>(kWave), U - strip));
    int lane_begin = 0, lane_end = 0, lane_key = 0, lane_pos0 = 0, lane_grow0 = 0;
    A lane_state = A(0), lane_pw0 = A(1);
    if (lane < rows_here) {
      lane_begin = segment_starts[strip + lane];
      lane_end = segment_starts[strip + lane + 1];
      lane_key = keys_sorted[lane_begin];
      lane_pos0 = positions_sorted[lane_begin];
      lane_state = state[lane_key];
      lane_grow0 = grad_rows[lane_pos0];
      if constexpr (WEIGHTED) lane_pw0 = to_acc(psw[lane_pos0]);
    }
  for (int i0 = 0; i0 < rows_here; i0 += groups) {
    const bool valid = i0 + r < rows_here;
    const int src = valid ? i0 + r : 0;
    const int64_t u = strip + src;
    const int seg_begin = shfl_idx(lane_begin, src);
    int seg_end = shfl_idx(lane_end, src);
    if (!valid) seg_end = seg_begin;
    const int64_t key = shfl_idx(lane_key, src);
    const int first_pos = shfl_idx(lane_pos0, src);
    const int first_grow = shfl_idx(lane_grow0, src);
    const A first_pw = shfl_idx(lane_pw0, src);
    const A state_in = shfl_idx(lane_state, src);
    // where the row and its gradient rows live
    const RowPlace place = place_row<MIXED>(key, first_grow, D, mt);
    const int row_D = valid ? place.row_D : 0;
    const int64_t row_element = place.row_element;
    const int64_t grad_stride = place.grad_stride;
    const int grad_column = place.grad_column;
    const int row_chunks = valid ? row_D / VEC : 0;
    const bool in_registers = row_chunks <= group;   // one vector per lane holds the row
    const bool mine = c < row_chunks;                // this lane owns a vector of a register-held row
    if (valid && in_registers && seg_end - seg_begin > kApproxLong) {
      // a long walk: the row gets a wavefront of its own in approx_adagrad_long_kernel
      if (c == 0) long_queue[atomicAdd(&counters[1], 1)] = static_cast<int32_t>(u);
      seg_end = seg_begin;  // nothing to do here
    }
    const bool handled_here = seg_end > seg_begin;
    T *wrow = weights + row_element;
    A s = state_in;
    V w;
    w.zero();
    if (handled_here && in_registers && mine) w.load(wrow + static_cast<int64_t>(c) * VEC);

    for (int k0 = seg_begin; __any(k0 < seg_end); k0 += batch) {
      // bookkeeping of up to `batch` occurrences, one per lane of the group
      int my_pos = first_pos, my_grow = first_grow;  // the segment's first occurrence is known already
      A my_pw = first_pw;
      if (c < batch && k0 + c < seg_end && k0 + c > seg_begin) {
        my_pos = positions_sorted[k0 + c];
        my_grow = grad_rows[my_pos];
        if constexpr (WEIGHTED) my_pw = to_acc(psw[my_pos]);
      }
      // the gradient vectors of a register-held row, requested together
      R raw[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int src = group_base + (j < batch ? j : 0);
        const int grow = shfl_idx(my_grow, src);
        const int64_t gbase = MIXED ? static_cast<int64_t>(grow / mt.T) * grad_stride + grad_column
                                    : static_cast<int64_t>(grow) * grad_stride;
        if (in_registers && mine && j < batch && k0 + j < seg_end)
          raw[j] = V::load_raw(grad_output + gbase + static_cast<int64_t>(c) * VEC);
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        if (j >= batch) break;
        if (!__any(k0 + j < seg_end)) break;
        const bool live = k0 + j < seg_end;
        const int src = group_base + j;
        const int pos = shfl_idx(my_pos, src);
        const int grow = shfl_idx(my_grow, src);
        const A pw = shfl_idx(my_pw, src);
        const int64_t gbase = MIXED ? static_cast<int64_t>(grow / mt.T) * grad_stride + grad_column
                                    : static_cast<int64_t>(grow) * grad_stride;
        const T *grow_ptr = grad_output + gbase;
        // the k-th update of a row in this call rounds with its own random words
        const StochasticRounding sr_k = rounding_of_update(sr, k0 + j - seg_begin);

        // ||grad||^2 of the bag (the reference computes it once per bag, tbe.cu:668-675)
        A local = A(0);
        V g;
        g.zero();
        if (in_registers) {
          if (live && mine) g.unpack(raw[j]);
#pragma unroll
          for (int i = 0; i < VEC; ++i) local += g.v[i] * g.v[i];
        } else if (live) {
          for (int cb = c; cb < row_chunks; cb += group) {
            V x;
            x.load(grow_ptr + static_cast<int64_t>(cb) * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) local += x.v[i] * x.v[i];
          }
        }
        const A gss = group_sum_pow2<A>(local, group);
        A mult = A(0);
        if (live) {
          const A wss = WEIGHTED ? gss * pw * pw : gss;
          s = s + wss;
          mult = approx_multiplier<A>(s, pw, WEIGHTED, lr, eps);
        }
        A dot = A(0);
        if (in_registers) {
          if (live && mine) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WEIGHTED) dot += w.v[i] * g.v[i];
              w.v[i] = w.v[i] - g.v[i] * mult;
            }
            round_trip<T, VEC>(w, sr_k, row_element + static_cast<int64_t>(c) * VEC);
          }
        } else if (live) {
          for (int cb = c; cb < row_chunks; cb += group) {
            V x, y;
            x.load(grow_ptr + static_cast<int64_t>(cb) * VEC);
            y.load(wrow + static_cast<int64_t>(cb) * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WEIGHTED) dot += y.v[i] * x.v[i];
              y.v[i] = y.v[i] - x.v[i] * mult;
            }
            store_row<T, VEC, false>(wrow + static_cast<int64_t>(cb) * VEC, y, sr_k,
                                     row_element + static_cast<int64_t>(cb) * VEC);
          }
        }
        if constexpr (WEIGHTED) {
          dot = group_sum_pow2<A>(dot, group);
          if (live && c == 0) grad_psw[pos] = from_acc<T, A>(dot);
        }
      }
    }
    if (handled_here && c == 0) state[key] = s;
    // (fp16: the last update already rounded the row to the stored type, this conversion is exact)
    if (handled_here && in_registers && mine) w.store(wrow + static_cast<int64_t>(c) * VEC);
  }
  }
}

// One wavefront per queued row.  Same arithmetic as approx_adagrad_kernel, except that the
// running state of the 64 occurrences of a batch comes from a wavefront prefix sum instead of
// dependent additions.  Per batch: bookkeeping one occurrence per lane, requested a batch ahead;
// ||grad||^2 of the 64 gradient rows by all lane groups side by side; the 64 multipliers side by
// side; then the serial `row -= mult * grad` walk by lane group 0, which requests the rows
// (cache-resident by then) eight at a time.
template <typename T, int VEC, bool WEIGHTED, bool MIXED>
__global__ __launch_bounds__(kBlockThreads) void approx_adagrad_long_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw, T *__restrict__ grad_psw,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ long_queue, int D, int group,
    float lr, float eps, MixedTables mt, StochasticRounding sr) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;
  constexpr int kRows = 8;  // gradient rows a lane group has in flight while the norms are formed
  constexpr int batch_rows = kWave;
  __shared__ A s_gss_all[kWavesPerBlock][kWave];

  const int lane = threadIdx.x & (kWave - 1);
  A *s_gss = s_gss_all[threadIdx.x >> 6];
  const int r = lane / group;
  const int c = lane - r * group;
  const int groups = kWave / group;
  const int num_long = counters[1];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t wave_stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;

  for (int64_t q = wave_id; q < num_long; q += wave_stride) {
    const int u = long_queue[q];
    const int seg_begin = segment_starts[u];
    const int seg_end = segment_starts[u + 1];
    const int64_t key = keys_sorted[seg_begin];
    const RowPlace place = place_row<MIXED>(key, grad_rows[positions_sorted[seg_begin]], D, mt);
    const int row_chunks = place.row_D / VEC;
    const bool mine = c < row_chunks;
    const bool owner = r == 0 && mine;  // lane group 0 holds the row
    T *wrow = weights + place.row_element;
    const int64_t col = static_cast<int64_t>(c) * VEC;
    V w;
    w.zero();
    if (owner) w.load(wrow + col);
    A s = state[key];

    // bookkeeping of the first batch: one occurrence per lane
    int cur_pos = positions_sorted[min(seg_begin + lane, seg_end - 1)];
    int64_t cur_goff = grad_row_offset<MIXED>(grad_rows[cur_pos], place, mt);
    A cur_pw = A(1);
    if constexpr (WEIGHTED) cur_pw = to_acc(psw[cur_pos]);

    for (int k0 = seg_begin; k0 < seg_end; k0 += batch_rows) {
      const int nb = min(batch_rows, seg_end - k0);
      // the next batch's bookkeeping is requested now and used one iteration later
      const int nxt_pos = positions_sorted[min(k0 + batch_rows + lane, seg_end - 1)];
      const int nxt_grow = grad_rows[nxt_pos];
      A nxt_pw = A(1);
      if constexpr (WEIGHTED) nxt_pw = to_acc(psw[nxt_pos]);

      // gradient rows -> LDS, and ||grad||^2 of every occurrence: lane group r takes occurrences
      // r, r + groups, ...
      for (int j0 = 0; j0 < nb; j0 += groups * kRows) {
        R raw[kRows];
#pragma unroll
        for (int x = 0; x < kRows; ++x) {
          const int j = min(j0 + x * groups + r, nb - 1);
          const int64_t goff = shfl_idx(cur_goff, j);
          if (mine) raw[x] = V::load_raw(grad_output + goff + col);
        }
#pragma unroll
        for (int x = 0; x < kRows; ++x) {
          const int j = j0 + x * groups + r;
          A local = A(0);
          if (mine) {
            V g;
            g.unpack(raw[x]);
#pragma unroll
            for (int i = 0; i < VEC; ++i) local += g.v[i] * g.v[i];
          }
          const A gss = group_sum_pow2<A>(local, group);
          if (c == 0 && j < nb) s_gss[j] = gss;
        }
      }
      __builtin_amdgcn_wave_barrier();
      // running state and multiplier of every occurrence, one per lane
      A wss = A(0);
      if (lane < nb) {
        const A gss = s_gss[lane];
        wss = WEIGHTED ? gss * cur_pw * cur_pw : gss;
      }
      A incl = wss;
#pragma unroll
      for (int d = 1; d < kWave; d <<= 1) {
        const A y = __shfl_up(incl, d, kWave);
        if (lane >= d) incl += y;
      }
      const A my_mult = lane < nb ? approx_multiplier<A>(s + incl, cur_pw, WEIGHTED, lr, eps) : A(0);
      s = s + broadcast_lane(incl, nb - 1);

      // the row itself: one update after the other
      for (int j0 = 0; j0 < nb; j0 += kBatch) {
        R raw[kBatch];
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          const int64_t goff = broadcast_lane(cur_goff, min(j0 + b, nb - 1));
          if (owner) raw[b] = V::load_raw(grad_output + goff + col);
        }
#pragma unroll
        for (int b = 0; b < kBatch; ++b) {
          const int j = j0 + b;
          if (j >= nb) break;
          const A mult = broadcast_lane(my_mult, j);
          A dot = A(0);
          if (owner) {
            V g;
            g.unpack(raw[b]);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WEIGHTED) dot += w.v[i] * g.v[i];
              w.v[i] = w.v[i] - g.v[i] * mult;
            }
            round_trip<T, VEC>(w, rounding_of_update(sr, k0 + j - seg_begin), place.row_element + col);
          }
          if constexpr (WEIGHTED) {
            dot = group_sum_pow2<A>(dot, group);
            const int pos = broadcast_lane(cur_pos, j);
            if (lane == 0) grad_psw[pos] = from_acc<T, A>(dot);
          }
        }
      }
      __builtin_amdgcn_wave_barrier();  // the next batch overwrites the norms in LDS
      cur_pos = nxt_pos;
      cur_goff = grad_row_offset<MIXED>(nxt_grow, place, mt);
      cur_pw = nxt_pw;
    }
    if (lane == 0) state[key] = s;
    if (owner) w.store(wrow + col);
  }
}

struct ApproxArgs {
  const void *grad_output;
  void *weights;
  void *state;
  const void *psw;
  void *grad_psw;
  int32_t dtype;
  int32_t vec;   // elements per vector (fp16: 8 or 4)
  int32_t D;     // uniform tables; 0 with mixed-D tables
  int64_t n;
  float lr, eps;
  MixedTables mt;
  StochasticRounding sr;
};

template <typename T, int VEC>
void launch_approx(const ApproxArgs &a, const tbe_workspace_layout_t &l, char *ws, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  auto i32 = [&](uint64_t off) { return reinterpret_cast<const int32_t *>(ws + off); };
  const bool mixed = a.D == 0;
  int group = kWave;
  if (!mixed) {
    const int chunks = a.D / VEC;
    group = 1;
    while (group < chunks && group < kWave) group <<= 1;
  }
  const int groups = kWave / group;
  const int64_t want = ceil_div(ceil_div(a.n, groups), kWavesPerBlock);
  const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 64))));
  const dim3 block(kBlockThreads);
  // the queue of long rows borrows the exact update's chunk-record region (at least n / 17 records
  // of 32 bytes, against at most n / 17 queued rows of 4 bytes); its counter is word 1 of the
  // counter block, which the segment stage left at zero
  int32_t *counters = reinterpret_cast<int32_t *>(ws + l.num_unique);
  int32_t *long_queue = reinterpret_cast<int32_t *>(ws + l.chunk_segments);
  const int64_t most_long = a.n / (kShortSegment + 1) + 1;  // (the short-row kernel queues rows of 17 and more)
  const dim3 grid_long(static_cast<unsigned>(
      std::max<int64_t>(1, std::min<int64_t>(ceil_div(most_long, kWavesPerBlock), 256 * 8))));
  const dim3 block_long(kBlockThreads);
#define TBE_APPROX(WEIGHTED, MIXED)                                                                    \
  TBE_LAUNCH("update_approx", stream, (approx_adagrad_kernel<T, VEC, WEIGHTED, MIXED>), grid, block,   \
             static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights),                       \
             static_cast<A *>(a.state), static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw),   \
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),     \
             counters, long_queue, a.D, group, a.lr, a.eps, a.mt, a.sr);                               \
  TBE_LAUNCH("update_approx_long", stream, (approx_adagrad_long_kernel<T, VEC, WEIGHTED, MIXED>),      \
             grid_long, block_long, static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights), \
             static_cast<A *>(a.state), static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw),   \
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),     \
             counters, long_queue, a.D, group, a.lr, a.eps, a.mt, a.sr)
#define TBE_APPROX_LONG(WEIGHTED)                                                                      \
  TBE_LAUNCH("update_approx_long", stream, (approx_adagrad_long_kernel<T, VEC, WEIGHTED, false>),      \
             grid_long, block_long, static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights), \
             static_cast<A *>(a.state), static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw),   \
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),     \
             counters, long_queue, a.D, group, a.lr, a.eps, a.mt, a.sr)
  if (mixed) {
    if (a.psw) { TBE_APPROX(true, true); }
    else { TBE_APPROX(false, true); }
  } else if (approx_short_serves(a.dtype, a.D)) {
    // uniform tables whose rows fit a wavefront: rows of up to kShortSegment occurrences go through
    // the exact update's position-balanced short-row kernel in its per-lookup form, the others
    // (queued by it) get a wavefront each
    UpdateArgs ua{};
    ua.grad_output = a.grad_output;
    ua.weights = a.weights;
    ua.optimizer_state = a.state;
    ua.per_sample_weights = a.psw;
    ua.grad_per_sample_weights = a.grad_psw;
    ua.keys_sorted = i32(l.keys_sorted);
    ua.positions_sorted = i32(l.positions_sorted);
    ua.grad_rows = i32(l.grad_rows);
    ua.segment_starts = i32(l.segment_starts);
    ua.counters = counters;
    ua.segment_ids = i32(l.segment_ids);
    ua.num_indices = a.n;
    ua.dtype = a.dtype;
    ua.D = a.D;
    ua.optimizer = kOptAdagrad;
    ua.learning_rate = a.lr;
    ua.eps = a.eps;
    ua.stochastic_rounding = a.sr;
    (void)segment_update_approx_short(ua, long_queue, stream);
    if (a.psw) { TBE_APPROX_LONG(true); }
    else { TBE_APPROX_LONG(false); }
  } else {
    if (a.psw) { TBE_APPROX(true, false); }
    else { TBE_APPROX(false, false); }
  }
#undef TBE_APPROX_LONG
#undef TBE_APPROX
}

}  // namespace

// Runs the approximate update on a workspace that already holds the batch's plan
// (gradient rows, sorted keys and positions, run boundaries).
int approx_update(const void *grad_output, void *weights, void *state, const void *psw, void *grad_psw,
                  int32_t dtype, int32_t fp16_vector_width, int32_t D, int64_t n, float lr, float eps,
                  const int64_t *mixed_table_offsets, const int32_t *table_dim_offsets,
                  const int32_t *dim_offsets, int32_t total_D, int32_t T, StochasticRounding sr,
                  const tbe_workspace_layout_t &l, void *workspace, hipStream_t stream) {
  ApproxArgs a{grad_output, weights, state, psw, grad_psw, dtype, fp16_vector_width, D, n, lr, eps,
               MixedTables{mixed_table_offsets, table_dim_offsets, dim_offsets, total_D, T}, sr};
  char *ws = static_cast<char *>(workspace);
  switch (dtype) {
    case TBE_DTYPE_F32: launch_approx<float, 4>(a, l, ws, stream); break;
    case TBE_DTYPE_F16:
      if (a.vec == 8) launch_approx<__half, 8>(a, l, ws, stream);
      else launch_approx<__half, 4>(a, l, ws, stream);
      break;
    default: launch_approx<double, 2>(a, l, ws, stream); break;
  }
  return check_launch("tbe approximate Adagrad update");
}

}  // namespace tbe

extern "C" int tbe_backward_approx_adagrad(const void *grad_output, void *weights, int32_t dtype,
                                           int64_t total_rows, int64_t max_table_rows, int32_t D,
                                           const int32_t *table_offsets, int32_t T,
                                           const int32_t *indices, int64_t num_indices,
                                           const int32_t *offsets, int32_t B,
                                           const void *per_sample_weights, void *optimizer_state,
                                           float learning_rate, float eps,
                                           void *grad_per_sample_weights,
                                           int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                           void *workspace, uint64_t workspace_bytes, void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_approx_adagrad";
  TBE_REQUIRE(T > 0, "%s: T must be positive (got %d)", name, T);
  TBE_REQUIRE(B > 0, "%s: B must be positive (got %d)", name, B);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(grad_output && weights && table_offsets && offsets && optimizer_state, "%s: null pointer argument", name);
  TBE_REQUIRE(indices || num_indices == 0, "%s: indices is null but num_indices > 0", name);
  TBE_REQUIRE((per_sample_weights == nullptr) == (grad_per_sample_weights == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, D, dtype, T, &l);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = build_plan(l, workspace, table_offsets, T, indices, num_indices, offsets, B, total_rows,
                          max_table_rows, s))
    return rc;
  const RowGeometry g = row_geometry(dtype, D);
  return approx_update(grad_output, weights, optimizer_state, per_sample_weights, grad_per_sample_weights,
                       dtype, g.vec, D, num_indices, learning_rate, eps, nullptr, nullptr, nullptr, 0, T,
                       StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0},
                       l, workspace, s);
}
