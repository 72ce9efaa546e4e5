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

#include <algorithm>

#include "tbe_stages.h"

namespace tbe {
namespace {

template <typename A> __device__ __forceinline__ A approx_multiplier(A state_new, A psw, bool weighted, float lr, float eps);
// (element_weight *) learning_rate * (1.0 / (sqrt(s) + eps)) with the reference's types: float
// sqrt and sum, double reciprocal and product, rounded to float (tbe.cu:453-454, 515-518).
template <> __device__ __forceinline__ float approx_multiplier<float>(float s, float pw, bool weighted, float lr, float eps) {
  const double inv = 1.0 / static_cast<double>(sqrtf(s) + eps);
  return weighted ? static_cast<float>(static_cast<double>(pw * lr) * inv)
                  : static_cast<float>(static_cast<double>(lr) * inv);
}
template <> __device__ __forceinline__ double approx_multiplier<double>(double s, double pw, bool weighted, float lr, float eps) {
  const double inv = 1.0 / (sqrt(s) + static_cast<double>(eps));
  return weighted ? pw * static_cast<double>(lr) * inv : static_cast<double>(lr) * inv;
}

// Sum over the `group` lanes (a power of two) around the caller; every lane gets the result.
template <typename A> __device__ __forceinline__ A group_sum_pow2(A v, int group) {
  for (int m = group >> 1; m > 0; m >>= 1) v += shfl_x(v, m);
  return v;
}

// The value a row element has after it was stored in the weights' type and read again.
template <typename T, int VEC>
__device__ __forceinline__ void round_trip(RowVec<T, VEC> &w, const StochasticRounding &sr, int64_t element) {
  if constexpr (sizeof(T) == 2) w.unpack(pack_rounded<T, VEC>(w, sr, element));
}

struct MixedTables {
  const int64_t *table_offsets;      // [T+1] first element of each table
  const int32_t *table_dim_offsets;  // [T+1] first row id of each table
  const int32_t *dim_offsets;        // [T+1] first output column of each table
  int32_t total_D;
  int32_t T;
};

constexpr int kBatch = 8;  // occurrences whose gradient rows are requested together

template <typename T, int VEC, bool WEIGHTED, bool MIXED>
__global__ __launch_bounds__(kBlockThreads) void approx_adagrad_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw, T *__restrict__ grad_psw,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, int D, int group, float lr, float eps, MixedTables mt,
    StochasticRounding sr) {
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

  // every lane of the wavefront runs the same trip counts (the shuffles need all of them)
  for (int64_t u0 = wave_id * groups; u0 < U; u0 += wave_stride * groups) {
    const int64_t u = u0 + r;
    const bool valid = u < U;
    int seg_begin = 0, seg_end = 0;
    int64_t key = 0;
    if (valid) {
      seg_begin = segment_starts[u];
      seg_end = segment_starts[u + 1];
      key = keys_sorted[seg_begin];
    }
    // where the row and its gradient rows live
    int row_D = D;
    int64_t row_element = key * D;   // first element of the row inside `weights`
    int64_t grad_stride = D;         // elements between consecutive gradient rows ...
    int grad_column = 0;             // ... and the first column of this table inside one
    int table = 0;
    if constexpr (MIXED) {
      if (valid) {
        const int first_pos = positions_sorted[seg_begin];
        table = grad_rows[first_pos] % mt.T;
        const int column0 = mt.dim_offsets[table];
        row_D = mt.dim_offsets[table + 1] - column0;
        row_element = mt.table_offsets[table] + (key - mt.table_dim_offsets[table]) * row_D;
        grad_column = column0;
      } else {
        row_D = 0;
      }
      grad_stride = mt.total_D;
    }
    const int row_chunks = valid ? row_D / VEC : 0;
    const bool in_registers = row_chunks <= group;   // one vector per lane holds the row
    const bool mine = c < row_chunks;                // this lane owns a vector of a register-held row
    T *wrow = weights + row_element;
    A s = A(0);
    if (valid) s = state[key];
    V w;
    w.zero();
    if (in_registers && mine) w.load(wrow + static_cast<int64_t>(c) * VEC);

    for (int k0 = seg_begin; __any(k0 < seg_end); k0 += batch) {
      // bookkeeping of up to `batch` occurrences, one per lane of the group
      int my_pos = 0, my_grow = 0;
      A my_pw = A(1);
      if (c < batch && k0 + c < seg_end) {
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
        StochasticRounding sr_k = sr;
        sr_k.seed ^= static_cast<uint64_t>(k0 + j - seg_begin) * 0x9E3779B97F4A7C15ull;

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
    if (valid && c == 0) state[key] = s;
    // (fp16: the last update already rounded the row to the stored type, this conversion is exact)
    if (in_registers && mine) w.store(wrow + static_cast<int64_t>(c) * VEC);
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
#define TBE_APPROX(WEIGHTED, MIXED)                                                                  \
  TBE_LAUNCH("update_approx", stream, (approx_adagrad_kernel<T, VEC, WEIGHTED, MIXED>), grid, block, \
             static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights),                     \
             static_cast<A *>(a.state), static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw), \
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),   \
             i32(l.num_unique), a.D, group, a.lr, a.eps, a.mt, a.sr)
  if (mixed) {
    if (a.psw) TBE_APPROX(true, true);
    else TBE_APPROX(false, true);
  } else {
    if (a.psw) TBE_APPROX(true, false);
    else TBE_APPROX(false, false);
  }
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
