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

// keys[p] = table_dim_offsets[t] + indices[p]; grad_rows[p] = b * T + t.
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
  const int32_t row0 = table_dim_offsets[t];
  const int32_t grow = b * num_tables + t;
  const int end = offsets[bag + 1];
  for (int p = offsets[bag] + static_cast<int>(gid % kLanes); p < end; p += kLanes) {
    keys[p] = row0 + indices[p];
    grad_rows[p] = grow;
  }
}

// One wavefront per unique row; passes as in the reference's exact kernel (sum of squares
// first, then the update), plus the per-occurrence dot products when weighted.
template <typename T, int VEC, int OPT, bool WEIGHTED>
__global__ __launch_bounds__(kBlockThreads) void update_mixed_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int64_t *__restrict__ table_offsets,
    const int32_t *__restrict__ table_dim_offsets, const int32_t *__restrict__ dim_offsets,
    int num_tables, int total_D, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ counters, float lr,
    float eps, StochasticRounding sr) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;

  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;

  for (int64_t u = wave_id; u < U; u += stride) {
    const int seg_begin = segment_starts[u];
    const int seg_end = segment_starts[u + 1];
    const int32_t key = keys_sorted[seg_begin];
    // table of the row: the last t with table_dim_offsets[t] <= key
    int lo = 0, hi = num_tables;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (table_dim_offsets[mid] <= key) lo = mid;
      else hi = mid;
    }
    const int t = lo;
    const int dim_start = dim_offsets[t];
    const int D = dim_offsets[t + 1] - dim_start;
    const int chunks = D / VEC;
    const int64_t row_element = table_offsets[t] + static_cast<int64_t>(key - table_dim_offsets[t]) * D;
    T *wrow = weights + row_element;
    const T *gcol = grad_output + dim_start;

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
      const A s_new = state[key] + gss;
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
  const int64_t want = ceil_div(a.n, kWavesPerBlock);
  const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 32))));
  TBE_LAUNCH("update_mixed", stream, (update_mixed_kernel<T, VEC, OPT, WEIGHTED>), grid, dim3(kBlockThreads),
             static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights), static_cast<A *>(a.state),
             static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw), a.table_offsets, a.table_dim_offsets,
             a.dim_offsets, a.T, a.total_D, i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows),
             i32(l.segment_starts), i32(l.num_unique), a.lr, a.eps, a.sr);
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
                                  const int64_t *table_offsets, const int32_t *table_dim_offsets,
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
             table_dim_offsets, indices, offsets, B, T, static_cast<int>(num_bags), i32(l.keys), i32(l.grad_rows));
  int rc = sort_pairs(i32(l.keys), nullptr, i32(l.keys_sorted), i32(l.positions_sorted), num_indices,
                      key_bits_for(total_rows), ws + l.sort_scratch, s, nullptr);
  if (rc) return rc;
  rc = find_segments(i32(l.keys_sorted), num_indices, i32(l.segment_starts), i32(l.num_unique), nullptr,
                     ws + l.segment_scratch, s);
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
