// Segment reduction of output gradients per unique row, fused with the exact
// SGD / row-wise Adagrad update, for gfx950.  No atomics touch weights or state
// and every sum has a fixed order, so two runs are bit-identical.
//
// Input: keys sorted ascending with their original positions, run boundaries
// (segment_starts, U) and grad_rows[p] = b*T + t.  For the u-th unique row:
//   G      = sum over occurrences i in [start_u, start_{u+1}) of (psw[p_i] *) grad_output[grad_rows[p_i]][:]
//   SGD    : w -= lr * G                                (SGDFunctor, tbe.cu:318-331, applied once per row)
//   Adagrad: s += sum_d G_d^2 ; w -= lr / (sqrt(s) + eps) * G   (AdaGradFunctor, tbe.cu:437-471)
//   weighted: grad_psw[p_i] = <w_before, grad_output[grad_rows[p_i]]>    (tbe.cu:529-553)
// (tbe.cu = table_batched_embeddings_cuda.cu.)  The reference gathers every
// gradient row twice (tbe.cu:1548-1585); here G stays in registers.
//
// Work decomposition.  `chunks` lanes (one 16-byte vector each) own a row, a
// wavefront holds 64/chunks such lane groups, each group takes one segment at a
// time (grid-stride).  A group first loads the bookkeeping of up to `chunks`
// occurrences with one coalesced load, then streams the gradient rows with
// several loads in flight.  Segments longer than kLongSegment are not reduced
// by one group: they are registered in a list, cut into chunks of kChunkLen
// occurrences, each chunk is reduced by a whole wavefront into an fp32 partial
// row, and a last kernel adds a segment's partials in chunk order and applies
// the update.  Rows wider than 64 vectors take a multi-pass wavefront-per-
// segment path.

#include <algorithm>

#include "tbe_stages.h"

namespace tbe {
namespace {

template <typename A> __device__ __forceinline__ A adagrad_multiplier(A state_new, float lr, float eps);
// lr * (1.0 / (sqrt(s) + eps)) with the reference's types: float sqrt and add,
// double reciprocal and product, rounded to float (tbe.cu:453-454).
template <> __device__ __forceinline__ float adagrad_multiplier<float>(float s, float lr, float eps) {
  return static_cast<float>(static_cast<double>(lr) * (1.0 / static_cast<double>(sqrtf(s) + eps)));
}
template <> __device__ __forceinline__ double adagrad_multiplier<double>(double s, float lr, float eps) {
  return static_cast<double>(lr) * (1.0 / (sqrt(s) + static_cast<double>(eps)));
}

// Address of the row behind the u-th unique key: its slot in the HBM row cache when the
// tables are cache-fronted and the row is resident, else its row in `weights`.
template <typename T>
__device__ __forceinline__ T *resolve_row(T *weights, T *cache_rows,
                                          const int32_t *__restrict__ unique_slots, int64_t u,
                                          int64_t row, int D) {
  if (unique_slots) {
    const int slot = unique_slots[u];
    if (slot >= 0) return cache_rows + static_cast<int64_t>(slot) * D;
  }
  return weights + row * D;
}

// Applies the optimizer to one row held by a lane group.  `w_old` and `G` are
// this lane's vector of the row.
template <typename T, int VEC, int CHUNKS, int OPT>
__device__ __forceinline__ void apply_update(T *wrow, const RowVec<T, VEC> &w_old,
                                             const RowVec<T, VEC> &G,
                                             typename AccOf<T>::type *state_row, float lr,
                                             float eps, int chunks, int group_base, int c) {
  using A = typename AccOf<T>::type;
  RowVec<T, VEC> w_new;
  if constexpr (OPT == kOptSgd) {
#pragma unroll
    for (int i = 0; i < VEC; ++i) w_new.v[i] = w_old.v[i] - G.v[i] * static_cast<A>(lr);
  } else {
    A local = A(0);
#pragma unroll
    for (int i = 0; i < VEC; ++i) local += G.v[i] * G.v[i];
    const A gss = group_sum<CHUNKS, A>(local, chunks, group_base);
    const A s_new = *state_row + gss;
    if (c == 0) *state_row = s_new;
    const A mult = adagrad_multiplier<A>(s_new, lr, eps);
#pragma unroll
    for (int i = 0; i < VEC; ++i) w_new.v[i] = w_old.v[i] - G.v[i] * mult;
  }
  w_new.store(wrow);
}

// ------------------------------------------------------------ short segments
template <typename T, int VEC, int CHUNKS, int OPT, bool WEIGHTED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void update_short_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, int32_t *__restrict__ counters,
    int32_t *__restrict__ long_segments, int32_t *__restrict__ chunk_segments, int64_t max_long,
    int D, int chunks_rt, float lr, float eps, const int32_t *__restrict__ unique_slots,
    T *__restrict__ cache_rows) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const int group_base = r * chunks;
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock * groups;
  const int64_t col = static_cast<int64_t>(c) * VEC;

  for (int64_t u = (r < groups) ? wave_id * groups + r : U; u < U; u += stride) {
    const int seg_begin = segment_starts[u];
    const int seg_end = segment_starts[u + 1];
    const int len = seg_end - seg_begin;
    if (len > kLongSegment) {
      // Register the segment for the chunked path.
      const int nch = (len + kChunkLen - 1) / kChunkLen;
      int slot = 0, first_chunk = 0;
      if (c == 0) {
        slot = atomicAdd(&counters[1], 1);
        first_chunk = atomicAdd(&counters[2], nch);
        long_segments[slot] = static_cast<int32_t>(u);
        long_segments[max_long + slot] = first_chunk;
      }
      slot = shfl_idx(slot, group_base);
      first_chunk = shfl_idx(first_chunk, group_base);
      for (int k = c; k < nch; k += chunks) chunk_segments[first_chunk + k] = slot;
      continue;
    }
    const int64_t row = keys_sorted[seg_begin];
    T *wrow = resolve_row(weights, cache_rows, unique_slots, u, row, D) + col;
    V w_old;
    w_old.load(wrow);
    V G;
    G.zero();
    for (int base = seg_begin; base < seg_end; base += chunks) {
      const int n = min(chunks, seg_end - base);
      int my_pos = 0, my_grow = 0;
      A my_w = A(0);
      if (c < n) {
        my_pos = positions_sorted[base + c];
        my_grow = grad_rows[my_pos];
        if constexpr (WEIGHTED) my_w = to_acc(psw[my_pos]);
      }
      for (int j0 = 0; j0 < n; j0 += UNROLL) {
        R raw[UNROLL];
#pragma unroll
        for (int q = 0; q < UNROLL; ++q) {
          const int j = j0 + q;
          const int src = group_base + (j < n ? j : 0);
          const int64_t grow = shfl_idx(my_grow, src);
          if (j < n) raw[q] = V::load_raw(grad_output + grow * D + col);
        }
#pragma unroll
        for (int q = 0; q < UNROLL; ++q) {
          const int j = j0 + q;
          if (j < n) {
            V x;
            x.unpack(raw[q]);
            if constexpr (WEIGHTED) {
              const int src = group_base + j;
              const A pw = shfl_idx(my_w, src);
              const int pos = shfl_idx(my_pos, src);
              A dot = A(0);
#pragma unroll
              for (int i = 0; i < VEC; ++i) dot += w_old.v[i] * x.v[i];
              dot = group_sum<CHUNKS, A>(dot, chunks, group_base);
              if (c == 0) grad_psw[pos] = from_acc<T, A>(dot);
#pragma unroll
              for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * pw;
            } else {
#pragma unroll
              for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i];
            }
          }
        }
      }
    }
    apply_update<T, VEC, CHUNKS, OPT>(wrow, w_old, G, state ? state + row : nullptr, lr, eps,
                                      chunks, group_base, c);
  }
}

// ------------------------------------------------- long segments: chunk sums
// One wavefront per chunk of at most kChunkLen occurrences.  Lane group r adds
// occurrences r, r+groups, ... of the chunk; the groups are then combined in a
// fixed tree and group 0 stores the partial row.
template <typename T, int VEC, int CHUNKS, bool WEIGHTED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void update_long_partial_kernel(
    const T *__restrict__ grad_output, const T *__restrict__ weights, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ counters,
    const int32_t *__restrict__ long_segments, const int32_t *__restrict__ chunk_segments,
    typename AccOf<T>::type *__restrict__ partial_sums, int64_t max_long, int D, int chunks_rt,
    const int32_t *__restrict__ unique_slots, const T *__restrict__ cache_rows) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const int group_base = r * chunks;
  const bool active = r < groups;
  const int num_chunks = counters[2];
  const int64_t col = static_cast<int64_t>(c) * VEC;
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;

  for (int64_t q = wave_id; q < num_chunks; q += stride) {
    const int slot = chunk_segments[q];
    const int u = long_segments[slot];
    const int first_chunk = long_segments[max_long + slot];
    const int seg_begin = segment_starts[u];
    const int seg_end = segment_starts[u + 1];
    const int begin = seg_begin + static_cast<int>(q - first_chunk) * kChunkLen;
    const int end = min(seg_end, begin + kChunkLen);
    V w_old;
    w_old.zero();
    if constexpr (WEIGHTED) {
      const int64_t row = keys_sorted[seg_begin];
      if (active)
        w_old.load(resolve_row<const T>(weights, cache_rows, unique_slots, u, row, D) + col);
    }
    V G;
    G.zero();
    for (int base = begin; base < end; base += kWave) {
      const int n = min(kWave, end - base);
      int my_pos = 0, my_grow = 0;
      A my_w = A(0);
      if (lane < n) {
        my_pos = positions_sorted[base + lane];
        my_grow = grad_rows[my_pos];
        if constexpr (WEIGHTED) my_w = to_acc(psw[my_pos]);
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
          const int64_t grow = shfl_idx(my_grow, src[k]);
          if (ok[k]) raw[k] = V::load_raw(grad_output + grow * D + col);
        }
#pragma unroll
        for (int k = 0; k < UNROLL; ++k) {
          A pw = A(0);
          int pos = 0;
          if constexpr (WEIGHTED) {
            pw = shfl_idx(my_w, src[k]);
            pos = shfl_idx(my_pos, src[k]);
          }
          if (ok[k]) {
            V x;
            x.unpack(raw[k]);
            if constexpr (WEIGHTED) {
              A dot = A(0);
#pragma unroll
              for (int i = 0; i < VEC; ++i) dot += w_old.v[i] * x.v[i];
              dot = group_sum<CHUNKS, A>(dot, chunks, group_base);
              if (c == 0) grad_psw[pos] = from_acc<T, A>(dot);
#pragma unroll
              for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * pw;
            } else {
#pragma unroll
              for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i];
            }
          }
        }
      }
    }
    if constexpr (CHUNKS > 0) {
#pragma unroll
      for (int m = kWave / 2; m >= CHUNKS; m >>= 1) {
#pragma unroll
        for (int i = 0; i < VEC; ++i) G.v[i] += shfl_x(G.v[i], m);
      }
    } else {
      int live = groups;
      while (live > 1) {
        const int s = (live + 1) / 2;
        const int from = min(lane + s * chunks, kWave - 1);
        const bool take = active && (r + s < live);
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
          const A o = shfl_idx(G.v[i], from);
          if (take) G.v[i] += o;
        }
        live = s;
      }
    }
    if (r == 0) {
      A *dst = partial_sums + q * D + col;
#pragma unroll
      for (int i = 0; i < VEC; ++i) dst[i] = G.v[i];
    }
  }
}

// --------------------------------------------- long segments: combine + update
template <typename T, int VEC, int CHUNKS, int OPT>
__global__ __launch_bounds__(kBlockThreads) void update_long_finish_kernel(
    T *__restrict__ weights, typename AccOf<T>::type *__restrict__ state,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ long_segments,
    const typename AccOf<T>::type *__restrict__ partial_sums, int64_t max_long, int D,
    int chunks_rt, float lr, float eps, const int32_t *__restrict__ unique_slots,
    T *__restrict__ cache_rows) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;

  const int lane = threadIdx.x & (kWave - 1);
  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const int group_base = r * chunks;
  const int num_long = counters[1];
  const int64_t col = static_cast<int64_t>(c) * VEC;
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock * groups;

  for (int64_t slot = (r < groups) ? wave_id * groups + r : num_long; slot < num_long;
       slot += stride) {
    const int u = long_segments[slot];
    const int first_chunk = long_segments[max_long + slot];
    const int seg_begin = segment_starts[u];
    const int len = segment_starts[u + 1] - seg_begin;
    const int nch = (len + kChunkLen - 1) / kChunkLen;
    const int64_t row = keys_sorted[seg_begin];
    T *wrow = resolve_row(weights, cache_rows, unique_slots, u, row, D) + col;
    V w_old;
    w_old.load(wrow);
    V G;
    G.zero();
    for (int k = 0; k < nch; ++k) {
      const A *src = partial_sums + static_cast<int64_t>(first_chunk + k) * D + col;
#pragma unroll
      for (int i = 0; i < VEC; ++i) G.v[i] += src[i];
    }
    apply_update<T, VEC, CHUNKS, OPT>(wrow, w_old, G, state ? state + row : nullptr, lr, eps,
                                      chunks, group_base, c);
  }
}

// ---------------------------------------------------- rows wider than a wavefront
// One wavefront per segment, any length, any D.  Passes over the segment:
//   (weighted) per occurrence, <w_before, g> over all column blocks -> grad_psw
//   (Adagrad)  per column block, G -> sum of squares
//   per column block, G again -> update            (the reference's two-pass scheme, tbe.cu:1548-1585)
template <typename T, int VEC, int OPT, bool WEIGHTED>
__global__ __launch_bounds__(kBlockThreads) void update_wide_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ counters, int D,
    int chunks, float lr, float eps, const int32_t *__restrict__ unique_slots,
    T *__restrict__ cache_rows) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;

  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;

  for (int64_t u = wave_id; u < U; u += stride) {
    const int seg_begin = segment_starts[u];
    const int seg_end = segment_starts[u + 1];
    const int64_t row = keys_sorted[seg_begin];
    T *wrow = resolve_row(weights, cache_rows, unique_slots, u, row, D);

    if constexpr (WEIGHTED) {
      for (int i = seg_begin; i < seg_end; ++i) {
        const int pos = positions_sorted[i];
        const T *grow = grad_output + static_cast<int64_t>(grad_rows[pos]) * D;
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
          g.load(grad_output + static_cast<int64_t>(grad_rows[pos]) * D + static_cast<int64_t>(cb) * VEC);
          A pw = A(1);
          if constexpr (WEIGHTED) pw = to_acc(psw[pos]);
#pragma unroll
          for (int k = 0; k < VEC; ++k) G.v[k] += WEIGHTED ? g.v[k] * pw : g.v[k];
        }
#pragma unroll
        for (int k = 0; k < VEC; ++k) local += G.v[k] * G.v[k];
      }
      const A gss = group_sum<kWave, A>(local, kWave, 0);
      const A s_new = state[row] + gss;
      if (lane == 0) state[row] = s_new;
      mult = adagrad_multiplier<A>(s_new, lr, eps);
    }

    for (int cb = lane; cb < chunks; cb += kWave) {
      V G;
      G.zero();
      for (int i = seg_begin; i < seg_end; ++i) {
        const int pos = positions_sorted[i];
        V g;
        g.load(grad_output + static_cast<int64_t>(grad_rows[pos]) * D + static_cast<int64_t>(cb) * VEC);
        A pw = A(1);
        if constexpr (WEIGHTED) pw = to_acc(psw[pos]);
#pragma unroll
        for (int k = 0; k < VEC; ++k) G.v[k] += WEIGHTED ? g.v[k] * pw : g.v[k];
      }
      V w;
      w.load(wrow + static_cast<int64_t>(cb) * VEC);
#pragma unroll
      for (int k = 0; k < VEC; ++k) w.v[k] = w.v[k] - G.v[k] * mult;
      w.store(wrow + static_cast<int64_t>(cb) * VEC);
    }
  }
}

__global__ void zero_counters_kernel(int32_t *counters) {
  if (threadIdx.x == 1 || threadIdx.x == 2) counters[threadIdx.x] = 0;
}

constexpr int kShortUnroll = 4;
constexpr int kLongUnroll = 4;

template <typename T, int VEC, int CHUNKS, int OPT, bool WEIGHTED>
void launch_narrow(const UpdateArgs &a, const RowGeometry &g, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  const T *go = static_cast<const T *>(a.grad_output);
  T *w = static_cast<T *>(a.weights);
  A *st = static_cast<A *>(a.optimizer_state);
  const T *psw = static_cast<const T *>(a.per_sample_weights);
  T *gpsw = static_cast<T *>(a.grad_per_sample_weights);
  A *partial = static_cast<A *>(a.partial_sums);
  T *cr = static_cast<T *>(a.cache_rows);
  const int groups = kWave / g.chunks;
  const dim3 block(kBlockThreads);

  // Enough wavefronts to cover the worst case U == N once, capped so that the
  // grid-stride loop amortises launch cost on large inputs.
  const int64_t want = ceil_div(ceil_div(a.num_indices, groups), kWavesPerBlock);
  const dim3 grid_short(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 32))));
  TBE_LAUNCH("update_short", stream,
             (update_short_kernel<T, VEC, CHUNKS, OPT, WEIGHTED, kShortUnroll>), grid_short, block,
             go, w, st, psw, gpsw, a.keys_sorted, a.positions_sorted, a.grad_rows,
             a.segment_starts, a.counters, a.long_segments, a.chunk_segments, a.max_long, a.D,
             g.chunks, a.learning_rate, a.eps, a.unique_slots, cr);

  const int64_t want_chunks = ceil_div(a.max_chunks, kWavesPerBlock);
  const dim3 grid_partial(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_chunks, 256 * 8))));
  TBE_LAUNCH("update_long_partial", stream,
             (update_long_partial_kernel<T, VEC, CHUNKS, WEIGHTED, kLongUnroll>), grid_partial,
             block, go, w, psw, gpsw, a.keys_sorted, a.positions_sorted, a.grad_rows,
             a.segment_starts, a.counters, a.long_segments, a.chunk_segments, partial, a.max_long,
             a.D, g.chunks, a.unique_slots, cr);

  const int64_t want_long = ceil_div(ceil_div(a.max_long, groups), kWavesPerBlock);
  const dim3 grid_finish(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_long, 256 * 4))));
  TBE_LAUNCH("update_long_finish", stream, (update_long_finish_kernel<T, VEC, CHUNKS, OPT>),
             grid_finish, block, w, st, a.keys_sorted, a.segment_starts, a.counters,
             a.long_segments, partial, a.max_long, a.D, g.chunks, a.learning_rate, a.eps,
             a.unique_slots, cr);
}

template <typename T, int VEC, int OPT, bool WEIGHTED>
void launch_geometry(const UpdateArgs &a, const RowGeometry &g, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  if (g.wide) {
    const int64_t want = ceil_div(a.num_indices, kWavesPerBlock);
    const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 32))));
    TBE_LAUNCH("update_wide", stream, (update_wide_kernel<T, VEC, OPT, WEIGHTED>), grid,
               dim3(kBlockThreads), static_cast<const T *>(a.grad_output),
               static_cast<T *>(a.weights), static_cast<A *>(a.optimizer_state),
               static_cast<const T *>(a.per_sample_weights),
               static_cast<T *>(a.grad_per_sample_weights), a.keys_sorted, a.positions_sorted,
               a.grad_rows, a.segment_starts, a.counters, a.D, g.chunks, a.learning_rate, a.eps,
               a.unique_slots, static_cast<T *>(a.cache_rows));
    return;
  }
  switch (g.tmpl) {
    case 64: launch_narrow<T, VEC, 64, OPT, WEIGHTED>(a, g, stream); break;
    case 32: launch_narrow<T, VEC, 32, OPT, WEIGHTED>(a, g, stream); break;
    case 16: launch_narrow<T, VEC, 16, OPT, WEIGHTED>(a, g, stream); break;
    case 8: launch_narrow<T, VEC, 8, OPT, WEIGHTED>(a, g, stream); break;
    case 4: launch_narrow<T, VEC, 4, OPT, WEIGHTED>(a, g, stream); break;
    default: launch_narrow<T, VEC, 0, OPT, WEIGHTED>(a, g, stream); break;
  }
}

template <typename T, int VEC>
void launch_variant(const UpdateArgs &a, const RowGeometry &g, hipStream_t stream) {
  const bool weighted = a.per_sample_weights != nullptr;
  if (a.optimizer == kOptSgd) {
    if (weighted) launch_geometry<T, VEC, kOptSgd, true>(a, g, stream);
    else launch_geometry<T, VEC, kOptSgd, false>(a, g, stream);
  } else {
    if (weighted) launch_geometry<T, VEC, kOptAdagrad, true>(a, g, stream);
    else launch_geometry<T, VEC, kOptAdagrad, false>(a, g, stream);
  }
}

}  // namespace

int segment_update(const UpdateArgs &a, hipStream_t stream) {
  if (a.num_indices == 0) return TBE_OK;
  const RowGeometry g = row_geometry(a.dtype, a.D);
  TBE_LAUNCH("zero_counters", stream, zero_counters_kernel, dim3(1), dim3(kWave), a.counters);
  switch (a.dtype) {
    case TBE_DTYPE_F32: launch_variant<float, 4>(a, g, stream); break;
    case TBE_DTYPE_F16:
      if (g.vec == 8) launch_variant<__half, 8>(a, g, stream);
      else launch_variant<__half, 4>(a, g, stream);
      break;
    default: launch_variant<double, 2>(a, g, stream); break;
  }
  return check_launch("tbe segment update");
}

}  // namespace tbe
