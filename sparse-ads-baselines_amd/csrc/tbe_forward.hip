// Pooled forward gather-sum for gfx950: one 64-lane wavefront per bag.
//
// A row of D elements is `chunks` 16-byte vectors.  `chunks` consecutive lanes
// own one row at a time, so one wavefront-wide load instruction fetches
// floor(64 / chunks) different rows (2 for D=128 fp32, 8 for D=64 fp16), and the
// loop is unrolled so every lane keeps several independent 16-byte loads in
// flight.  The 64 indices (and per-sample weights) of a bag slice are fetched
// with one coalesced load and handed to the owning lane group by a lane shuffle.
// Accumulation is fp32 (fp64 for double); the row groups are combined with a
// shuffle tree and lane group 0 writes the D outputs once.
//
// Semantics follow batched_embedding_forward_kernel_1
// (table_batched_embeddings_cuda.cu:193-251): bag index b_t = t*B + b,
// output[b][t][:], empty bag -> zeros, weighted variant multiplies each row by
// indice_weights[position] (WeightedForward, :176-191).

#include "tbe_common.h"

namespace tbe {
namespace {

template <typename T, int VEC, int CHUNKS, bool WEIGHTED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void forward_kernel(
    const T *__restrict__ weights, const int32_t *__restrict__ table_offsets,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets,
    const T *__restrict__ psw, T *__restrict__ output, int B, int num_tables, int D,
    int chunks_rt, int num_bags, int64_t blocks_per_xcd) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t logical = xcd_contiguous(blockIdx.x, blocks_per_xcd);
  const int64_t bag64 = logical * kWavesPerBlock + (threadIdx.x >> 6);
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const int t = bag / B;
  const int b = bag - t * B;

  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;  // rows fetched per wavefront-wide load
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const bool active = r < groups;

  const int start = offsets[bag];
  const int end = offsets[bag + 1];
  const int64_t table_row0 = table_offsets[t];
  const T *col = weights + static_cast<int64_t>(c) * VEC;

  V acc;
  acc.zero();

  for (int base = start; base < end; base += kWave) {
    const int n = min(kWave, end - base);
    int my_idx = 0;
    A my_w = A(0);
    if (lane < n) {
      my_idx = __builtin_nontemporal_load(indices + base + lane);
      if constexpr (WEIGHTED) my_w = to_acc(psw[base + lane]);
    }
    for (int j0 = 0; j0 < n; j0 += groups * UNROLL) {
      R raw[UNROLL];
      A w[UNROLL];
      bool ok[UNROLL];
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int j = j0 + u * groups + r;
        ok[u] = active && j < n;
        const int src = ok[u] ? j : 0;
        const int idx = shfl_idx(my_idx, src);
        if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, src);
        if (ok[u]) raw[u] = V::load_raw(col + (table_row0 + idx) * D);
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        if (ok[u]) {
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

  // Combine the row groups into group 0.
  if constexpr (CHUNKS > 0) {
#pragma unroll
    for (int m = kWave / 2; m >= CHUNKS; m >>= 1) {
#pragma unroll
      for (int i = 0; i < VEC; ++i) acc.v[i] += shfl_x(acc.v[i], m);
    }
  } else {
    int live = groups;
    while (live > 1) {
      const int s = (live + 1) / 2;
      const int src = min(lane + s * chunks, kWave - 1);
      const bool take = active && (r + s < live);
#pragma unroll
      for (int i = 0; i < VEC; ++i) {
        const A o = shfl_idx(acc.v[i], src);
        if (take) acc.v[i] += o;
      }
      live = s;
    }
  }

  if (r == 0) {
    acc.store(output + (static_cast<int64_t>(b) * num_tables + t) * D + static_cast<int64_t>(c) * VEC);
  }
}

// Rows wider than 64 vectors: the wavefront walks the row in blocks of 64
// vectors and sums the bag serially per block.
template <typename T, int VEC, bool WEIGHTED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void forward_wide_kernel(
    const T *__restrict__ weights, const int32_t *__restrict__ table_offsets,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets,
    const T *__restrict__ psw, T *__restrict__ output, int B, int num_tables, int D,
    int chunks, int num_bags, int64_t blocks_per_xcd) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t logical = xcd_contiguous(blockIdx.x, blocks_per_xcd);
  const int64_t bag64 = logical * kWavesPerBlock + (threadIdx.x >> 6);
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const int t = bag / B;
  const int b = bag - t * B;
  const int start = offsets[bag];
  const int end = offsets[bag + 1];
  const int64_t table_row0 = table_offsets[t];
  T *out_row = output + (static_cast<int64_t>(b) * num_tables + t) * D;

  for (int cb = 0; cb < chunks; cb += kWave) {
    const int c = cb + lane;
    const bool ok_c = c < chunks;
    const T *col = weights + static_cast<int64_t>(c) * VEC;
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
          const int idx = shfl_idx(my_idx, j);
          if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, j);
          if (ok_c && j0 + u < n) raw[u] = V::load_raw(col + (table_row0 + idx) * D);
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

template <typename T, int VEC, bool WEIGHTED>
int launch_forward(const RowGeometry &g, const void *weights, int32_t D,
                   const int32_t *table_offsets, int32_t T_, const int32_t *indices,
                   const int32_t *offsets, int32_t B, const void *psw, void *output,
                   hipStream_t stream) {
  const int num_bags = T_ * B;
  const int64_t nblocks = ceil_div(num_bags, kWavesPerBlock);
  const int64_t per_xcd = ceil_div(nblocks, kNumXcd);
  const dim3 grid(static_cast<unsigned>(per_xcd * kNumXcd));
  const dim3 block(kBlockThreads);
  const T *w = static_cast<const T *>(weights);
  const T *p = static_cast<const T *>(psw);
  T *o = static_cast<T *>(output);
  constexpr int kUnroll = 8;
#define TBE_FWD(CH)                                                                        \
  TBE_LAUNCH("forward", stream, (forward_kernel<T, VEC, CH, WEIGHTED, kUnroll>), grid,   \
             block, w, table_offsets, indices, offsets, p, o, B, T_, D, g.chunks, num_bags, \
             per_xcd)
  if (g.wide) {
    TBE_LAUNCH("forward_wide", stream, (forward_wide_kernel<T, VEC, WEIGHTED, 4>), grid, block,
               w, table_offsets, indices, offsets, p, o, B, T_, D, g.chunks, num_bags, per_xcd);
  } else {
    switch (g.tmpl) {
      case 64: TBE_FWD(64); break;
      case 32: TBE_FWD(32); break;
      case 16: TBE_FWD(16); break;
      case 8: TBE_FWD(8); break;
      case 4: TBE_FWD(4); break;
      default: TBE_FWD(0); break;
    }
  }
#undef TBE_FWD
  return check_launch("tbe_forward");
}

template <typename T, int VEC>
int launch_forward_w(bool weighted, const RowGeometry &g, const void *weights, int32_t D,
                     const int32_t *table_offsets, int32_t T_, const int32_t *indices,
                     const int32_t *offsets, int32_t B, const void *psw, void *output,
                     hipStream_t stream) {
  return weighted ? launch_forward<T, VEC, true>(g, weights, D, table_offsets, T_, indices,
                                                 offsets, B, psw, output, stream)
                  : launch_forward<T, VEC, false>(g, weights, D, table_offsets, T_, indices,
                                                  offsets, B, psw, output, stream);
}

}  // namespace
}  // namespace tbe

extern "C" int tbe_forward(const void *weights, int32_t dtype, int32_t D,
                           const int32_t *table_offsets, int32_t T, const int32_t *indices,
                           int64_t num_indices, const int32_t *offsets, int32_t B,
                           const void *per_sample_weights, void *output, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(T > 0, "tbe_forward: T must be positive (got %d)", T);
  TBE_REQUIRE(D > 0, "tbe_forward: D must be positive (got %d)", D);
  TBE_REQUIRE(B > 0, "tbe_forward: B must be positive (got %d)", B);
  TBE_REQUIRE(D % 4 == 0, "tbe_forward: D must be a multiple of 4 (got %d)", D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "tbe_forward: bad dtype %d", dtype);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "tbe_forward: num_indices out of range");
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "tbe_forward: T*B out of range");
  TBE_REQUIRE(weights && table_offsets && offsets && output, "tbe_forward: null pointer argument");
  TBE_REQUIRE(indices || num_indices == 0, "tbe_forward: indices is null but num_indices > 0");
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RowGeometry g = row_geometry(dtype, D);
  const bool weighted = per_sample_weights != nullptr;
  switch (dtype) {
    case TBE_DTYPE_F32:
      return launch_forward_w<float, 4>(weighted, g, weights, D, table_offsets, T, indices,
                                        offsets, B, per_sample_weights, output, s);
    case TBE_DTYPE_F16:
      if (g.vec == 8)
        return launch_forward_w<__half, 8>(weighted, g, weights, D, table_offsets, T, indices,
                                           offsets, B, per_sample_weights, output, s);
      return launch_forward_w<__half, 4>(weighted, g, weights, D, table_offsets, T, indices,
                                         offsets, B, per_sample_weights, output, s);
    default:
      return launch_forward_w<double, 2>(weighted, g, weights, D, table_offsets, T, indices,
                                         offsets, B, per_sample_weights, output, s);
  }
}
