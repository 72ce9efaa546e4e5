// Pooled forward gather-sum for gfx950: one 64-lane wavefront per bag (forward_kernel), or one
// lane group per bag for short bags of narrow rows (forward_grouped_kernel).
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
//
// Interleaved tables (the older sparse_embedding_cuda layout, sparse_embedding_cuda_kernel.cu:221-284,
// 349-379): weights [E][T][D], bags numbered b*T + t, bag (b, t) bounded by offsets[b * stride + t]
// and the entry after it (stride = T for one flat array, T + 1 for the [B][T+1] form).  The same
// kernels serve it -- `table_offsets` is null then, the row of a lookup is idx * T + t and the
// bag's output row is the bag's number -- so no index array is rewritten.

#include "tbe_common.h"

namespace tbe {
namespace {

// Where a bag lives.  Table-major (table_offsets given): bag = t*B + b, rows table_offsets[t] + idx.
// Interleaved (table_offsets null): bag = b*T + t, rows idx*T + t, offsets with a row stride.
struct BagPlace {
  int start, end;          // the bag's lookups
  int64_t row0;            // row of a lookup = row0 + idx * row_mul
  int row_mul;             // (1, or T for interleaved tables, where idx * T < 2^31)
  int64_t out_row;         // b*T + t
};
__device__ __forceinline__ BagPlace place_bag(int bag, bool has_end, int B, int num_tables,
                                              const int32_t *__restrict__ table_offsets,
                                              const int32_t *__restrict__ offsets, int offsets_stride) {
  BagPlace p;
  if (table_offsets) {
    const int t = bag / B;
    const int b = bag - t * B;
    p.start = offsets[bag];
    p.end = has_end ? offsets[bag + 1] : p.start;
    p.row0 = table_offsets[t];
    p.row_mul = 1;
    p.out_row = static_cast<int64_t>(b) * num_tables + t;
  } else {
    // The wavefronts still walk the bags table by table (bag = t*B + b names the bag b*T + t), so that
    // an XCD, which takes an eighth of the bags, works on an eighth of the tables and finds their hot
    // rows in its own L2, as with table-major tables.  (Walking them in their own order, every XCD
    // touches every table: 380 instead of 317 us for 64 tables of 100 k rows of 128, Zipf 1.05.)
    const int t = bag / B;
    const int b = bag - t * B;
    const int64_t at = static_cast<int64_t>(b) * offsets_stride + t;
    p.start = offsets[at];
    p.end = has_end ? offsets[at + 1] : p.start;
    p.row0 = t;
    p.row_mul = num_tables;
    p.out_row = static_cast<int64_t>(b) * num_tables + t;
  }
  return p;
}

// Row r of a table of rows of CHUNKS 16-byte vectors (r < 2^31).  With CHUNKS known at compile time the row's
// offset is a shift of the 32-bit row number; otherwise one 32 x 32 -> 64-bit multiply with D.  (A 64-bit row
// number times D costs three quarter-rate 32-bit multiplies per row: the vector ALU was busy with those for a
// fifth of the forward of 512-byte rows.)
template <typename T, int VEC, int CHUNKS>
__device__ __forceinline__ const T *narrow_row(const T *base, uint32_t row, int D = 0) {
  if constexpr (CHUNKS > 0) return base + (static_cast<uint64_t>(row) * static_cast<uint64_t>(CHUNKS * VEC));
  else return base + static_cast<uint64_t>(row) * static_cast<uint32_t>(D);
}

// CACHED: every lookup carries a location (lookup_slots[p]); a non-negative value is a slot of
// the HBM row cache (row at cache_rows + slot * D), a negative one means the row is read from
// `weights` (the host-resident backing table) directly.
template <typename T, int VEC, int CHUNKS, bool WEIGHTED, bool CACHED, int UNROLL, bool INTERLEAVED>
__global__ __launch_bounds__(kBlockThreads) void forward_kernel(
    const T *__restrict__ weights, const int32_t *__restrict__ table_offsets,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets,
    const T *__restrict__ psw, T *__restrict__ output, int B, int num_tables, int D_rt,
    int chunks_rt, int num_bags, int64_t blocks_per_xcd,
    const int32_t *__restrict__ lookup_slots, const T *__restrict__ cache_rows, int offsets_stride) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t logical = xcd_contiguous(blockIdx.x, blocks_per_xcd);
  const int64_t bag64 = logical * kWavesPerBlock + (threadIdx.x >> 6);
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);

  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int D = CHUNKS > 0 ? CHUNKS * VEC : D_rt;
  const int groups = kWave / chunks;  // rows fetched per wavefront-wide load
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const bool active = r < groups;

  const BagPlace place = place_bag(bag, true, B, num_tables, table_offsets, offsets, offsets_stride);
  const int start = place.start;
  const int end = place.end;
  const uint32_t row0_32 = static_cast<uint32_t>(place.row0);  // rows are numbered below 2^31
  const uint32_t row_mul = static_cast<uint32_t>(place.row_mul);
  const T *col = weights + static_cast<int64_t>(c) * VEC;
  const T *cache_col = cache_rows + static_cast<int64_t>(c) * VEC;

  V acc;
  acc.zero();

  for (int base = start; base < end; base += kWave) {
    const int n = min(kWave, end - base);
    int my_idx = 0;
    int my_slot = -1;
    A my_w = A(0);
    if (lane < n) {
      my_idx = __builtin_nontemporal_load(indices + base + lane);
      if constexpr (WEIGHTED) my_w = to_acc(psw[base + lane]);
      if constexpr (CACHED) my_slot = __builtin_nontemporal_load(lookup_slots + base + lane);
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
        const uint32_t idx = static_cast<uint32_t>(shfl_idx(my_idx, src));
        if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, src);
        const T *row = narrow_row<T, VEC, CHUNKS>(col, row0_32 + (INTERLEAVED ? idx * row_mul : idx), D);
        if constexpr (CACHED) {
          const int slot = shfl_idx(my_slot, src);
          if (slot >= 0) row = narrow_row<T, VEC, CHUNKS>(cache_col, static_cast<uint32_t>(slot), D);
        }
        if (ok[u]) raw[u] = V::load_raw(row);
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
    acc.store(output + place.out_row * D + static_cast<int64_t>(c) * VEC);
  }
}

// Narrow rows (4, 8 or 16 vectors) and short bags: one lane *group* per bag, 64 / CHUNKS bags
// per wavefront.  A bag of 20 rows keeps a wavefront-per-bag kernel busy for one partly filled
// batch and pays a cross-group reduction; here every group walks its own bag (32 indices fetched
// per step, up to 8 independent row loads in flight per lane), nothing is reduced across lanes
// and the instruction stream is shared by all the wavefront's bags.  Same sums as
// forward_kernel in a different order (each lane adds its bag's rows in bag order).
constexpr int kGroupedWaves = 4;  // wavefronts of a workgroup of forward_grouped_kernel (8: 81 instead of 70 us for 32 tables of fp16 rows of 64, bags of 0..40)
template <typename T, int VEC, int CHUNKS, bool WEIGHTED, bool CACHED, bool INTERLEAVED>
__global__ __launch_bounds__(kGroupedWaves * kWave) void forward_grouped_kernel(
    const T *__restrict__ weights, const int32_t *__restrict__ table_offsets,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets,
    const T *__restrict__ psw, T *__restrict__ output, int B, int num_tables, int /*D*/, int num_bags,
    int64_t blocks_per_xcd, const int32_t *__restrict__ lookup_slots,
    const T *__restrict__ cache_rows, int offsets_stride) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;
  constexpr int D = CHUNKS * VEC;
  constexpr int kGroups = kWave / CHUNKS;
  constexpr int kPerLane = 32 / CHUNKS;        // indices held per lane: a step covers 32 lookups of every bag
  constexpr int kStep = kPerLane * CHUNKS;
  constexpr int kUnroll = CHUNKS < 8 ? CHUNKS : 8;
  static_assert(CHUNKS == 4 || CHUNKS == 8 || CHUNKS == 16, "lane groups of 4, 8 or 16 vectors");

  const int lane = threadIdx.x & (kWave - 1);
  const int r = lane / CHUNKS;
  const int c = lane - r * CHUNKS;
  const int group_base = r * CHUNKS;
  // A wavefront is busy for the longest of its bags, so the workgroup's bags are dealt to its
  // wavefronts by length: the first wavefront takes the kGroups longest, the last the shortest (with
  // lengths spread evenly over 0..40, 3.5 instead of 4.6 steps of eight lookups per wavefront on
  // average).  Which lane group adds a bag up does not change its sum.
  constexpr int kBlockBags = kGroupedWaves * kGroups;
  __shared__ int s_len[kBlockBags];
  __shared__ int s_order[kBlockBags];
  const int64_t block_first = xcd_contiguous(blockIdx.x, blocks_per_xcd) * kBlockBags;
  const int tid = static_cast<int>(threadIdx.x);
  int my_len = -1;
  if (tid < kBlockBags) {
    if (block_first + tid < num_bags) {
      const BagPlace q = place_bag(static_cast<int>(block_first) + tid, true, B, num_tables, table_offsets, offsets,
                                   offsets_stride);
      my_len = q.end - q.start;
    }
    s_len[tid] = my_len;
  }
  __syncthreads();
  if (tid < kBlockBags) {
    int rank = 0;
#pragma unroll 8
    for (int j = 0; j < kBlockBags; ++j) {
      const int other = s_len[j];
      rank += (other > my_len || (other == my_len && j < tid)) ? 1 : 0;
    }
    s_order[rank] = tid;
  }
  __syncthreads();
  const int64_t bag64 = block_first + s_order[(tid >> 6) * kGroups + r];
  const bool valid = bag64 < num_bags;
  const int bag = static_cast<int>(valid ? bag64 : num_bags - 1);
  const BagPlace place = place_bag(bag, valid, B, num_tables, table_offsets, offsets, offsets_stride);
  const int start = place.start;
  const int end = place.end;
  const int64_t table_row0 = place.row0;
  const int row_mul = place.row_mul;
  const T *col = weights + static_cast<int64_t>(c) * VEC;
  const T *cache_col = cache_rows + static_cast<int64_t>(c) * VEC;
  const uint32_t row0_32 = static_cast<uint32_t>(table_row0);  // rows are numbered below 2^31
  // (interleaved tables: index 0 of the bag's own table, which exists)
  const int idle_idx = INTERLEAVED ? 0 : -static_cast<int>(table_row0);

  V acc;
  acc.zero();
  for (int base = start; __ballot(base < end) != 0ull; base += kStep) {
    int idx[kPerLane], slot[kPerLane];
    T w_raw[kPerLane];
    A w[kPerLane];
#pragma unroll
    for (int q = 0; q < kPerLane; ++q) {
      const int p = base + q * CHUNKS + c;
      // A lane without a lookup still loads (never adds) a row: row 0 of `weights` -- the index
      // cancels the table's first row, so the address exists even for a table without rows -- or,
      // behind the row cache, slot 0, so that idle lanes never reach over the host link.
      idx[q] = idle_idx;
      slot[q] = CACHED ? 0 : -1;
      w_raw[q] = T(0);
      if (p < end) {
        idx[q] = __builtin_nontemporal_load(indices + p);
        if constexpr (WEIGHTED) w_raw[q] = psw[p];  // converted once all of the step's loads are issued
        if constexpr (CACHED) slot[q] = __builtin_nontemporal_load(lookup_slots + p);
      }
    }
#pragma unroll
    for (int q = 0; q < kPerLane; ++q) w[q] = WEIGHTED ? to_acc(w_raw[q]) : A(0);
#pragma unroll
    for (int q = 0; q < kPerLane; ++q) {
      const int left = end - (base + q * CHUNKS);  // rows of this group's bag in this slice
      if (__ballot(left > 0) == 0ull) break;
#pragma unroll
      for (int j0 = 0; j0 < CHUNKS; j0 += kUnroll) {
        if (__ballot(j0 < left) == 0ull) break;
        R raw[kUnroll];
        A ww[kUnroll];
        bool ok[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          const int j = j0 + u;
          ok[u] = j < left;
          const int src = group_base + j;
          const uint32_t i = static_cast<uint32_t>(shfl_idx(idx[q], src));
          if constexpr (WEIGHTED) ww[u] = shfl_idx(w[q], src);
          const uint32_t row32 = row0_32 + (INTERLEAVED ? i * static_cast<uint32_t>(row_mul) : i);
          const T *row = narrow_row<T, VEC, CHUNKS>(col, row32);
          if constexpr (CACHED) {
            const int s = shfl_idx(slot[q], src);
            if (s >= 0) row = narrow_row<T, VEC, CHUNKS>(cache_col, static_cast<uint32_t>(s));
          }
          raw[u] = V::load_raw(row);  // every lane loads (straight-line code keeps the loads back to back)
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
          keep_if(raw[u], ok[u]);
          V x;
          x.unpack(raw[u]);
#pragma unroll
          for (int k = 0; k < VEC; ++k) {
            if constexpr (WEIGHTED) acc.v[k] += x.v[k] * ww[u];
            else acc.v[k] += x.v[k];
          }
        }
      }
    }
  }
  if (valid) acc.store(output + place.out_row * D + static_cast<int64_t>(c) * VEC);
}

// Rows wider than 64 vectors: the wavefront walks the row in blocks of 64
// vectors and sums the bag serially per block.
template <typename T, int VEC, bool WEIGHTED, bool CACHED, int UNROLL>
__global__ __launch_bounds__(kBlockThreads) void forward_wide_kernel(
    const T *__restrict__ weights, const int32_t *__restrict__ table_offsets,
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets,
    const T *__restrict__ psw, T *__restrict__ output, int B, int num_tables, int D,
    int chunks, int num_bags, int64_t blocks_per_xcd,
    const int32_t *__restrict__ lookup_slots, const T *__restrict__ cache_rows, int offsets_stride) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int64_t logical = xcd_contiguous(blockIdx.x, blocks_per_xcd);
  const int64_t bag64 = logical * kWavesPerBlock + (threadIdx.x >> 6);
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const BagPlace place = place_bag(bag, true, B, num_tables, table_offsets, offsets, offsets_stride);
  const int start = place.start;
  const int end = place.end;
  const int64_t table_row0 = place.row0;
  const int row_mul = place.row_mul;
  T *out_row = output + place.out_row * D;

  for (int cb = 0; cb < chunks; cb += kWave) {
    const int c = cb + lane;
    const bool ok_c = c < chunks;
    const T *col = weights + static_cast<int64_t>(c) * VEC;
    V acc;
    acc.zero();
    for (int base = start; base < end; base += kWave) {
      const int n = min(kWave, end - base);
      int my_idx = 0;
      int my_slot = -1;
      A my_w = A(0);
      if (lane < n) {
        my_idx = indices[base + lane];
        if constexpr (WEIGHTED) my_w = to_acc(psw[base + lane]);
        if constexpr (CACHED) my_slot = lookup_slots[base + lane];
      }
      for (int j0 = 0; j0 < n; j0 += UNROLL) {
        R raw[UNROLL];
        A w[UNROLL];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int j = min(j0 + u, n - 1);
          const int idx = shfl_idx(my_idx, j);
          if constexpr (WEIGHTED) w[u] = shfl_idx(my_w, j);
          const T *row = col + (table_row0 + idx * row_mul) * D;
          if constexpr (CACHED) {
            const int slot = shfl_idx(my_slot, j);
            if (slot >= 0) row = cache_rows + static_cast<int64_t>(slot) * D + static_cast<int64_t>(c) * VEC;
          }
          if (ok_c && j0 + u < n) raw[u] = V::load_raw(row);
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

struct ForwardArgs {
  const void *weights;
  int32_t dtype;
  int32_t D;
  const int32_t *table_offsets;
  int32_t T;
  const int32_t *indices;
  const int32_t *offsets;
  int32_t B;
  const void *psw;
  void *output;
  const int32_t *lookup_slots;  // null unless the rows are fronted by the HBM row cache
  const void *cache_rows;
  int64_t num_indices;
  int32_t offsets_stride = 0;   // interleaved tables (table_offsets null): entries of `offsets` per b
};

template <typename T, int VEC, bool WEIGHTED, bool CACHED>
void launch_forward(const ForwardArgs &a, const RowGeometry &g, hipStream_t stream) {
  const int num_bags = a.T * a.B;
  const int64_t nblocks = ceil_div(num_bags, kWavesPerBlock);
  const int64_t per_xcd = ceil_div(nblocks, kNumXcd);
  const dim3 grid(static_cast<unsigned>(per_xcd * kNumXcd));
  const dim3 block(kBlockThreads);
  const T *w = static_cast<const T *>(a.weights);
  const T *p = static_cast<const T *>(a.psw);
  const T *cr = static_cast<const T *>(a.cache_rows);
  T *o = static_cast<T *>(a.output);
  constexpr int kUnroll = 8;
#define TBE_FWD_L(CH, IL)                                                                          \
  TBE_LAUNCH("forward", stream, (forward_kernel<T, VEC, CH, WEIGHTED, CACHED, kUnroll, IL>), grid, \
             block, w, a.table_offsets, a.indices, a.offsets, p, o, a.B, a.T, a.D, g.chunks,       \
             num_bags, per_xcd, a.lookup_slots, cr, a.offsets_stride)
  // (the row cache fronts table-major tables only)
#define TBE_FWD(CH)                                                             \
  do {                                                                          \
    if constexpr (!CACHED) {                                                    \
      if (!a.table_offsets) { TBE_FWD_L(CH, true); break; }                     \
    }                                                                           \
    TBE_FWD_L(CH, false);                                                       \
  } while (0)
  // short bags of narrow rows: a lane group per bag instead of a wavefront per bag
  const bool grouped = !g.wide && (g.tmpl == 4 || g.tmpl == 8 || g.tmpl == 16) &&
                       a.num_indices <= static_cast<int64_t>(num_bags) * 48;
  if (grouped) {
    const int groups = kWave / g.tmpl;
    const int64_t gblocks = ceil_div(ceil_div(num_bags, groups), kGroupedWaves);
    const int64_t gper_xcd = ceil_div(gblocks, kNumXcd);
    const dim3 ggrid(static_cast<unsigned>(gper_xcd * kNumXcd));
#define TBE_FWD_GROUPED_L(CH, IL)                                                                   \
  TBE_LAUNCH("forward", stream, (forward_grouped_kernel<T, VEC, CH, WEIGHTED, CACHED, IL>), ggrid,  \
             dim3(kGroupedWaves * kWave), w, a.table_offsets, a.indices, a.offsets, p, o, a.B, a.T, a.D, num_bags,        \
             gper_xcd, a.lookup_slots, cr, a.offsets_stride)
    // (the row cache fronts table-major tables only)
#define TBE_FWD_GROUPED(CH)                                                     \
  do {                                                                          \
    if constexpr (!CACHED) {                                                    \
      if (!a.table_offsets) { TBE_FWD_GROUPED_L(CH, true); break; }             \
    }                                                                           \
    TBE_FWD_GROUPED_L(CH, false);                                               \
  } while (0)
    if (g.tmpl == 4) TBE_FWD_GROUPED(4);
    else if (g.tmpl == 8) TBE_FWD_GROUPED(8);
    else TBE_FWD_GROUPED(16);
#undef TBE_FWD_GROUPED_L
#undef TBE_FWD_GROUPED
  } else if (g.wide) {
    TBE_LAUNCH("forward_wide", stream, (forward_wide_kernel<T, VEC, WEIGHTED, CACHED, 4>), grid,
               block, w, a.table_offsets, a.indices, a.offsets, p, o, a.B, a.T, a.D, g.chunks,
               num_bags, per_xcd, a.lookup_slots, cr, a.offsets_stride);
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
#undef TBE_FWD_L
}

template <typename T, int VEC>
void launch_forward_variant(const ForwardArgs &a, const RowGeometry &g, hipStream_t stream) {
  const bool weighted = a.psw != nullptr;
  const bool cached = a.lookup_slots != nullptr;
  if (cached) {
    if (weighted) launch_forward<T, VEC, true, true>(a, g, stream);
    else launch_forward<T, VEC, false, true>(a, g, stream);
  } else {
    if (weighted) launch_forward<T, VEC, true, false>(a, g, stream);
    else launch_forward<T, VEC, false, false>(a, g, stream);
  }
}

int validate_forward(const char *name, const ForwardArgs &a, int64_t num_indices) {
  TBE_REQUIRE(a.T > 0, "%s: T must be positive (got %d)", name, a.T);
  TBE_REQUIRE(a.D > 0, "%s: D must be positive (got %d)", name, a.D);
  TBE_REQUIRE(a.B > 0, "%s: B must be positive (got %d)", name, a.B);
  TBE_REQUIRE(a.D % 4 == 0, "%s: D must be a multiple of 4 (got %d)", name, a.D);
  TBE_REQUIRE(a.dtype >= TBE_DTYPE_F32 && a.dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, a.dtype);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(a.T) * a.B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(a.weights && (a.table_offsets || a.offsets_stride >= a.T) && a.offsets && a.output,
              "%s: null pointer argument", name);
  TBE_REQUIRE(a.indices || num_indices == 0, "%s: indices is null but num_indices > 0", name);
  return TBE_OK;
}

}  // namespace

int run_forward(const ForwardArgs &a, hipStream_t stream) {
  const RowGeometry g = row_geometry(a.dtype, a.D);
  switch (a.dtype) {
    case TBE_DTYPE_F32: launch_forward_variant<float, 4>(a, g, stream); break;
    case TBE_DTYPE_F16:
      if (g.vec == 8) launch_forward_variant<__half, 8>(a, g, stream);
      else launch_forward_variant<__half, 4>(a, g, stream);
      break;
    default: launch_forward_variant<double, 2>(a, g, stream); break;
  }
  return check_launch("tbe_forward");
}

}  // namespace tbe

extern "C" int tbe_forward(const void *weights, int32_t dtype, int32_t D,
                           const int32_t *table_offsets, int32_t T, const int32_t *indices,
                           int64_t num_indices, const int32_t *offsets, int32_t B,
                           const void *per_sample_weights, void *output, void *stream) {
  using namespace tbe;
  const ForwardArgs a{weights, dtype, D, table_offsets, T, indices, offsets, B,
                      per_sample_weights, output, nullptr, nullptr, num_indices};
  if (int rc = validate_forward("tbe_forward", a, num_indices)) return rc;
  return run_forward(a, static_cast<hipStream_t>(stream));
}

extern "C" int tbe_forward_cached(const tbe_cache_t *cache, int32_t dtype, int32_t D,
                                  const int32_t *table_offsets, int32_t T,
                                  const int32_t *indices, int64_t num_indices,
                                  const int32_t *offsets, int32_t B,
                                  const void *per_sample_weights, const int32_t *lookup_slots,
                                  void *output, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(cache && cache->rows && cache->backing_rows, "tbe_forward_cached: null cache");
  TBE_REQUIRE(lookup_slots || num_indices == 0, "tbe_forward_cached: null lookup_slots");
  const ForwardArgs a{cache->backing_rows, dtype, D, table_offsets, T, indices, offsets, B,
                      per_sample_weights, output, lookup_slots, cache->rows, num_indices};
  if (int rc = validate_forward("tbe_forward_cached", a, num_indices)) return rc;
  if (num_indices == 0) {
    const ForwardArgs plain{cache->backing_rows, dtype, D, table_offsets, T, indices, offsets, B,
                            per_sample_weights, output, nullptr, nullptr, num_indices};
    return run_forward(plain, static_cast<hipStream_t>(stream));
  }
  return run_forward(a, static_cast<hipStream_t>(stream));
}

extern "C" int tbe_forward_interleaved(const void *weights, int32_t dtype, int64_t E, int32_t T, int32_t D,
                                       const int32_t *indices, int64_t num_indices, const int32_t *offsets,
                                       int32_t offsets_row_stride, int32_t B, void *output, void *stream) {
  using namespace tbe;
  const char *name = "tbe_forward_interleaved";
  TBE_REQUIRE(E > 0 && T > 0 && E * T < INT32_MAX, "%s: E * T must fit a 32-bit row number", name);
  TBE_REQUIRE(offsets_row_stride == T || offsets_row_stride == T + 1,
              "%s: offsets_row_stride must be T (flat offsets) or T + 1 ([B][T+1] offsets), got %d", name,
              offsets_row_stride);
  ForwardArgs a{weights, dtype, D, nullptr, T, indices, offsets, B, nullptr, output, nullptr, nullptr, num_indices};
  a.offsets_stride = offsets_row_stride;
  if (int rc = validate_forward(name, a, num_indices)) return rc;
  return run_forward(a, static_cast<hipStream_t>(stream));
}
