// Integer stages of the backward pass for gfx950:
//   linearize      (table,row) keys and the gradient row of every lookup
//   sort_pairs     stable LSD radix sort, 8-bit digits, LDS-staged scatter
//   find_segments  run boundaries of the sorted keys (one per unique row)
//
// The sort is the contract of cub::DeviceRadixSort::SortPairs as the reference
// calls it (table_batched_embeddings_cuda.cu:1639-1655): ascending, stable,
// key bits [0, end_bit).  A pass handles a digit of 8 to 10 bits (the fewest passes that cover
// end_bit).  Each pass is three kernels:
//   histogram  per-tile digit counts (LDS atomics) -> counts[digit][tile]
//   scan       one workgroup per digit: exclusive prefix over tiles, and the digit's total
//   scatter    ranks each key inside its tile with wavefront ballots (all lanes
//              holding the same digit are found with one ballot per digit bit; the lowest lane
//              reserves the run in a per-wavefront LDS counter), reorders the
//              tile in LDS so every digit's keys are contiguous, and writes
//              them out in runs.
// A tile is 4096 pairs; position order inside a tile is (wavefront, item, lane),
// which the ranking preserves, so the sort is stable.

#include "tbe_common.h"

namespace tbe {
namespace {

constexpr int kMaxRadixBits = 10;                 // widest digit of a pass
constexpr int kMaxBins = 1 << kMaxRadixBits;
constexpr int kItems = 16;                        // pairs per thread per tile
constexpr int kTile = kBlockThreads * kItems;     // 4096
constexpr int kWaveTile = kWave * kItems;         // 1024 pairs per wavefront

constexpr int kSegItems = 8;
constexpr int kSegTile = kBlockThreads * kSegItems;  // 2048

// Inclusive prefix sum over the 256 threads of a workgroup.  `total` receives the
// workgroup sum.  `s_wave` is 4 words of LDS.  Ends with a barrier-free state:
// callers that reuse `s_wave` must __syncthreads() first.
__device__ __forceinline__ uint32_t block_inclusive_scan(uint32_t x, uint32_t *s_wave,
                                                         uint32_t &total) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const uint32_t y = __shfl_up(x, d, kWave);
    if (lane >= d) x += y;
  }
  if (lane == kWave - 1) s_wave[wave] = x;
  __syncthreads();
  uint32_t base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    const uint32_t v = s_wave[w];
    if (w < wave) base += v;
    sum += v;
  }
  total = sum;
  return x + base;
}

// ------------------------------------------------------------------ linearize
// 16 lanes per bag.  Mirrors linear_index_weight_offsets_kernel
// (table_batched_embeddings_cuda.cu:1471-1497); instead of the 8-byte
// IndexInfo{b_t, indices_idx} payload it records the gradient row b*T + t of
// each position, and the sort carries the position itself.
constexpr int kLinLanes = 16;
__global__ __launch_bounds__(kBlockThreads) void linearize_kernel(
    const int32_t *__restrict__ table_offsets, const int32_t *__restrict__ indices,
    const int32_t *__restrict__ offsets, int B, int num_tables, int num_bags,
    int32_t *__restrict__ keys, int32_t *__restrict__ grad_rows) {
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t bag64 = gid / kLinLanes;
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const int sub = static_cast<int>(gid % kLinLanes);
  const int t = bag / B;
  const int b = bag - t * B;
  const int32_t row0 = table_offsets[t];
  const int32_t grow = b * num_tables + t;
  const int start = offsets[bag];
  const int end = offsets[bag + 1];
  for (int p = start + sub; p < end; p += kLinLanes) {
    keys[p] = row0 + indices[p];
    grad_rows[p] = grow;
  }
}

// Row numbers for tables stored interleaved, weights[row][table][D] (the layout of the older
// sparse_embedding_cuda kernels, sparse_embedding_cuda_kernel.cu:349-379: weights[ind][t][d]).
// Viewed as a [E*T][D] matrix, row `ind` of table t is matrix row ind*T + t; bags are numbered
// bag-major (b*T + t), so the table of a bag is bag % T.
__global__ __launch_bounds__(kBlockThreads) void interleaved_rows_kernel(
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets, int num_tables,
    int num_bags, int32_t *__restrict__ rows) {
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t bag = gid / kLinLanes;
  if (bag >= num_bags) return;
  const int t = static_cast<int>(bag % num_tables);
  const int end = offsets[bag + 1];
  for (int p = offsets[bag] + static_cast<int>(gid % kLinLanes); p < end; p += kLinLanes)
    rows[p] = indices[p] * num_tables + t;
}

// ------------------------------------------------------------------ radix sort
// BITS = digit width of the pass (8, 9 or 10): 2^BITS bins, each thread owns 2^BITS / 256
// consecutive digits in the per-digit steps.
template <int BITS>
__global__ __launch_bounds__(kBlockThreads) void radix_histogram_kernel(
    const uint32_t *__restrict__ keys, int64_t n, int shift, uint32_t mask, int num_tiles,
    uint32_t *__restrict__ counts) {
  constexpr int kBinsT = 1 << BITS;
  __shared__ uint32_t s_hist[kBinsT];
  const int tid = threadIdx.x;
#pragma unroll
  for (int d = tid; d < kBinsT; d += kBlockThreads) s_hist[d] = 0;
  __syncthreads();
  const int64_t base = static_cast<int64_t>(blockIdx.x) * kTile;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = base + k * kBlockThreads + tid;
    if (i < n) atomicAdd(&s_hist[(keys[i] >> shift) & mask], 1u);
  }
  __syncthreads();
#pragma unroll
  for (int d = tid; d < kBinsT; d += kBlockThreads)
    counts[static_cast<int64_t>(d) * num_tiles + blockIdx.x] = s_hist[d];
}

// Workgroup `d` turns counts[d][0..num_tiles) into an exclusive prefix over tiles (keys with
// digit d in earlier tiles) and publishes the row total; the scatter kernel adds the number
// of keys with a smaller digit, which it gets from a scan of the digit totals.
__global__ __launch_bounds__(kBlockThreads) void radix_scan_kernel(
    uint32_t *__restrict__ counts, uint32_t *__restrict__ totals, int num_tiles) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int tid = threadIdx.x;
  const int d = blockIdx.x;
  uint32_t carry = 0;
  uint32_t *row = counts + static_cast<int64_t>(d) * num_tiles;
  for (int c0 = 0; c0 < num_tiles; c0 += kBlockThreads) {
    const int i = c0 + tid;
    const uint32_t x = i < num_tiles ? row[i] : 0u;
    uint32_t total;
    const uint32_t incl = block_inclusive_scan(x, s_wave, total);
    if (i < num_tiles) row[i] = carry + incl - x;
    carry += total;
    __syncthreads();
  }
  if (tid == 0) totals[d] = carry;
}

template <int BITS>
__global__ __launch_bounds__(kBlockThreads) void radix_scatter_kernel(
    const uint32_t *__restrict__ keys_in, const uint32_t *__restrict__ values_in,
    uint32_t *__restrict__ keys_out, uint32_t *__restrict__ values_out, int64_t n, int shift,
    uint32_t mask, int num_tiles, const uint32_t *__restrict__ bases,
    const uint32_t *__restrict__ totals) {
  constexpr int kBinsT = 1 << BITS;
  constexpr int kOwned = kBinsT / kBlockThreads;  // consecutive digits per thread
  __shared__ uint32_t s_keys[kTile];
  __shared__ uint32_t s_vals[kTile];
  __shared__ uint32_t s_wave_count[kWavesPerBlock][kBinsT];
  __shared__ uint32_t s_bin_start[kBinsT];
  __shared__ uint32_t s_dest[kBinsT];
  __shared__ uint32_t s_scan[kWavesPerBlock];

  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  const int64_t tile_base = static_cast<int64_t>(blockIdx.x) * kTile;
  const int tile_count = static_cast<int>(min(static_cast<int64_t>(kTile), n - tile_base));

#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w)
#pragma unroll
    for (int d = tid; d < kBinsT; d += kBlockThreads) s_wave_count[w][d] = 0;

  uint32_t key[kItems], val[kItems];
  const int64_t wave_base = tile_base + wave * kWaveTile;
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int64_t i = wave_base + k * kWave + lane;
    const bool valid = i < n;
    key[k] = valid ? keys_in[i] : 0xffffffffu;
    val[k] = valid ? (values_in ? values_in[i] : static_cast<uint32_t>(i)) : 0u;
  }
  __syncthreads();

  // Rank of each key among the keys of its wavefront that share its digit.
  uint32_t rank[kItems];
#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const bool valid = (wave_base + k * kWave + lane) < n;
    const uint32_t digit = (key[k] >> shift) & mask;
    unsigned long long peers = __ballot(valid);
#pragma unroll
    for (int bit = 0; bit < BITS; ++bit) {
      const bool set = (digit >> bit) & 1u;
      const unsigned long long vote = __ballot(set);
      peers &= set ? vote : ~vote;
    }
    const unsigned long long below = peers & ((1ull << lane) - 1ull);
    uint32_t run_start = 0;
    if (valid && below == 0ull) {
      run_start = atomicAdd(&s_wave_count[wave][digit], static_cast<uint32_t>(__popcll(peers)));
    }
    const int leader = valid ? (__ffsll(static_cast<long long>(peers)) - 1) : lane;
    run_start = __shfl(run_start, leader, kWave);
    rank[k] = run_start + static_cast<uint32_t>(__popcll(below));
  }
  __syncthreads();

  // Thread `tid` owns digits [tid * kOwned, (tid + 1) * kOwned): prefix over wavefronts, then
  // over digits (thread-local, then across the workgroup).
  {
    uint32_t digit_count[kOwned];
    uint32_t mine = 0;
#pragma unroll
    for (int q = 0; q < kOwned; ++q) {
      const int d = tid * kOwned + q;
      uint32_t running = 0;
#pragma unroll
      for (int w = 0; w < kWavesPerBlock; ++w) {
        const uint32_t c = s_wave_count[w][d];
        s_wave_count[w][d] = running;
        running += c;
      }
      digit_count[q] = running;
      mine += running;
    }
    uint32_t total;
    uint32_t bin_start = block_inclusive_scan(mine, s_scan, total) - mine;
    __syncthreads();
    uint32_t totals_mine = 0;
    uint32_t digit_total[kOwned];
#pragma unroll
    for (int q = 0; q < kOwned; ++q) {
      digit_total[q] = totals[tid * kOwned + q];
      totals_mine += digit_total[q];
    }
    uint32_t smaller = block_inclusive_scan(totals_mine, s_scan, total) - totals_mine;
#pragma unroll
    for (int q = 0; q < kOwned; ++q) {
      const int d = tid * kOwned + q;
      s_bin_start[d] = bin_start;
      s_dest[d] = smaller + bases[static_cast<int64_t>(d) * num_tiles + blockIdx.x] - bin_start;
      bin_start += digit_count[q];
      smaller += digit_total[q];
    }
  }
  __syncthreads();

#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const bool valid = (wave_base + k * kWave + lane) < n;
    if (valid) {
      const uint32_t digit = (key[k] >> shift) & mask;
      const uint32_t local = s_bin_start[digit] + s_wave_count[wave][digit] + rank[k];
      s_keys[local] = key[k];
      s_vals[local] = val[k];
    }
  }
  __syncthreads();

#pragma unroll
  for (int k = 0; k < kItems; ++k) {
    const int local = k * kBlockThreads + tid;
    if (local < tile_count) {
      const uint32_t kk = s_keys[local];
      const uint32_t dst = s_dest[(kk >> shift) & mask] + static_cast<uint32_t>(local);
      keys_out[dst] = kk;
      values_out[dst] = s_vals[local];
    }
  }
}

// -------------------------------------------------------------- find segments
// Thread owns kSegItems consecutive sorted positions.  head(i) = i == 0 || key[i] != key[i-1]
// (table_batched_embeddings_cuda.cu:1523-1525).
__device__ __forceinline__ uint32_t segment_head_flags(const uint32_t *__restrict__ keys, int64_t n,
                                                       int64_t first) {
  uint32_t flags = 0;
  if (first >= n) return 0;
  uint32_t prev = first > 0 ? keys[first - 1] : 0u;
#pragma unroll
  for (int k = 0; k < kSegItems; ++k) {
    const int64_t i = first + k;
    if (i < n) {
      const uint32_t cur = keys[i];
      if (i == 0 || cur != prev) flags |= 1u << k;
      prev = cur;
    }
  }
  return flags;
}

__global__ __launch_bounds__(kBlockThreads) void segment_count_kernel(
    const uint32_t *__restrict__ keys, int64_t n, uint32_t *__restrict__ tile_heads) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x) * kSegItems;
  uint32_t total;
  (void)block_inclusive_scan(__popc(segment_head_flags(keys, n, first)), s_wave, total);
  if (threadIdx.x == 0) tile_heads[blockIdx.x] = total;
}

// Single workgroup: exclusive scan of the per-tile head counts; publishes U and
// the closing boundary segment_starts[U] = n.
__global__ __launch_bounds__(kBlockThreads) void segment_scan_kernel(
    uint32_t *__restrict__ tile_heads, int num_tiles, int64_t n,
    int32_t *__restrict__ segment_starts, int32_t *__restrict__ num_unique, int clear_queue_counters) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int tid = threadIdx.x;
  uint32_t carry = 0;
  for (int c0 = 0; c0 < num_tiles; c0 += kBlockThreads) {
    const int i = c0 + tid;
    const uint32_t x = i < num_tiles ? tile_heads[i] : 0u;
    uint32_t total;
    const uint32_t incl = block_inclusive_scan(x, s_wave, total);
    if (i < num_tiles) tile_heads[i] = carry + incl - x;
    carry += total;
    __syncthreads();
  }
  if (tid == 0) {
    num_unique[0] = static_cast<int32_t>(carry);
    segment_starts[carry] = static_cast<int32_t>(n);
  }
  // the update stage keeps three queue counters next to U; starting them at zero here saves a launch
  if (clear_queue_counters && tid >= 1 && tid <= 3) num_unique[tid] = 0;
}

__global__ __launch_bounds__(kBlockThreads) void segment_write_kernel(
    const uint32_t *__restrict__ keys, int64_t n, const uint32_t *__restrict__ tile_base,
    int32_t *__restrict__ segment_starts, int32_t *__restrict__ segment_ids) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t first = (static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x) * kSegItems;
  const uint32_t flags = segment_head_flags(keys, n, first);
  const uint32_t mine = __popc(flags);
  uint32_t total;
  const uint32_t incl = block_inclusive_scan(mine, s_wave, total);
  uint32_t u = tile_base[blockIdx.x] + incl - mine;
#pragma unroll
  for (int k = 0; k < kSegItems; ++k) {
    if (flags & (1u << k)) segment_starts[u++] = static_cast<int32_t>(first + k);
    // u now counts the heads at or before this position: its segment is u - 1
    if (segment_ids && first + k < n) segment_ids[first + k] = static_cast<int32_t>(u) - 1;
  }
}

inline int num_sort_tiles(int64_t n) { return static_cast<int>(ceil_div(n, kTile)); }
inline int num_seg_tiles(int64_t n) { return static_cast<int>(ceil_div(n, kSegTile)); }

}  // namespace

// Sort workspace: [tmp keys n][tmp values n][counts 1024*tiles][totals 1024*passes]
constexpr int kMaxPasses = 4;

uint64_t sort_workspace_bytes(int64_t n) {
  const uint64_t tiles = num_sort_tiles(n > 0 ? n : 1);
  return align_up(static_cast<uint64_t>(n > 0 ? n : 1) * 4, 256) * 2 +
         align_up(tiles * kMaxBins * 4, 256) + align_up(kMaxPasses * kMaxBins * 4, 256);
}

namespace {
template <int BITS>
void launch_radix_pass(const uint32_t *src_k, const uint32_t *src_v, uint32_t *dst_k, uint32_t *dst_v,
                       int64_t n, int shift, uint32_t mask, int tiles, uint32_t *counts, uint32_t *totals,
                       hipStream_t stream) {
  const dim3 block(kBlockThreads);
  TBE_LAUNCH("radix_histogram", stream, radix_histogram_kernel<BITS>, dim3(tiles), block, src_k, n, shift,
             mask, tiles, counts);
  TBE_LAUNCH("radix_scan", stream, radix_scan_kernel, dim3(1 << BITS), block, counts, totals, tiles);
  TBE_LAUNCH("radix_scatter", stream, radix_scatter_kernel<BITS>, dim3(tiles), block, src_k, src_v, dst_k,
             dst_v, n, shift, mask, tiles, counts, totals);
}
}  // namespace

int sort_pairs(const int32_t *keys_in, const int32_t *values_in, int32_t *keys_out,
               int32_t *values_out, int64_t n, int32_t end_bit, void *workspace,
               hipStream_t stream) {
  if (n == 0) return TBE_OK;
  // Fewest passes with digits of at most 10 bits, the bits spread evenly over the passes
  // (23 bits -> 8+8+7, 25 -> 9+8+8, 27 -> 9+9+9, 17 -> 9+8).
  const int passes = end_bit <= 0 ? 1 : static_cast<int>(ceil_div(end_bit, kMaxRadixBits));
  const int tiles = num_sort_tiles(n);
  char *ws = static_cast<char *>(workspace);
  uint32_t *tmp_keys = reinterpret_cast<uint32_t *>(ws);
  ws += align_up(static_cast<uint64_t>(n) * 4, 256);
  uint32_t *tmp_vals = reinterpret_cast<uint32_t *>(ws);
  ws += align_up(static_cast<uint64_t>(n) * 4, 256);
  uint32_t *counts = reinterpret_cast<uint32_t *>(ws);
  ws += align_up(static_cast<uint64_t>(tiles) * kMaxBins * 4, 256);
  uint32_t *totals = reinterpret_cast<uint32_t *>(ws);

  const uint32_t *src_k = reinterpret_cast<const uint32_t *>(keys_in);
  const uint32_t *src_v = reinterpret_cast<const uint32_t *>(values_in);
  int shift = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const int remaining = end_bit <= 0 ? 0 : end_bit - shift;
    const int bits = static_cast<int>(ceil_div(remaining, passes - pass));
    const uint32_t mask = (1u << bits) - 1u;
    const bool to_out = ((passes - 1 - pass) % 2) == 0;
    uint32_t *dst_k = to_out ? reinterpret_cast<uint32_t *>(keys_out) : tmp_keys;
    uint32_t *dst_v = to_out ? reinterpret_cast<uint32_t *>(values_out) : tmp_vals;
    uint32_t *pass_totals = totals + pass * kMaxBins;
    if (bits <= 8)
      launch_radix_pass<8>(src_k, src_v, dst_k, dst_v, n, shift, mask, tiles, counts, pass_totals, stream);
    else if (bits == 9)
      launch_radix_pass<9>(src_k, src_v, dst_k, dst_v, n, shift, mask, tiles, counts, pass_totals, stream);
    else
      launch_radix_pass<10>(src_k, src_v, dst_k, dst_v, n, shift, mask, tiles, counts, pass_totals, stream);
    src_k = dst_k;
    src_v = dst_v;
    shift += bits;
  }
  return check_launch("tbe_sort_pairs");
}

uint64_t segments_workspace_bytes(int64_t n) {
  return align_up(static_cast<uint64_t>(num_seg_tiles(n > 0 ? n : 1)) * 4, 256);
}

int find_segments(const int32_t *keys_sorted, int64_t n, int32_t *segment_starts,
                  int32_t *num_unique, int32_t *segment_ids, void *workspace, hipStream_t stream,
                  bool clear_queue_counters) {
  const int tiles = n > 0 ? num_seg_tiles(n) : 0;
  uint32_t *tile_heads = static_cast<uint32_t *>(workspace);
  const uint32_t *keys = reinterpret_cast<const uint32_t *>(keys_sorted);
  const dim3 block(kBlockThreads);
  if (tiles > 0)
    TBE_LAUNCH("segment_count", stream, segment_count_kernel, dim3(tiles), block, keys, n,
               tile_heads);
  TBE_LAUNCH("segment_scan", stream, segment_scan_kernel, dim3(1), block, tile_heads, tiles, n,
             segment_starts, num_unique, clear_queue_counters ? 1 : 0);
  if (tiles > 0)
    TBE_LAUNCH("segment_write", stream, segment_write_kernel, dim3(tiles), block, keys, n,
               tile_heads, segment_starts, segment_ids);
  return check_launch("tbe_find_segments");
}

int linearize(const int32_t *table_offsets, int32_t T, const int32_t *indices,
              const int32_t *offsets, int32_t B, int32_t *keys, int32_t *grad_rows,
              hipStream_t stream) {
  const int64_t num_bags = static_cast<int64_t>(T) * B;
  const dim3 grid(static_cast<unsigned>(ceil_div(num_bags * kLinLanes, kBlockThreads)));
  TBE_LAUNCH("linearize", stream, linearize_kernel, grid, dim3(kBlockThreads), table_offsets,
             indices, offsets, B, T, static_cast<int>(num_bags), keys, grad_rows);
  return check_launch("tbe_linearize");
}

}  // namespace tbe

extern "C" int tbe_linearize(const int32_t *table_offsets, int32_t T, const int32_t *indices,
                             int64_t num_indices, const int32_t *offsets, int32_t B,
                             int32_t *keys, int32_t *grad_rows, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(T > 0 && B > 0, "tbe_linearize: T and B must be positive (got %d, %d)", T, B);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "tbe_linearize: T*B out of range");
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "tbe_linearize: num_indices out of range");
  TBE_REQUIRE(table_offsets && offsets, "tbe_linearize: null pointer argument");
  if (num_indices == 0) return TBE_OK;
  TBE_REQUIRE(indices && keys && grad_rows, "tbe_linearize: null pointer argument");
  return linearize(table_offsets, T, indices, offsets, B, keys, grad_rows,
                   static_cast<hipStream_t>(stream));
}

extern "C" int tbe_interleaved_rows(const int32_t *indices, int64_t num_indices,
                                    const int32_t *offsets, int32_t T, int32_t B, int32_t *rows,
                                    void *stream) {
  using namespace tbe;
  TBE_REQUIRE(T > 0 && B > 0, "tbe_interleaved_rows: T and B must be positive (got %d, %d)", T, B);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "tbe_interleaved_rows: T*B out of range");
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "tbe_interleaved_rows: num_indices out of range");
  TBE_REQUIRE(offsets, "tbe_interleaved_rows: null offsets");
  if (num_indices == 0) return TBE_OK;
  TBE_REQUIRE(indices && rows, "tbe_interleaved_rows: null pointer argument");
  const int64_t num_bags = static_cast<int64_t>(T) * B;
  hipStream_t s = static_cast<hipStream_t>(stream);
  TBE_LAUNCH("interleaved_rows", s, interleaved_rows_kernel,
             dim3(static_cast<unsigned>(ceil_div(num_bags * kLinLanes, kBlockThreads))), dim3(kBlockThreads),
             indices, offsets, T, static_cast<int>(num_bags), rows);
  return check_launch("tbe_interleaved_rows");
}

extern "C" uint64_t tbe_sort_workspace_bytes(int64_t n) { return tbe::sort_workspace_bytes(n); }

extern "C" int tbe_sort_pairs(const int32_t *keys_in, const int32_t *values_in, int32_t *keys_out,
                              int32_t *values_out, int64_t n, int32_t end_bit, void *workspace,
                              uint64_t workspace_bytes, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(n >= 0 && n < INT32_MAX, "tbe_sort_pairs: n out of range");
  TBE_REQUIRE(end_bit >= 0 && end_bit <= 32, "tbe_sort_pairs: end_bit must be in [0, 32] (got %d)", end_bit);
  if (n == 0) return TBE_OK;
  TBE_REQUIRE(keys_in && keys_out && values_out, "tbe_sort_pairs: null pointer argument");
  if (!workspace || workspace_bytes < sort_workspace_bytes(n))
    return fail(TBE_ERR_WORKSPACE, "tbe_sort_pairs: workspace of %llu bytes needed, %llu given",
                (unsigned long long)sort_workspace_bytes(n), (unsigned long long)workspace_bytes);
  return sort_pairs(keys_in, values_in, keys_out, values_out, n, end_bit, workspace,
                    static_cast<hipStream_t>(stream));
}

extern "C" uint64_t tbe_segments_workspace_bytes(int64_t n) { return tbe::segments_workspace_bytes(n); }

extern "C" int tbe_find_segments(const int32_t *keys_sorted, int64_t n, int32_t *segment_starts,
                                 int32_t *num_unique, void *workspace, uint64_t workspace_bytes,
                                 void *stream) {
  using namespace tbe;
  TBE_REQUIRE(n >= 0 && n < INT32_MAX, "tbe_find_segments: n out of range");
  TBE_REQUIRE(segment_starts && num_unique, "tbe_find_segments: null pointer argument");
  TBE_REQUIRE(keys_sorted || n == 0, "tbe_find_segments: null keys");
  if (!workspace || workspace_bytes < segments_workspace_bytes(n))
    return fail(TBE_ERR_WORKSPACE, "tbe_find_segments: workspace of %llu bytes needed, %llu given",
                (unsigned long long)segments_workspace_bytes(n), (unsigned long long)workspace_bytes);
  return find_segments(keys_sorted, n, segment_starts, num_unique, nullptr, workspace,
                       static_cast<hipStream_t>(stream), /*clear_queue_counters=*/false);
}
