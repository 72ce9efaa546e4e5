// Integer stages of the backward pass for gfx950:
//   linearize      (table,row) keys and the gradient row of every lookup
//   sort_pairs     stable LSD radix sort, 8-bit digits, LDS-staged scatter
//   find_segments  run boundaries of the sorted keys (one per unique row)
//
// The sort is the contract of cub::DeviceRadixSort::SortPairs as the reference
// calls it (table_batched_embeddings_cuda.cu:1639-1655): ascending, stable,
// key bits [0, end_bit).  A pass handles a digit of 8 to 10 bits (the fewest passes that cover
// end_bit).  Each pass is two or four kernels:
//   histogram  per-tile digit counts (LDS atomics)
//   scan       turns the counts into the output position of every (table, digit, tile) run.
//              Many tables of few tiles each (the backward's case: every table is sorted on its
//              own): no kernel.  Counts are kept as counts[tile][digit], the histogram also adds
//              its counts to per-table digit totals (and to totals of every 64 tiles), and the
//              scatter kernel of a tile scans the table's totals over the digits and adds up the
//              counts of the table's earlier tiles itself.  Otherwise: counts[table][digit][tile]
//              and a linear exclusive prefix sum over the whole array (workgroup sums, then the
//              chunks)
//   scatter    ranks each key inside its tile with wavefront ballots (all lanes
//              holding the same digit are found with one ballot per digit bit; the lowest lane
//              reserves the run in a per-wavefront LDS counter), reorders the
//              tile in LDS so every digit's keys are contiguous, and writes
//              them out in runs.
// A tile is 4096 pairs (1024 for small inputs); position order inside a tile is (wavefront, item, lane),
// which the ranking preserves, so the sort is stable.

#include <algorithm>

#include "tbe_stages.h"

namespace tbe {
namespace {

constexpr int kMaxRadixBits = 10;                 // widest digit of a pass
constexpr int kMaxBins = 1 << kMaxRadixBits;
constexpr int kItems = 16;                        // pairs per thread per tile
constexpr int kTile = kBlockThreads * kItems;     // 4096
// Small inputs are sorted in tiles of a quarter that size: at 4096 pairs per workgroup they would
// leave most compute units without work, and what they move fits in L2, where the shorter runs
// of the scatter cost nothing.
constexpr int kSmallItems = 4;
constexpr int64_t kSmallSortPairs = 1 << 19;      // up to this many pairs: kSmallItems per thread
inline int sort_items(int64_t n) { return n <= kSmallSortPairs ? kSmallItems : kItems; }

// Per-table layout of the counts: the scatter kernel of a tile adds up the counts of the earlier
// tiles of its table itself.  So that a table of many tiles costs it few loads, the histogram
// kernel also collects the counts of every kGroupTiles consecutive tiles (numbered over all tables)
// in group totals: a range of tiles is then its whole groups plus fewer than kGroupTiles tiles at
// either end.
constexpr int kGroupTiles = 64;

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
// 8 lanes per bag.  Mirrors linear_index_weight_offsets_kernel
// (table_batched_embeddings_cuda.cu:1471-1497); instead of the 8-byte
// IndexInfo{b_t, indices_idx} payload it records the gradient row b*T + t of
// each position, and the sort carries the position itself.  `keys` may be null (the fused
// backward sorts the indices themselves, table by table).
constexpr int kLinLanes = 8;  // measured: 8 lanes per bag 11.5 us, 16: 14.1, 4: 12.7, 32: 21.3 (5.2 M lookups, ~20 per bag)
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
  const int32_t row0 = keys ? table_offsets[t] : 0;
  const int32_t grow = b * num_tables + t;
  const int start = offsets[bag];
  const int end = offsets[bag + 1];
  if (keys) {
    for (int p = start + sub; p < end; p += kLinLanes) {
      keys[p] = row0 + indices[p];
      grad_rows[p] = grow;
    }
  } else {
    for (int p = start + sub; p < end; p += kLinLanes) grad_rows[p] = grow;
  }
}

// ------------------------------------------------ interleaved tables -> table-major batch
// Tables stored [E][T][D] number their bags b*T + t and bound bag (b, t) by offsets[b * stride + t]
// and the entry after it (sparse_embedding_cuda_kernel.cu:221-284).  The backward needs the lookups
// table by table (the sort works on one table's consecutive positions, the update walks gradient
// rows table by table), so the batch is put into that order once: three small launches, one pass
// over the indices.  After them `indices_tm` / `offsets_tm` are a table-major batch [T][B].
//
// Bags are taken kBlockThreads at a time: chunk c of table t holds bags c*256 ... of that table.
// Launch 1, one workgroup per chunk: the chunk's lookups.
__global__ __launch_bounds__(kBlockThreads) void interleaved_chunk_sums_kernel(
    const int32_t *__restrict__ offsets, int offsets_stride, int B, int chunks_per_table,
    int32_t *__restrict__ chunk_sums) {
  __shared__ int32_t s_part[kWavesPerBlock];
  const int t = blockIdx.x / chunks_per_table;
  const int b = (blockIdx.x - t * chunks_per_table) * kBlockThreads + threadIdx.x;
  int32_t sum = 0;
  if (b < B) {
    const int64_t at = static_cast<int64_t>(b) * offsets_stride + t;
    sum = offsets[at + 1] - offsets[at];
  }
  for (int m = kWave / 2; m > 0; m >>= 1) sum += __shfl_xor(sum, m, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) s_part[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t total = 0;
    for (int w = 0; w < kWavesPerBlock; ++w) total += s_part[w];
    chunk_sums[blockIdx.x] = total;
  }
}

// Launch 2, one workgroup per table: the table's lookups, and bias[t] = t for the sort's last pass.
__global__ __launch_bounds__(kBlockThreads) void interleaved_totals_kernel(
    const int32_t *__restrict__ chunk_sums, int chunks_per_table, int32_t *__restrict__ totals,
    int32_t *__restrict__ bias) {
  __shared__ int32_t s_part[kWavesPerBlock];
  const int t = blockIdx.x;
  int32_t sum = 0;
  for (int c = threadIdx.x; c < chunks_per_table; c += kBlockThreads)
    sum += chunk_sums[static_cast<int64_t>(t) * chunks_per_table + c];
  for (int m = kWave / 2; m > 0; m >>= 1) sum += __shfl_xor(sum, m, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0) s_part[threadIdx.x >> 6] = sum;
  __syncthreads();
  if (threadIdx.x == 0) {
    int32_t total = 0;
    for (int w = 0; w < kWavesPerBlock; ++w) total += s_part[w];
    totals[t] = total;
    bias[t] = t;
  }
}

// Launch 3, one workgroup per chunk: offsets_tm[t*B + b] = lookups of the tables before t + of the
// table's chunks before this one + of the chunk's bags before b; the last workgroup also writes
// offsets_tm[T*B].
__global__ __launch_bounds__(kBlockThreads) void interleaved_offsets_kernel(
    const int32_t *__restrict__ offsets, int offsets_stride, int B, int num_tables, int chunks_per_table,
    const int32_t *__restrict__ totals, const int32_t *__restrict__ chunk_sums,
    int32_t *__restrict__ offsets_tm) {
  __shared__ int32_t s_part[kWavesPerBlock];
  __shared__ int32_t s_scan[kWavesPerBlock];
  const int t = blockIdx.x / chunks_per_table;
  const int chunk = blockIdx.x - t * chunks_per_table;
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  int32_t before = 0;
  for (int k = threadIdx.x; k < t; k += kBlockThreads) before += totals[k];
  for (int k = threadIdx.x; k < chunk; k += kBlockThreads)
    before += chunk_sums[static_cast<int64_t>(t) * chunks_per_table + k];
  for (int m = kWave / 2; m > 0; m >>= 1) before += __shfl_xor(before, m, kWave);
  const int b = chunk * kBlockThreads + threadIdx.x;
  int32_t len = 0;
  if (b < B) {
    const int64_t at = static_cast<int64_t>(b) * offsets_stride + t;
    len = offsets[at + 1] - offsets[at];
  }
  int32_t x = len;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int32_t y = __shfl_up(x, d, kWave);
    if (lane >= d) x += y;
  }
  if (lane == 0) s_part[wave] = before;
  if (lane == kWave - 1) s_scan[wave] = x;
  __syncthreads();
  int32_t carry = 0, all = 0;
#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w) {
    carry += s_part[w];
    if (w < wave) carry += s_scan[w];
    all += s_scan[w];
  }
  if (b < B) offsets_tm[static_cast<int64_t>(t) * B + b] = carry + x - len;
  if (blockIdx.x == gridDim.x - 1 && threadIdx.x == kBlockThreads - 1)
    offsets_tm[static_cast<int64_t>(num_tables) * B] = carry + x;
}

// 8 lanes per bag: the bag's indices go to their place in the table-major order.
__global__ __launch_bounds__(kBlockThreads) void interleaved_permute_kernel(
    const int32_t *__restrict__ indices, const int32_t *__restrict__ offsets, int offsets_stride, int B,
    int num_tables, int num_bags, const int32_t *__restrict__ offsets_tm, int32_t *__restrict__ indices_tm) {
  const int64_t gid = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  const int64_t bag64 = gid / kLinLanes;
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);  // t*B + b: consecutive wavefronts write consecutive memory
  const int t = bag / B;
  const int b = bag - t * B;
  const int64_t at = static_cast<int64_t>(b) * offsets_stride + t;
  const int src = offsets[at];
  const int len = offsets[at + 1] - src;
  const int dst = offsets_tm[bag];
  for (int i = static_cast<int>(gid % kLinLanes); i < len; i += kLinLanes) indices_tm[dst + i] = indices[src + i];
}

// The gradient row b*T + t of every position, 8 lanes per bag, for workgroup `block` of
// ceil(num_bags * 8 / 256): what linearize_kernel writes when it is given no keys.
__device__ __forceinline__ void record_gradient_rows(const int32_t *__restrict__ offsets, int B,
                                                     int num_tables, int num_bags, int64_t block,
                                                     int32_t *__restrict__ grad_rows) {
  const int64_t gid = block * kBlockThreads + threadIdx.x;
  const int64_t bag64 = gid / kLinLanes;
  if (bag64 >= num_bags) return;
  const int bag = static_cast<int>(bag64);
  const int t = bag / B;
  const int32_t grow = (bag - t * B) * num_tables + t;
  const int end = offsets[bag + 1];
  for (int p = offsets[bag] + static_cast<int>(gid % kLinLanes); p < end; p += kLinLanes) grad_rows[p] = grow;
}

// ------------------------------------------------------------------ radix sort
// The pairs may come in consecutive *tables* (table t owns positions [offsets[t*B], offsets[(t+1)*B]),
// as in the bag layout): every table is then sorted on its own, so only the bits of a row number
// inside its table are sorted, and the result is the sort by (table, row).  Tiles never straddle
// tables: table t owns ceil(n_t / 4096) tiles, tile_prefix[] is the running tile count.  Without
// tables the whole input is one table.
//
// counts[] holds, for table t with tiles_t tiles, a [bins][tiles_t] block at bins * tile_prefix[t]:
// in that order (table, digit, tile) one exclusive prefix sum over the whole array is the output
// position of the first key of every (table, digit, tile) run.

constexpr int kScanItems = 8;
constexpr int kScanChunk = kBlockThreads * kScanItems;  // 2048 count entries per workgroup

// Workgroup 0 derives the tables' position ranges and tile counts; the first setup_blocks
// workgroups clear the per-table digit totals of every pass (`totals_words` words; none with the
// linear scan).  The workgroups after them, if any, record the gradient row of every position
// (grad_rows non-null, with tables): work of the caller's that depends on nothing here and would
// otherwise be one more launch in the chain.
// device_count (nullable): the number of pairs to sort when only the device knows it (at most n,
// for which the launches are sized: tiles past the count find nothing to do).
template <int ITEMS>
__global__ __launch_bounds__(kBlockThreads) void sort_setup_kernel(
    const int32_t *__restrict__ offsets, int B, int num_tables, uint32_t n,
    uint32_t *__restrict__ table_starts, uint32_t *__restrict__ tile_prefix,
    uint32_t *__restrict__ totals, int64_t totals_words, const int32_t *__restrict__ device_count,
    int setup_blocks, int32_t *__restrict__ grad_rows) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int tid = threadIdx.x;
  if (static_cast<int>(blockIdx.x) >= setup_blocks) {
    record_gradient_rows(offsets, B, num_tables, num_tables * B, static_cast<int64_t>(blockIdx.x) - setup_blocks,
                         grad_rows);
    return;
  }
  if (device_count) n = min(n, static_cast<uint32_t>(max(*device_count, 0)));
  for (int64_t i = (static_cast<int64_t>(blockIdx.x) * kBlockThreads + tid) * 4; i < totals_words;
       i += static_cast<int64_t>(setup_blocks) * kBlockThreads * 4)
    *reinterpret_cast<uint4 *>(totals + i) = make_uint4(0, 0, 0, 0);
  if (blockIdx.x != 0) return;
  uint32_t carry = 0;
  for (int c0 = 0; c0 < num_tables; c0 += kBlockThreads) {
    const int t = c0 + tid;
    uint32_t tiles = 0;
    if (t < num_tables) {
      uint32_t start = 0, end = n;
      if (offsets) {
        start = min(static_cast<uint32_t>(max(offsets[static_cast<int64_t>(t) * B], 0)), n);
        if (t + 1 < num_tables)
          end = min(static_cast<uint32_t>(max(offsets[static_cast<int64_t>(t + 1) * B], 0)), n);
      }
      end = max(end, start);
      tiles = (end - start + kBlockThreads * ITEMS - 1) / (kBlockThreads * ITEMS);
      table_starts[t] = start;
    }
    uint32_t total;
    const uint32_t incl = block_inclusive_scan(tiles, s_wave, total);
    if (t < num_tables) tile_prefix[t] = carry + incl - tiles;
    carry += total;
    __syncthreads();
  }
  if (tid == 0) {
    table_starts[num_tables] = n;
    tile_prefix[num_tables] = carry;
  }
}

// What a workgroup needs to know about its tile.
struct TileInfo {
  int table;
  int64_t begin;       // first position of the tile
  int count;           // pairs in the tile (0: nothing to do)
  int64_t count_base;  // index of counts[table][digit 0][this tile]
  int table_tiles;     // stride between digits in counts[]
  int64_t tile_index;  // number of the tile among all tiles
  int64_t first_tile;  // number of the table's first tile
};

template <int BITS, int ITEMS>
__device__ __forceinline__ TileInfo locate_tile(const uint32_t *__restrict__ table_starts,
                                                const uint32_t *__restrict__ tile_prefix,
                                                int num_tables, int max_tiles) {
  TileInfo info{0, 0, 0, 0, 0, 0, 0};
  // Workgroups go to the eight XCDs in turn: workgroup b takes tile (b % 8) * ceil(tiles / 8) + b / 8,
  // so that an XCD works on consecutive tiles (mostly of one table at a time).  The runs that those
  // tiles scatter into the same output lines then meet in one L2, and the scatter kernel finds the
  // keys and the counts there that the histogram kernel of the same tiles left.
  const uint32_t all_tiles = tile_prefix[num_tables];
  const uint32_t per_xcd = (all_tiles + kNumXcd - 1) / kNumXcd;
  const uint32_t turn = blockIdx.x / kNumXcd;
  const uint32_t tile = (blockIdx.x % kNumXcd) * per_xcd + turn;
  if (turn >= per_xcd || tile >= all_tiles) return info;
  int lo = 0, hi = num_tables;  // tile_prefix[lo] <= tile < tile_prefix[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (tile_prefix[mid] <= tile) lo = mid; else hi = mid;
  }
  const uint32_t first_tile = tile_prefix[lo];
  const uint32_t tiles = tile_prefix[lo + 1] - first_tile;
  if (first_tile + tiles > static_cast<uint32_t>(max_tiles)) return info;  // inconsistent offsets
  const uint32_t j = tile - first_tile;
  info.table = lo;
  info.begin = static_cast<int64_t>(table_starts[lo]) + static_cast<int64_t>(j) * (kBlockThreads * ITEMS);
  const int64_t left = static_cast<int64_t>(table_starts[lo + 1]) - info.begin;
  info.count = static_cast<int>(max(int64_t{0}, min(left, static_cast<int64_t>(kBlockThreads * ITEMS))));
  info.count_base = (static_cast<int64_t>(first_tile) << BITS) + j;
  info.table_tiles = static_cast<int>(tiles);
  info.tile_index = static_cast<int64_t>(tile);
  info.first_tile = static_cast<int64_t>(first_tile);
  return info;
}

// Where the count of digit d of a tile lives.  LOCAL: counts[tile][digit] (a tile's counts are
// contiguous: coalesced stores and loads); else counts[table][digit][tile] (the order of the
// linear scan).
template <int BITS, bool LOCAL>
__device__ __forceinline__ int64_t count_index(const TileInfo &tile, int d) {
  if constexpr (LOCAL) return (tile.tile_index << BITS) + d;
  else return tile.count_base + static_cast<int64_t>(d) * tile.table_tiles;
}

// BITS = digit width of the pass (8, 9 or 10): 2^BITS bins, each thread owns 2^BITS / 256
// consecutive digits in the per-digit steps.
template <int BITS, bool LOCAL, int ITEMS>
__global__ __launch_bounds__(kBlockThreads) void radix_histogram_kernel(
    const uint32_t *__restrict__ keys, const uint32_t *__restrict__ table_starts,
    const uint32_t *__restrict__ tile_prefix, int num_tables, int max_tiles, int shift,
    uint32_t mask, uint32_t *__restrict__ counts, uint32_t *__restrict__ totals,
    uint32_t *__restrict__ group_totals) {
  constexpr int kBinsT = 1 << BITS;
  // Four counters per digit, in neighbouring LDS banks, one for every fourth lane: the lanes of a
  // wavefront that hold a hot digit (a popular row) then queue at four addresses instead of one.
  constexpr int kCopies = 4;
  __shared__ uint4 s_hist[kBinsT];
  uint32_t *s_counter = reinterpret_cast<uint32_t *>(s_hist);
  const TileInfo tile = locate_tile<BITS, ITEMS>(table_starts, tile_prefix, num_tables, max_tiles);
  if (tile.table_tiles == 0) return;
  const int tid = threadIdx.x;
#pragma unroll
  for (int d = tid; d < kBinsT; d += kBlockThreads) s_hist[d] = make_uint4(0, 0, 0, 0);
  __syncthreads();
  // every thread loads all its keys first (an index past the tile's end is clamped, the key
  // dropped): straight-line loads are issued back to back, predicated ones one at a time
  if (tile.count > 0) {
    uint32_t key[ITEMS];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      key[k] = keys[tile.begin + min(k * kBlockThreads + tid, tile.count - 1)];
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) {
      if (k * kBlockThreads + tid < tile.count)
        atomicAdd(&s_counter[((key[k] >> shift) & mask) * kCopies + (tid & (kCopies - 1))], 1u);
    }
  }
  __syncthreads();
  // (linear-scan layout: one 4-byte store per digit, a tile apart -- these scattered stores are
  // most of the kernel's time there; per-table layout: coalesced stores, and the table's digit
  // totals collect the counts with integer atomics, whose order does not matter; so do the group
  // totals, which only the tiles of a table of more than kGroupTiles tiles can be asked for)
  const bool grouped = LOCAL && tile.table_tiles > kGroupTiles;
#pragma unroll
  for (int d = tid; d < kBinsT; d += kBlockThreads) {
    const uint4 four = s_hist[d];
    const uint32_t c = four.x + four.y + four.z + four.w;
    counts[count_index<BITS, LOCAL>(tile, d)] = c;
    if constexpr (LOCAL) {
      if (c) atomicAdd(&totals[(static_cast<int64_t>(tile.table) << BITS) + d], c);
      if (c && grouped) atomicAdd(&group_totals[((tile.tile_index / kGroupTiles) << BITS) + d], c);
    }
  }
}

// Exclusive prefix sum over counts[0, bins * tiles): workgroup sums first, then every workgroup
// adds up the sums before it and scans its own chunk.
__device__ __forceinline__ void load_scan_items(const uint32_t *__restrict__ counts, int64_t first,
                                                int64_t entries, uint32_t (&x)[kScanItems]) {
  if (first < entries) {  // `entries` is a multiple of 256, so all eight are inside
    const uint4 a = *reinterpret_cast<const uint4 *>(counts + first);
    const uint4 b = *reinterpret_cast<const uint4 *>(counts + first + 4);
    x[0] = a.x; x[1] = a.y; x[2] = a.z; x[3] = a.w;
    x[4] = b.x; x[5] = b.y; x[6] = b.z; x[7] = b.w;
  } else {
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) x[k] = 0;
  }
}

__global__ __launch_bounds__(kBlockThreads) void radix_scan_reduce_kernel(
    const uint32_t *__restrict__ counts, const uint32_t *__restrict__ tile_prefix, int num_tables,
    int bits, uint32_t *__restrict__ block_sums) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t entries = static_cast<int64_t>(tile_prefix[num_tables]) << bits;
  const int64_t first = static_cast<int64_t>(blockIdx.x) * kScanChunk + threadIdx.x * kScanItems;
  uint32_t x[kScanItems];
  load_scan_items(counts, first, entries, x);
  uint32_t mine = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) mine += x[k];
  uint32_t total;
  (void)block_inclusive_scan(mine, s_wave, total);
  if (threadIdx.x == 0) block_sums[blockIdx.x] = total;
}

__global__ __launch_bounds__(kBlockThreads) void radix_scan_kernel(
    uint32_t *__restrict__ counts, const uint32_t *__restrict__ tile_prefix, int num_tables,
    int bits, const uint32_t *__restrict__ block_sums) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int64_t entries = static_cast<int64_t>(tile_prefix[num_tables]) << bits;
  const int64_t chunk_first = static_cast<int64_t>(blockIdx.x) * kScanChunk;
  if (chunk_first >= entries) return;
  uint32_t before = 0;
  for (int i = threadIdx.x; i < static_cast<int>(blockIdx.x); i += kBlockThreads) before += block_sums[i];
  uint32_t prior;
  (void)block_inclusive_scan(before, s_wave, prior);
  __syncthreads();
  const int64_t first = chunk_first + threadIdx.x * kScanItems;
  uint32_t x[kScanItems];
  load_scan_items(counts, first, entries, x);
  uint32_t mine = 0;
#pragma unroll
  for (int k = 0; k < kScanItems; ++k) mine += x[k];
  uint32_t total;
  uint32_t running = prior + block_inclusive_scan(mine, s_wave, total) - mine;
  if (first < entries) {
    uint32_t y[kScanItems];
#pragma unroll
    for (int k = 0; k < kScanItems; ++k) {
      y[k] = running;
      running += x[k];
    }
    *reinterpret_cast<uint4 *>(counts + first) = make_uint4(y[0], y[1], y[2], y[3]);
    *reinterpret_cast<uint4 *>(counts + first + 4) = make_uint4(y[4], y[5], y[6], y[7]);
  }
}

// key_bias (nullable): added to the keys of table t as they are written (the last pass turns
// rows inside a table into rows of the concatenated tables), after a multiplication by key_mul
// (1; T for tables stored interleaved, whose row idx of table t is row idx*T + t of one array).
template <int BITS, bool LOCAL, int ITEMS>
__global__ __launch_bounds__(kBlockThreads) void radix_scatter_kernel(
    const uint32_t *__restrict__ keys_in, const uint32_t *__restrict__ values_in,
    uint32_t *__restrict__ keys_out, uint32_t *__restrict__ values_out,
    const uint32_t *__restrict__ table_starts, const uint32_t *__restrict__ tile_prefix,
    int num_tables, int max_tiles, int shift, uint32_t mask, const uint32_t *__restrict__ bases,
    const uint32_t *__restrict__ totals, const uint32_t *__restrict__ group_totals,
    const int32_t *__restrict__ key_bias, uint32_t key_mul) {
  constexpr int kBinsT = 1 << BITS;
  constexpr int kOwned = kBinsT / kBlockThreads;  // consecutive digits per thread
  // The per-wavefront digit counters are only needed until every key knows its slot in the
  // reordered tile.  For 9- and 10-bit digits (8 and 16 KB of counters) they share LDS with the
  // reordered keys, which keeps four workgroups on a compute unit at the price of one more barrier.
  constexpr int kTileT = kBlockThreads * ITEMS;
  constexpr int kWaveTileT = kWave * ITEMS;
  constexpr bool kShareCounters = BITS >= 9 && kWavesPerBlock * kBinsT <= kTileT;
  __shared__ uint32_t s_keys[kTileT];
  __shared__ uint32_t s_vals[kTileT];
  __shared__ uint32_t s_own_count[kShareCounters ? 1 : kWavesPerBlock][kShareCounters ? 1 : kBinsT];
  __shared__ uint32_t s_bin_start[kBinsT];
  __shared__ uint32_t s_dest[kBinsT];
  __shared__ uint32_t s_scan[kWavesPerBlock];
  uint32_t(*s_wave_count)[kBinsT] =
      kShareCounters ? reinterpret_cast<uint32_t(*)[kBinsT]>(s_keys) : reinterpret_cast<uint32_t(*)[kBinsT]>(s_own_count);

  const TileInfo tile = locate_tile<BITS, ITEMS>(table_starts, tile_prefix, num_tables, max_tiles);
  if (tile.table_tiles == 0 || tile.count == 0) return;
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;

  // output position of the tile's first key of every digit this thread owns (needed late;
  // fetched first so the latency hides behind the ranking)
  uint32_t digit_base[kOwned];
  uint32_t digit_total[kOwned];  // per-table layout: keys of the table with each digit
  if constexpr (LOCAL) {
    // bases[] holds counts[tile][digit]: this tile's keys of digit d go behind the table's keys of
    // smaller digits (added up further down, once the totals are here) and behind the keys of
    // digit d in the earlier tiles of the table, [first, tile): fewer than kGroupTiles tiles up to
    // a multiple of kGroupTiles, whole groups, and fewer than kGroupTiles tiles again.
#pragma unroll
    for (int q = 0; q < kOwned; ++q) {
      digit_total[q] = totals[(static_cast<int64_t>(tile.table) << BITS) + tid * kOwned + q];
      digit_base[q] = 0;
    }
    // adds rows [from, to) of a [row][digit] array to digit_base, eight rows requested at a time
    auto add_rows = [&](const uint32_t *__restrict__ rows, int64_t from, int64_t to) {
      constexpr int kAhead = 8;
      const uint32_t *mine = rows + tid * kOwned;
      for (int64_t r0 = from; r0 < to; r0 += kAhead) {
        uint32_t c[kAhead][kOwned];
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
#pragma unroll
          for (int q = 0; q < kOwned; ++q) c[a][q] = mine[(min(r0 + a, to - 1) << BITS) + q];
#pragma unroll
        for (int a = 0; a < kAhead; ++a)
#pragma unroll
          for (int q = 0; q < kOwned; ++q) digit_base[q] += (r0 + a < to) ? c[a][q] : 0u;
      }
    };
    const int64_t first = tile.first_tile;
    const int64_t head_end = (first + kGroupTiles - 1) / kGroupTiles * kGroupTiles;
    const int64_t tail_begin = tile.tile_index / kGroupTiles * kGroupTiles;
    if (head_end >= tail_begin) {
      add_rows(bases, first, tile.tile_index);  // no whole group in between
    } else {
      add_rows(bases, first, head_end);
      add_rows(group_totals, head_end / kGroupTiles, tail_begin / kGroupTiles);
      add_rows(bases, tail_begin, tile.tile_index);
    }
  } else {
#pragma unroll
    for (int q = 0; q < kOwned; ++q) digit_base[q] = bases[count_index<BITS, LOCAL>(tile, tid * kOwned + q)];
  }

#pragma unroll
  for (int w = 0; w < kWavesPerBlock; ++w)
#pragma unroll
    for (int d = tid; d < kBinsT; d += kBlockThreads) s_wave_count[w][d] = 0;

  uint32_t key[ITEMS], val[ITEMS];
  const int wave_first = wave * kWaveTileT;
  // straight-line loads (an index past the tile's end is clamped, what it loads replaced)
#pragma unroll
  for (int k = 0; k < ITEMS; ++k)
    key[k] = keys_in[tile.begin + min(wave_first + k * kWave + lane, tile.count - 1)];
  if (values_in) {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k)
      val[k] = values_in[tile.begin + min(wave_first + k * kWave + lane, tile.count - 1)];
  } else {
#pragma unroll
    for (int k = 0; k < ITEMS; ++k) val[k] = static_cast<uint32_t>(tile.begin + wave_first + k * kWave + lane);
  }
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const bool valid = wave_first + k * kWave + lane < tile.count;
    key[k] = valid ? key[k] : 0xffffffffu;
    val[k] = valid ? val[k] : 0u;
  }
  __syncthreads();

  // Rank of each key among the keys of its wavefront that share its digit.
  uint32_t rank[ITEMS];
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const bool valid = (wave_first + k * kWave + lane) < tile.count;
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
    if constexpr (LOCAL) {
      // first output position of every digit inside the table: exclusive scan of the table's totals
      uint32_t table_sum = 0;
#pragma unroll
      for (int q = 0; q < kOwned; ++q) table_sum += digit_total[q];
      __syncthreads();  // s_scan is read by every wavefront above
      uint32_t all;
      uint32_t digit_start = table_starts[tile.table] + block_inclusive_scan(table_sum, s_scan, all) - table_sum;
#pragma unroll
      for (int q = 0; q < kOwned; ++q) {
        digit_base[q] += digit_start;
        digit_start += digit_total[q];
      }
    }
#pragma unroll
    for (int q = 0; q < kOwned; ++q) {
      const int d = tid * kOwned + q;
      s_bin_start[d] = bin_start;
      s_dest[d] = digit_base[q] - bin_start;
      bin_start += digit_count[q];
    }
  }
  __syncthreads();

  // slot of every key in the reordered tile; the counters are dead after this
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const uint32_t digit = (key[k] >> shift) & mask;
    const bool valid = (wave_first + k * kWave + lane) < tile.count;
    rank[k] += valid ? s_bin_start[digit] + s_wave_count[wave][digit] : 0u;
  }
  if constexpr (kShareCounters) __syncthreads();
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const bool valid = (wave_first + k * kWave + lane) < tile.count;
    if (valid) {
      s_keys[rank[k]] = key[k];
      s_vals[rank[k]] = val[k];
    }
  }
  __syncthreads();

  const uint32_t bias = key_bias ? static_cast<uint32_t>(key_bias[tile.table]) : 0u;
#pragma unroll
  for (int k = 0; k < ITEMS; ++k) {
    const int local = k * kBlockThreads + tid;
    if (local < tile.count) {
      const uint32_t kk = s_keys[local];
      const uint32_t dst = s_dest[(kk >> shift) & mask] + static_cast<uint32_t>(local);
      keys_out[dst] = key_bias ? kk * key_mul + bias : kk;
      values_out[dst] = s_vals[local];
    }
  }
}

// -------------------------------------------------------------- find segments
// Thread owns kSegItems = 8 consecutive sorted positions (two 16-byte loads).
// head(i) = i == 0 || key[i] != key[i-1]   (table_batched_embeddings_cuda.cu:1523-1525).
__device__ __forceinline__ uint32_t segment_head_flags(const uint32_t *__restrict__ keys, int64_t n,
                                                       int64_t first) {
  if (first >= n) return 0;
  uint32_t cur[kSegItems];
  if (first + kSegItems <= n) {
    const uint4 a = *reinterpret_cast<const uint4 *>(keys + first);
    const uint4 b = *reinterpret_cast<const uint4 *>(keys + first + 4);
    cur[0] = a.x; cur[1] = a.y; cur[2] = a.z; cur[3] = a.w;
    cur[4] = b.x; cur[5] = b.y; cur[6] = b.z; cur[7] = b.w;
  } else {
#pragma unroll
    for (int k = 0; k < kSegItems; ++k) cur[k] = first + k < n ? keys[first + k] : 0u;
  }
  // the key before this thread's first one: the neighbouring lane holds it, except in lane 0
  uint32_t prev = __shfl_up(cur[kSegItems - 1], 1, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0 && first > 0) prev = keys[first - 1];
  uint32_t flags = 0;
#pragma unroll
  for (int k = 0; k < kSegItems; ++k) {
    const int64_t i = first + k;
    if (i < n && (i == 0 || cur[k] != prev)) flags |= 1u << k;
    prev = cur[k];
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
  // the update stage keeps its queue counters next to U; starting them at zero here saves a launch
  if (clear_queue_counters) {
    for (int i = tid; i < kNumCounters; i += kBlockThreads)
      if (i >= 1) num_unique[i] = 0;
  }
}

// The heads of a tile are compacted in LDS and leave as one contiguous run; the segment of
// every position leaves in 16-byte stores.  SUM_TILES: `tile_base` holds the head count of
// every tile, not yet scanned: the workgroup adds up the counts of the tiles before its own (a
// few thousand tiles at most: see find_segments), and the last workgroup does what
// segment_scan_kernel does at its end -- one launch less on the path of every backward.
template <bool SUM_TILES>
__global__ __launch_bounds__(kBlockThreads) void segment_write_kernel(
    const uint32_t *__restrict__ keys, int64_t n, const uint32_t *__restrict__ tile_base,
    int32_t *__restrict__ segment_starts, int32_t *__restrict__ segment_ids,
    int32_t *__restrict__ num_unique, int clear_queue_counters) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  __shared__ uint32_t s_wave_tiles[kWavesPerBlock];
  __shared__ int32_t s_heads[kSegTile];
  const int64_t tile_first = static_cast<int64_t>(blockIdx.x) * kSegTile;
  const int64_t first = tile_first + threadIdx.x * kSegItems;
  uint32_t tiles_before = 0;
  if constexpr (SUM_TILES) {
    for (uint32_t i = threadIdx.x; i < blockIdx.x; i += kBlockThreads) tiles_before += tile_base[i];
  }
  const uint32_t flags = segment_head_flags(keys, n, first);
  const uint32_t mine = __popc(flags);
  uint32_t total;
  const uint32_t incl = block_inclusive_scan(mine, s_wave, total);
  uint32_t base;
  if constexpr (SUM_TILES) {
    (void)block_inclusive_scan(tiles_before, s_wave_tiles, base);
    if (blockIdx.x == gridDim.x - 1) {
      if (threadIdx.x == 0) {
        num_unique[0] = static_cast<int32_t>(base + total);
        segment_starts[base + total] = static_cast<int32_t>(n);
      }
      if (clear_queue_counters) {
        for (int i = threadIdx.x; i < kNumCounters; i += kBlockThreads)
          if (i >= 1) num_unique[i] = 0;
      }
    }
  } else {
    base = tile_base[blockIdx.x];
  }
  uint32_t local = incl - mine;
  int32_t ids[kSegItems];
#pragma unroll
  for (int k = 0; k < kSegItems; ++k) {
    if (flags & (1u << k)) s_heads[local++] = static_cast<int32_t>(first + k);
    // `local` now counts the tile's heads at or before this position: its segment is base + local - 1
    ids[k] = static_cast<int32_t>(base + local) - 1;
  }
  if (segment_ids) {
    if (first + kSegItems <= n) {
      *reinterpret_cast<int4 *>(segment_ids + first) = make_int4(ids[0], ids[1], ids[2], ids[3]);
      *reinterpret_cast<int4 *>(segment_ids + first + 4) = make_int4(ids[4], ids[5], ids[6], ids[7]);
    } else {
#pragma unroll
      for (int k = 0; k < kSegItems; ++k)
        if (first + k < n) segment_ids[first + k] = ids[k];
    }
  }
  __syncthreads();
  for (uint32_t i = threadIdx.x; i < total; i += kBlockThreads) segment_starts[base + i] = s_heads[i];
}

inline int num_seg_tiles(int64_t n) { return static_cast<int>(ceil_div(n, kSegTile)); }

}  // namespace

// Sort workspace: [tmp keys n][tmp values n][counts 1024 * max_tiles][workgroup sums of the count
// scan][table_starts T+1][tile_prefix T+2][digit totals 4 * 1024 * T][group totals 4 * 1024 *
// groups]; max_tiles = ceil(n / tile) + T, groups = ceil(max_tiles / kGroupTiles).
namespace {
struct SortScratch {
  uint64_t tmp_keys, tmp_vals, counts, block_sums, table_starts, tile_prefix, totals, total;
  int max_tiles;
  int scan_blocks;  // for the widest digit
  int64_t groups;   // groups of kGroupTiles tiles that the region behind the digit totals has room for
};

constexpr int kMaxPasses = 4;  // 32 key bits in digits of at least 8

// The per-table layout of the counts (no scan between the histogram and the scatter kernel) is
// used when the tables have few tiles each on average: the batch's lookups are spread over many
// tables.
inline bool use_table_scan(int64_t n, int32_t num_tables, bool have_tables) {
  return have_tables && num_tables >= 8 &&
         ceil_div(n, kBlockThreads * sort_items(n)) <= static_cast<int64_t>(num_tables) * 128 * (kItems / sort_items(n));
}

SortScratch sort_scratch(int64_t n, int32_t num_tables) {
  SortScratch s;
  const uint64_t nn = static_cast<uint64_t>(n > 0 ? n : 1);
  const uint64_t tables = static_cast<uint64_t>(num_tables > 0 ? num_tables : 1);
  s.max_tiles = static_cast<int>(ceil_div(nn, kBlockThreads * sort_items(n)) + tables);
  // The counters are sized so that a workspace for n pairs also serves every smaller n: just above
  // kSmallSortPairs the full-size tiles are fewer than the quarter-size tiles of kSmallSortPairs.
  uint64_t sized_tiles = static_cast<uint64_t>(s.max_tiles);
  if (n > kSmallSortPairs)
    sized_tiles = std::max<uint64_t>(sized_tiles, ceil_div(kSmallSortPairs, kBlockThreads * kSmallItems) + tables);
  s.scan_blocks = static_cast<int>(ceil_div(sized_tiles * kMaxBins, kScanChunk));
  uint64_t off = 0;
  s.tmp_keys = off; off += align_up(nn * 4, 256);
  s.tmp_vals = off; off += align_up(nn * 4, 256);
  s.counts = off; off += align_up(sized_tiles * kMaxBins * 4, 256);
  s.block_sums = off; off += align_up(static_cast<uint64_t>(s.scan_blocks) * 4, 256);
  s.table_starts = off; off += align_up((tables + 1) * 4, 256);
  s.tile_prefix = off; off += align_up((tables + 2) * 4, 256);
  // (sized for every table count, so that the layout does not depend on the path taken; the group
  // totals follow the digit totals at once, so that one clearing loop covers both)
  s.groups = static_cast<int64_t>(ceil_div(sized_tiles, kGroupTiles));
  s.totals = off;
  off += align_up((tables + static_cast<uint64_t>(s.groups)) * kMaxBins * kMaxPasses * 4, 256);
  s.total = off;
  return s;
}

struct RadixPass {
  const uint32_t *src_k, *src_v;
  uint32_t *dst_k, *dst_v;
  const uint32_t *table_starts, *tile_prefix;
  int num_tables, max_tiles, shift;
  uint32_t mask;
  uint32_t *counts, *block_sums;
  uint32_t *totals;        // this pass's per-table digit totals, zeroed; null: linear scan
  uint32_t *group_totals;  // this pass's digit totals of every kGroupTiles tiles, zeroed
  const int32_t *key_bias;
  uint32_t key_mul;
};

template <int BITS, int ITEMS>
void launch_radix_pass(const RadixPass &p, hipStream_t stream) {
  const dim3 block(kBlockThreads);
  const dim3 tiles(static_cast<unsigned>(ceil_div(p.max_tiles, kNumXcd) * kNumXcd));  // (whole turns of the XCDs)
  if (p.totals) {
    TBE_LAUNCH("radix_histogram", stream, (radix_histogram_kernel<BITS, true, ITEMS>), tiles, block, p.src_k,
               p.table_starts, p.tile_prefix, p.num_tables, p.max_tiles, p.shift, p.mask, p.counts, p.totals,
               p.group_totals);
    TBE_LAUNCH("radix_scatter", stream, (radix_scatter_kernel<BITS, true, ITEMS>), tiles, block, p.src_k, p.src_v,
               p.dst_k, p.dst_v, p.table_starts, p.tile_prefix, p.num_tables, p.max_tiles, p.shift, p.mask,
               p.counts, p.totals, p.group_totals, p.key_bias, p.key_mul);
    return;
  }
  const dim3 scan_blocks(static_cast<unsigned>(ceil_div(static_cast<int64_t>(p.max_tiles) << BITS, kScanChunk)));
  TBE_LAUNCH("radix_histogram", stream, (radix_histogram_kernel<BITS, false, ITEMS>), tiles, block, p.src_k,
             p.table_starts, p.tile_prefix, p.num_tables, p.max_tiles, p.shift, p.mask, p.counts, nullptr, nullptr);
  TBE_LAUNCH("radix_scan_reduce", stream, radix_scan_reduce_kernel, scan_blocks, block, p.counts,
             p.tile_prefix, p.num_tables, BITS, p.block_sums);
  TBE_LAUNCH("radix_scan", stream, radix_scan_kernel, scan_blocks, block, p.counts, p.tile_prefix,
             p.num_tables, BITS, p.block_sums);
  TBE_LAUNCH("radix_scatter", stream, (radix_scatter_kernel<BITS, false, ITEMS>), tiles, block, p.src_k, p.src_v,
             p.dst_k, p.dst_v, p.table_starts, p.tile_prefix, p.num_tables, p.max_tiles, p.shift, p.mask,
             p.counts, nullptr, nullptr, p.key_bias, p.key_mul);
}
}  // namespace

uint64_t sort_workspace_bytes(int64_t n, int32_t num_tables) { return sort_scratch(n, num_tables).total; }

int sort_pairs(const int32_t *keys_in, const int32_t *values_in, int32_t *keys_out,
               int32_t *values_out, int64_t n, int32_t end_bit, void *workspace,
               hipStream_t stream, const SortTables *tables, const int32_t *device_count) {
  if (n == 0) return TBE_OK;
  // Fewest passes with digits of at most 10 bits, the bits spread evenly over the passes
  // (23 bits -> 8+8+7, 25 -> 9+8+8, 27 -> 9+9+9, 17 -> 9+8).
  const int passes = end_bit <= 0 ? 1 : static_cast<int>(ceil_div(end_bit, kMaxRadixBits));
  const int num_tables = tables ? tables->num_tables : 1;
  const SortScratch scratch = sort_scratch(n, num_tables);
  char *ws = static_cast<char *>(workspace);
  uint32_t *tmp_keys = reinterpret_cast<uint32_t *>(ws + scratch.tmp_keys);
  uint32_t *tmp_vals = reinterpret_cast<uint32_t *>(ws + scratch.tmp_vals);

  RadixPass p;
  const int items = sort_items(n);
  p.table_starts = reinterpret_cast<uint32_t *>(ws + scratch.table_starts);
  p.tile_prefix = reinterpret_cast<uint32_t *>(ws + scratch.tile_prefix);
  p.num_tables = num_tables;
  p.max_tiles = scratch.max_tiles;
  p.counts = reinterpret_cast<uint32_t *>(ws + scratch.counts);
  p.block_sums = reinterpret_cast<uint32_t *>(ws + scratch.block_sums);
  const bool table_scan = use_table_scan(n, num_tables, tables != nullptr) && passes <= kMaxPasses;
  uint32_t *totals = reinterpret_cast<uint32_t *>(ws + scratch.totals);
  // per pass: T rows of digit totals; behind those of all passes, per pass, a row per group of tiles
  const int64_t groups = ceil_div(scratch.max_tiles, kGroupTiles);
  const int64_t totals_words = table_scan ? (num_tables + groups) * kMaxBins * passes : 0;
  uint32_t *group_totals = totals + static_cast<int64_t>(num_tables) * kMaxBins * passes;
  const unsigned setup_blocks = static_cast<unsigned>(1 + std::min<int64_t>(ceil_div(totals_words, kBlockThreads * 4), 255));
  int32_t *grad_rows = tables ? tables->grad_rows : nullptr;
  const unsigned row_blocks =
      grad_rows ? static_cast<unsigned>(ceil_div(static_cast<int64_t>(num_tables) * tables->bags_per_table * kLinLanes,
                                                 kBlockThreads))
                : 0u;
#define TBE_SORT_SETUP(ITEMS)                                                                          \
  TBE_LAUNCH("sort_setup", stream, sort_setup_kernel<ITEMS>, dim3(setup_blocks + row_blocks),          \
             dim3(kBlockThreads), tables ? tables->offsets : nullptr,                                  \
             tables ? tables->bags_per_table : 0, num_tables, static_cast<uint32_t>(n),                \
             const_cast<uint32_t *>(p.table_starts), const_cast<uint32_t *>(p.tile_prefix), totals,    \
             totals_words, device_count, static_cast<int>(setup_blocks), grad_rows)
  if (items == kSmallItems) { TBE_SORT_SETUP(kSmallItems); }
  else { TBE_SORT_SETUP(kItems); }
#undef TBE_SORT_SETUP

  p.src_k = reinterpret_cast<const uint32_t *>(keys_in);
  p.src_v = reinterpret_cast<const uint32_t *>(values_in);
  p.shift = 0;
  for (int pass = 0; pass < passes; ++pass) {
    const int remaining = end_bit <= 0 ? 0 : end_bit - p.shift;
    const int bits = static_cast<int>(ceil_div(remaining, passes - pass));
    p.mask = (1u << bits) - 1u;
    const bool to_out = ((passes - 1 - pass) % 2) == 0;
    p.dst_k = to_out ? reinterpret_cast<uint32_t *>(keys_out) : tmp_keys;
    p.dst_v = to_out ? reinterpret_cast<uint32_t *>(values_out) : tmp_vals;
    p.key_bias = (tables && pass == passes - 1) ? tables->key_bias : nullptr;
    p.key_mul = tables ? static_cast<uint32_t>(tables->key_mul) : 1u;
    p.totals = table_scan ? totals + static_cast<int64_t>(pass) * num_tables * kMaxBins : nullptr;
    p.group_totals = table_scan ? group_totals + static_cast<int64_t>(pass) * groups * kMaxBins : nullptr;
    if (items == kSmallItems) {
      if (bits <= 8) launch_radix_pass<8, kSmallItems>(p, stream);
      else if (bits == 9) launch_radix_pass<9, kSmallItems>(p, stream);
      else launch_radix_pass<10, kSmallItems>(p, stream);
    } else {
      if (bits <= 8) launch_radix_pass<8, kItems>(p, stream);
      else if (bits == 9) launch_radix_pass<9, kItems>(p, stream);
      else launch_radix_pass<10, kItems>(p, stream);
    }
    p.src_k = p.dst_k;
    p.src_v = p.dst_v;
    p.shift += bits;
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
  // Up to a few thousand tiles, every workgroup of the last kernel sums the counts before its
  // own (a few KB from L2 each); beyond that a kernel of one workgroup scans them first.
  constexpr int kMaxSummedTiles = 4096;
  if (tiles > 0 && tiles <= kMaxSummedTiles) {
    TBE_LAUNCH("segment_write", stream, segment_write_kernel<true>, dim3(tiles), block, keys, n,
               tile_heads, segment_starts, segment_ids, num_unique, clear_queue_counters ? 1 : 0);
    return check_launch("tbe_find_segments");
  }
  TBE_LAUNCH("segment_scan", stream, segment_scan_kernel, dim3(1), block, tile_heads, tiles, n,
             segment_starts, num_unique, clear_queue_counters ? 1 : 0);
  if (tiles > 0)
    TBE_LAUNCH("segment_write", stream, segment_write_kernel<false>, dim3(tiles), block, keys, n,
               tile_heads, segment_starts, segment_ids, num_unique, 0);
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

int interleaved_to_table_major(const int32_t *indices, const int32_t *offsets, int32_t offsets_stride,
                               int32_t T, int32_t B, int32_t *totals, int32_t *bias, int32_t *chunk_sums,
                               int32_t *offsets_tm, int32_t *indices_tm, hipStream_t stream) {
  const int64_t num_bags = static_cast<int64_t>(T) * B;
  const int chunks = static_cast<int>(interleaved_chunks_per_table(B));
  const dim3 block(kBlockThreads);
  const dim3 per_chunk(static_cast<unsigned>(static_cast<int64_t>(T) * chunks));
  TBE_LAUNCH("interleaved_offsets", stream, interleaved_chunk_sums_kernel, per_chunk, block, offsets, offsets_stride,
             B, chunks, chunk_sums);
  TBE_LAUNCH("interleaved_offsets", stream, interleaved_totals_kernel, dim3(static_cast<unsigned>(T)), block,
             chunk_sums, chunks, totals, bias);
  TBE_LAUNCH("interleaved_offsets", stream, interleaved_offsets_kernel, per_chunk, block, offsets, offsets_stride, B,
             T, chunks, totals, chunk_sums, offsets_tm);
  TBE_LAUNCH("interleaved_permute", stream, interleaved_permute_kernel,
             dim3(static_cast<unsigned>(ceil_div(num_bags * kLinLanes, kBlockThreads))), block, indices, offsets,
             offsets_stride, B, T, static_cast<int>(num_bags), offsets_tm, indices_tm);
  return check_launch("tbe_backward_sgd_interleaved");
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

extern "C" uint64_t tbe_sort_workspace_bytes(int64_t n) { return tbe::sort_workspace_bytes(n, 1); }

extern "C" int tbe_sort_pairs(const int32_t *keys_in, const int32_t *values_in, int32_t *keys_out,
                              int32_t *values_out, int64_t n, int32_t end_bit, void *workspace,
                              uint64_t workspace_bytes, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(n >= 0 && n < INT32_MAX, "tbe_sort_pairs: n out of range");
  TBE_REQUIRE(end_bit >= 0 && end_bit <= 32, "tbe_sort_pairs: end_bit must be in [0, 32] (got %d)", end_bit);
  if (n == 0) return TBE_OK;
  TBE_REQUIRE(keys_in && keys_out && values_out, "tbe_sort_pairs: null pointer argument");
  if (!workspace || workspace_bytes < sort_workspace_bytes(n, 1))
    return fail(TBE_ERR_WORKSPACE, "tbe_sort_pairs: workspace of %llu bytes needed, %llu given",
                (unsigned long long)sort_workspace_bytes(n, 1), (unsigned long long)workspace_bytes);
  return sort_pairs(keys_in, values_in, keys_out, values_out, n, end_bit, workspace,
                    static_cast<hipStream_t>(stream), nullptr);
}

extern "C" uint64_t tbe_segments_workspace_bytes(int64_t n) { return tbe::segments_workspace_bytes(n); }

extern "C" int tbe_find_segments(const int32_t *keys_sorted, int64_t n, int32_t *segment_starts,
                                 int32_t *num_unique, void *workspace, uint64_t workspace_bytes,
                                 void *stream) {
  using namespace tbe;
  TBE_REQUIRE(n >= 0 && n < INT32_MAX, "tbe_find_segments: n out of range");
  TBE_REQUIRE(segment_starts && num_unique, "tbe_find_segments: null pointer argument");
  TBE_REQUIRE(keys_sorted || n == 0, "tbe_find_segments: null keys");
  TBE_REQUIRE(reinterpret_cast<uintptr_t>(keys_sorted) % 16 == 0, "tbe_find_segments: keys_sorted must be 16-byte aligned");
  if (!workspace || workspace_bytes < segments_workspace_bytes(n))
    return fail(TBE_ERR_WORKSPACE, "tbe_find_segments: workspace of %llu bytes needed, %llu given",
                (unsigned long long)segments_workspace_bytes(n), (unsigned long long)workspace_bytes);
  return find_segments(keys_sorted, n, segment_starts, num_unique, nullptr, workspace,
                       static_cast<hipStream_t>(stream), /*clear_queue_counters=*/false);
}
