// HBM-resident set-associative row cache in front of a host-resident table, for gfx950.
//
// 64 ways per set = one wavefront probes a set with one coalesced 256-byte tag load and a
// ballot.  The reference has no cache; the specification is the comment above tbe_cache_t in
// include/tbe_hip.h.  Per step:
//   lookup   one wavefront per unique row: ballot match -> slot, mark used; misses count per set
//   scan     exclusive scan of the per-set miss counts
//   group    misses written into their set's range of miss_list (integer atomics; order inside
//            a range is irrelevant because the inserting wavefront picks the smallest row first)
//   insert   one wavefront per set: for each missing row in ascending order, victim = lowest
//            (priority, way) among slots not used in this step (wavefront min + ballot)
//   fill     (side stream) write back the evicted row, fetch the new row over the host link
//            (deferred write-back, cache->stage_of_row: or from the staging row that has held it
//            since the step before; beside it, in the same launch, the rows staged by the step
//            before that this step does not fetch go back to the backing table)
//   locate   slot of every lookup position, for the forward gather
// Every decision is a function of integers only, so the tags after a step are reproducible.

#include <algorithm>

#include "tbe_stages.h"

namespace tbe {
namespace {

constexpr int kWays = TBE_CACHE_WAYS;
static_assert(kWays == kWave, "one lane per way");
constexpr int kSetScanItems = 16;

// lowbias32 integer hash, then a multiplicative range reduction to [0, num_sets).
__device__ __forceinline__ uint32_t cache_set_of(uint32_t key, uint32_t num_sets) {
  uint32_t h = key;
  h ^= h >> 16;
  h *= 0x7feb352du;
  h ^= h >> 15;
  h *= 0x846ca68bu;
  h ^= h >> 16;
  return static_cast<uint32_t>((static_cast<uint64_t>(h) * num_sets) >> 32);
}

enum { kStatUnique = 0, kStatHits, kStatMisses, kStatInserted, kStatWrittenBack, kStatUncached, kStatStaged,
       kStatFromStaging };

__global__ __launch_bounds__(kBlockThreads) void cache_fill_i32_kernel(int32_t *p, int64_t n, int32_t v) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    p[i] = v;
}

__global__ __launch_bounds__(kBlockThreads) void cache_lookup_kernel(
    const int32_t *__restrict__ tags, int32_t *__restrict__ last_used,
    int32_t *__restrict__ use_count, uint32_t num_sets, int32_t step,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, int32_t *__restrict__ unique_slots,
    int32_t *__restrict__ evicted_keys, int32_t *__restrict__ miss_sets,
    int32_t *__restrict__ set_counts, int32_t *__restrict__ stats) {
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  int hits = 0, misses = 0;
  // A wavefront takes 64 unique rows at a time: every lane fetches the key of one of them, then
  // the sets are probed eight at a time (the whole wavefront reads a set's 64 tags with one
  // load), so that eight tag loads are in flight instead of one; lane j keeps the outcome of
  // row j and writes it at the end.
  constexpr int kProbe = 8;
  for (int64_t u0 = wave_id * kWave; u0 < U; u0 += stride * kWave) {
    const int rows = static_cast<int>(min(static_cast<int64_t>(kWave), U - u0));
    const int64_t my_u = u0 + min(lane, rows - 1);
    const int32_t my_key = keys_sorted[segment_starts[my_u]];
    const uint32_t my_set = cache_set_of(static_cast<uint32_t>(my_key), num_sets);
    int my_way = -1;
    for (int j0 = 0; j0 < rows; j0 += kProbe) {
      int32_t tag[kProbe];
#pragma unroll
      for (int q = 0; q < kProbe; ++q) {
        const uint32_t set = static_cast<uint32_t>(__shfl(static_cast<int>(my_set), min(j0 + q, rows - 1), kWave));
        tag[q] = tags[static_cast<int64_t>(set) * kWays + lane];
      }
#pragma unroll
      for (int q = 0; q < kProbe; ++q) {
        const int32_t key = __shfl(my_key, min(j0 + q, rows - 1), kWave);
        const unsigned long long match = __ballot(tag[q] == key);
        if (lane == j0 + q && match) my_way = __ffsll(static_cast<long long>(match)) - 1;
      }
    }
    if (lane < rows) {
      const int64_t u = u0 + lane;
      if (my_way >= 0) {
        const int64_t slot = static_cast<int64_t>(my_set) * kWays + my_way;
        unique_slots[u] = static_cast<int32_t>(slot);
        evicted_keys[u] = -2;
        miss_sets[u] = static_cast<int32_t>(num_sets);  // sorts behind every set
        last_used[slot] = step;
        const int32_t c = use_count[slot];
        use_count[slot] = c == INT32_MAX ? c : c + 1;
      } else {
        unique_slots[u] = -1;
        evicted_keys[u] = -2;
        miss_sets[u] = static_cast<int32_t>(my_set);
        atomicAdd(&set_counts[my_set], 1);
      }
    }
    const int hit_rows = static_cast<int>(__popcll(__ballot(lane < rows && my_way >= 0)));
    hits += hit_rows;
    misses += rows - hit_rows;
  }
  if (lane == 0) {
    if (hits) atomicAdd(&stats[kStatHits], hits);
    if (misses) atomicAdd(&stats[kStatMisses], misses);
    if (wave_id == 0) stats[kStatUnique] = U;
  }
}

// Single workgroup: set_starts = exclusive scan of set_counts, set_starts[num_sets] = total.
__global__ __launch_bounds__(kBlockThreads) void cache_scan_sets_kernel(
    const int32_t *__restrict__ set_counts, int64_t num_sets, int32_t *__restrict__ set_starts) {
  __shared__ uint32_t s_wave[kWavesPerBlock];
  const int tid = threadIdx.x;
  const int lane = tid & (kWave - 1);
  const int wave = tid >> 6;
  uint32_t carry = 0;
  for (int64_t base = 0; base < num_sets; base += kBlockThreads * kSetScanItems) {
    const int64_t first = base + static_cast<int64_t>(tid) * kSetScanItems;
    uint32_t local[kSetScanItems];
    uint32_t sum = 0;
#pragma unroll
    for (int k = 0; k < kSetScanItems; ++k) {
      local[k] = first + k < num_sets ? static_cast<uint32_t>(set_counts[first + k]) : 0u;
      sum += local[k];
    }
    uint32_t x = sum;
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
      const uint32_t y = __shfl_up(x, d, kWave);
      if (lane >= d) x += y;
    }
    if (lane == kWave - 1) s_wave[wave] = x;
    __syncthreads();
    uint32_t before = 0, total = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) {
      const uint32_t v = s_wave[w];
      if (w < wave) before += v;
      total += v;
    }
    uint32_t running = carry + before + x - sum;
#pragma unroll
    for (int k = 0; k < kSetScanItems; ++k) {
      if (first + k < num_sets) set_starts[first + k] = static_cast<int32_t>(running);
      running += local[k];
    }
    carry += total;
    __syncthreads();
  }
  if (tid == 0) set_starts[num_sets] = static_cast<int32_t>(carry);
}

__global__ __launch_bounds__(kBlockThreads) void cache_insert_kernel(
    int32_t *__restrict__ tags, int32_t *__restrict__ last_used, int32_t *__restrict__ use_count,
    int64_t num_sets, int32_t policy, int32_t step, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ set_starts,
    const int32_t *__restrict__ miss_list, int32_t *__restrict__ unique_slots,
    int32_t *__restrict__ evicted_keys, int32_t *__restrict__ stats, int64_t stage_slots,
    int64_t stage_base) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  int inserted = 0, written_back = 0, uncached = 0, staged = 0;
  for (int64_t set = wave_id; set < num_sets; set += stride) {
    const int begin = set_starts[set];
    const int end = set_starts[set + 1];
    if (begin == end) continue;
    const int64_t slot = set * kWays + lane;
    int32_t tag = tags[slot];
    int32_t used = last_used[slot];
    int32_t count = use_count[slot];
    // The set's missing rows, miss_list[begin, end), are in ascending order of their index u.  A
    // way can take a row while it has not served this step; every insertion uses one up, so the
    // first `takers` rows are inserted, one after the other (each picks its victim), and all the
    // others are staged or left in the backing table, which needs no order: lanes do them side
    // by side.  The work per set is bounded by 64 insertions plus a pass over its list.
    const int takers = min(static_cast<int>(__popcll(__ballot(used < step))), end - begin);
    for (int j0 = 0; j0 < takers; j0 += kWave) {
      const int32_t my_u = miss_list[begin + min(j0 + lane, takers - 1)];
      const int32_t my_key = keys_sorted[segment_starts[my_u]];
      const int batch = min(kWave, takers - j0);
      for (int j = 0; j < batch; ++j) {
        const int32_t u = __shfl(my_u, j, kWave);
        const int32_t key = __shfl(my_key, j, kWave);
        // victim: lowest (priority, way) among slots not used in this step
        const uint32_t priority = used < step ? static_cast<uint32_t>(policy == TBE_CACHE_LFU ? count : used)
                                              : 0xffffffffu;
        uint32_t best = priority;
#pragma unroll
        for (int m = kWave / 2; m > 0; m >>= 1) best = min(best, static_cast<uint32_t>(__shfl_xor(static_cast<int>(best), m, kWave)));
        const int way = __ffsll(static_cast<long long>(__ballot(priority == best))) - 1;
        const int32_t old_tag = __shfl(tag, way, kWave);
        if (lane == way) {
          tag = key;
          used = step;
          count = 1;
        }
        if (lane == 0) {
          unique_slots[u] = static_cast<int32_t>(set * kWays + way);
          evicted_keys[u] = old_tag >= 0 ? old_tag : -1;
        }
        ++inserted;
        if (old_tag >= 0) ++written_back;
      }
    }
    // Every way serves this step now.  The other rows get a staging row for the step (index:
    // misses of the sets before this one + rank among the set's staged rows), or, when the
    // staging area is exhausted, stay in the backing table.
    for (int j0 = begin + takers; j0 < end; j0 += kWave) {
      const int j = j0 + lane;
      const int64_t stage = static_cast<int64_t>(j) - takers;
      const bool here = j < end;
      const bool fits = here && stage < stage_slots;
      if (fits) {
        const int32_t u = miss_list[j];
        unique_slots[u] = static_cast<int32_t>(stage_base + stage);
        evicted_keys[u] = -1;
      }
      staged += static_cast<int>(__popcll(__ballot(fits)));
      uncached += static_cast<int>(__popcll(__ballot(here && !fits)));
    }
    tags[slot] = tag;
    last_used[slot] = used;
    use_count[slot] = count;
  }
  if (lane == 0) {
    if (inserted) atomicAdd(&stats[kStatInserted], inserted);
    if (written_back) atomicAdd(&stats[kStatWrittenBack], written_back);
    if (uncached) atomicAdd(&stats[kStatUncached], uncached);
    if (staged) atomicAdd(&stats[kStatStaged], staged);
  }
}

// Deferred write-back, after the step's slots are decided: where each row that this step fetches
// comes from, and where the rows that it stages are.  A fetched row that the step before staged
// is still in that step's staging row: fetch_source[u] = that row of `rows` (else -1: the backing
// table), and the entry of the staging row is marked consumed (-(key + 2)) so that it is not
// written back.  A row staged now is entered into stage_of_row / stage_keys.
__global__ __launch_bounds__(kBlockThreads) void cache_resolve_kernel(
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    const int32_t *__restrict__ evicted_keys, int32_t *__restrict__ stage_of_row,
    int32_t *__restrict__ stage_keys, int32_t *__restrict__ fetch_source, int64_t num_slots,
    int32_t *__restrict__ stats) {
  const int U = counters[0];
  int from_staging = 0;
  for (int64_t u = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; u < U;
       u += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    if (evicted_keys[u] == -2) continue;  // a hit, or a row left in the backing table
    const int32_t key = keys_sorted[segment_starts[u]];
    const int32_t slot = unique_slots[u];
    const int32_t held = stage_of_row[key];
    fetch_source[u] = held;
    if (held >= 0) {
      stage_keys[held - num_slots] = -(key + 2);
      ++from_staging;
    }
    if (slot >= num_slots) {
      stage_of_row[key] = slot;
      stage_keys[slot - num_slots] = key;
    } else if (held >= 0) {
      stage_of_row[key] = -1;  // the row lives in a slot of the cache now
    }
  }
  for (int m = kWave / 2; m > 0; m >>= 1) from_staging += __shfl_xor(from_staging, m, kWave);
  if ((threadIdx.x & (kWave - 1)) == 0 && from_staging) atomicAdd(&stats[kStatFromStaging], from_staging);
}

// One wavefront per row; rows move as 8-byte units (row_units = D * element size / 8).
// fetch_source (deferred write-back): per unique row, the row of `rows` to fetch it from, or -1.
// old_stage_keys (deferred write-back): the launch also carries the write-back of the step
// before -- the rows of that step's staging area whose entry holds a key (not consumed, not
// empty) go to the backing table.  Every wavefront alternates between an entry of that area
// and a unique row of this step, so that both directions of the host link are busy at once on
// every compute unit and neither side finishes long before the other, whatever their sizes.
// (Measured on the 35.6 GB configuration: 57 ms per launch against 65 ms when workgroups
// with an odd index wrote back and the others fetched.)
__global__ __launch_bounds__(kBlockThreads) void cache_fill_kernel(
    uint64_t *__restrict__ cache_rows, uint64_t *__restrict__ backing_rows, int row_units,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    const int32_t *__restrict__ evicted_keys, const int32_t *__restrict__ fetch_source,
    const int32_t *__restrict__ old_stage_keys, int64_t old_stage_base, int64_t stage_slots) {
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  const int64_t pending = old_stage_keys ? stage_slots : 0;
  const int64_t items = U > pending ? U : pending;
  for (int64_t i = wave_id; i < items; i += stride) {
    if (i < pending) {
      const int64_t key = old_stage_keys[i];
      if (key >= 0) {
        const uint64_t *src = cache_rows + (old_stage_base + i) * row_units;
        uint64_t *dst = backing_rows + key * row_units;
        for (int k = lane; k < row_units; k += kWave) dst[k] = src[k];
      }
    }
    if (i >= U) continue;
    const int32_t evicted = evicted_keys[i];
    if (evicted == -2) continue;
    const int64_t key = keys_sorted[segment_starts[i]];
    uint64_t *slot_row = cache_rows + static_cast<int64_t>(unique_slots[i]) * row_units;
    const uint64_t *new_row = backing_rows + key * row_units;
    if (fetch_source) {
      const int64_t held = fetch_source[i];
      if (held >= 0) new_row = cache_rows + held * row_units;
    }
    if (evicted >= 0) {
      uint64_t *old_row = backing_rows + static_cast<int64_t>(evicted) * row_units;
      for (int k = lane; k < row_units; k += kWave) old_row[k] = slot_row[k];
    }
    for (int k = lane; k < row_units; k += kWave) slot_row[k] = new_row[k];
  }
}

// Deferred write-back, outside a step (flush, or the check that the area a step stages into is
// empty): the rows of a staging area that hold a key go to the backing table.  A wavefront reads
// 64 entries at a time and copies the rows of those that hold one, so an empty area costs one
// pass over its entries.
__global__ __launch_bounds__(kBlockThreads) void cache_unstage_area_kernel(
    const uint64_t *__restrict__ cache_rows, uint64_t *__restrict__ backing_rows, int row_units,
    const int32_t *__restrict__ stage_keys, int64_t stage_base, int64_t stage_slots) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t i0 = wave_id * kWave; i0 < stage_slots; i0 += stride * kWave) {
    const int32_t my_key = i0 + lane < stage_slots ? stage_keys[i0 + lane] : -1;
    unsigned long long held = __ballot(my_key >= 0);
    while (held) {
      const int j = __ffsll(static_cast<long long>(held)) - 1;
      held &= held - 1;
      const int64_t key = __shfl(my_key, j, kWave);
      const uint64_t *src = cache_rows + (stage_base + i0 + j) * row_units;
      uint64_t *dst = backing_rows + key * row_units;
      for (int k = lane; k < row_units; k += kWave) dst[k] = src[k];
    }
  }
}

// Deferred write-back: the staging area of the step before is released -- its entries are
// emptied, and stage_of_row forgets the rows it held unless they have been staged again since.
__global__ __launch_bounds__(kBlockThreads) void cache_retire_stage_kernel(
    int32_t *__restrict__ stage_of_row, int32_t *__restrict__ old_stage_keys, int64_t old_stage_base,
    int64_t stage_slots) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < stage_slots;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int32_t entry = old_stage_keys[i];
    if (entry == -1) continue;
    const int32_t key = entry >= 0 ? entry : -(entry + 2);
    if (stage_of_row[key] == old_stage_base + i) stage_of_row[key] = -1;
    old_stage_keys[i] = -1;
  }
}

// After the update: staged rows (slot >= first_stage_slot) go back to the backing table.
__global__ __launch_bounds__(kBlockThreads) void cache_unstage_kernel(
    const uint64_t *__restrict__ cache_rows, uint64_t *__restrict__ backing_rows, int row_units,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    int64_t first_stage_slot) {
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t u = wave_id; u < U; u += stride) {
    const int64_t slot = unique_slots[u];
    if (slot < first_stage_slot) continue;
    const int64_t key = keys_sorted[segment_starts[u]];
    const uint64_t *src = cache_rows + slot * row_units;
    uint64_t *dst = backing_rows + key * row_units;
    for (int i = lane; i < row_units; i += kWave) dst[i] = src[i];
  }
}

__global__ __launch_bounds__(kBlockThreads) void cache_locate_kernel(
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ segment_ids,
    const int32_t *__restrict__ unique_slots, int64_t n, int32_t *__restrict__ lookup_slots) {
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x)
    lookup_slots[positions_sorted[i]] = unique_slots[segment_ids[i]];
}

__global__ __launch_bounds__(kBlockThreads) void cache_flush_kernel(
    const int32_t *__restrict__ tags, const uint64_t *__restrict__ cache_rows,
    uint64_t *__restrict__ backing_rows, int row_units, int64_t num_slots) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t slot = wave_id; slot < num_slots; slot += stride) {
    const int64_t key = tags[slot];
    if (key < 0) continue;
    const uint64_t *src = cache_rows + slot * row_units;
    uint64_t *dst = backing_rows + key * row_units;
    for (int i = lane; i < row_units; i += kWave) dst[i] = src[i];
  }
}

void cache_layout(int64_t n, int64_t num_sets, tbe_cache_workspace_layout_t *l) {
  const uint64_t nn = static_cast<uint64_t>(n > 0 ? n : 1);
  const uint64_t ints = align_up(nn * 4, 256);
  const uint64_t sets = align_up(static_cast<uint64_t>(num_sets + 1) * 4, 256);
  uint64_t off = 0;
  l->unique_slots = off; off += ints;
  l->lookup_slots = off; off += ints;
  l->evicted_keys = off; off += ints;
  l->miss_sets = off; off += ints;
  l->miss_list = off; off += ints;
  l->set_counts = off; off += sets;
  l->set_fill = off; off += sets;
  l->set_starts = off; off += sets;
  l->stats = off; off += 256;
  l->fetch_source = off; off += ints;
  l->total_bytes = off;
}

inline unsigned grid_for(int64_t work_items, int64_t per_block, int64_t cap) {
  return static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(ceil_div(work_items, per_block), cap)));
}

int validate_cache(const char *name, const tbe_cache_t *cache) {
  TBE_REQUIRE(cache, "%s: null cache", name);
  TBE_REQUIRE(cache->tags && cache->last_used && cache->use_count && cache->rows && cache->backing_rows,
              "%s: cache has a null array", name);
  TBE_REQUIRE(cache->num_sets > 0 && cache->num_sets * kWays < INT32_MAX, "%s: num_sets out of range", name);
  TBE_REQUIRE(cache->stage_slots >= 0 && cache->num_sets * kWays + cache->stage_slots < INT32_MAX,
              "%s: stage_slots out of range", name);
  TBE_REQUIRE(cache->policy == TBE_CACHE_LRU || cache->policy == TBE_CACHE_LFU, "%s: bad policy %d", name,
              cache->policy);
  if (cache->stage_of_row) {
    TBE_REQUIRE(cache->stage_keys && cache->total_rows > 0 && cache->total_rows < INT32_MAX,
                "%s: deferred write-back needs stage_keys and total_rows", name);
    TBE_REQUIRE(cache->num_sets * kWays + 2 * cache->stage_slots < INT32_MAX, "%s: stage_slots out of range", name);
  }
  return TBE_OK;
}

// Deferred write-back: the rows of the staging area at `stage_base` that still wait for their
// write-back go to the backing table, and the area is released.
void write_back_stage(const tbe_cache_t *cache, int row_units, int64_t half, hipStream_t stream) {
  const int64_t base = cache->num_sets * kWays + half * cache->stage_slots;
  int32_t *keys = cache->stage_keys + half * cache->stage_slots;
  TBE_LAUNCH("cache_unstage", stream, cache_unstage_area_kernel,
             dim3(grid_for(cache->stage_slots, kWavesPerBlock, 256 * 16)), dim3(kBlockThreads),
             static_cast<const uint64_t *>(cache->rows), static_cast<uint64_t *>(cache->backing_rows), row_units, keys,
             base, cache->stage_slots);
  TBE_LAUNCH("cache_retire_stage", stream, cache_retire_stage_kernel,
             dim3(grid_for(cache->stage_slots, kBlockThreads, 1024)), dim3(kBlockThreads), cache->stage_of_row, keys,
             base, cache->stage_slots);
}

// One event per calling thread, used to order the two streams.
hipEvent_t join_event(int which) {
  thread_local hipEvent_t events[2] = {nullptr, nullptr};
  if (!events[which]) {
    if (hipEventCreateWithFlags(&events[which], hipEventDisableTiming) != hipSuccess) return nullptr;
  }
  return events[which];
}

}  // namespace

int cache_unstage(const tbe_cache_t *cache, int32_t dtype, int32_t D, const int32_t *keys_sorted,
                  const int32_t *segment_starts, const int32_t *counters,
                  const int32_t *unique_slots, int64_t num_indices, hipStream_t stream) {
  if (cache->stage_slots <= 0 || num_indices == 0) return TBE_OK;
  if (cache->stage_of_row) return TBE_OK;  // deferred: the next tbe_cache_prepare (or a flush) writes them back
  const int row_units = static_cast<int>(static_cast<int64_t>(D) * dtype_size(dtype) / 8);
  TBE_LAUNCH("cache_unstage", stream, cache_unstage_kernel,
             dim3(grid_for(num_indices, kWavesPerBlock, 256 * 16)), dim3(kBlockThreads),
             static_cast<const uint64_t *>(cache->rows), static_cast<uint64_t *>(cache->backing_rows),
             row_units, keys_sorted, segment_starts, counters, unique_slots,
             cache->num_sets * static_cast<int64_t>(kWays));
  return check_launch("tbe_backward_cached");
}

}  // namespace tbe

extern "C" int tbe_cache_workspace_layout(int64_t num_indices, int64_t num_sets,
                                          tbe_cache_workspace_layout_t *layout) {
  using namespace tbe;
  TBE_REQUIRE(layout, "tbe_cache_workspace_layout: null layout");
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "tbe_cache_workspace_layout: num_indices out of range");
  TBE_REQUIRE(num_sets > 0 && num_sets * kWays < INT32_MAX, "tbe_cache_workspace_layout: num_sets out of range");
  cache_layout(num_indices, num_sets, layout);
  return TBE_OK;
}

extern "C" int tbe_cache_init(const tbe_cache_t *cache, void *stream) {
  using namespace tbe;
  if (int rc = validate_cache("tbe_cache_init", cache)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t slots = cache->num_sets * kWays;
  const dim3 grid(grid_for(slots, kBlockThreads, 4096)), block(kBlockThreads);
  TBE_LAUNCH("cache_init", s, cache_fill_i32_kernel, grid, block, cache->tags, slots, -1);
  TBE_LAUNCH("cache_init", s, cache_fill_i32_kernel, grid, block, cache->last_used, slots, 0);
  TBE_LAUNCH("cache_init", s, cache_fill_i32_kernel, grid, block, cache->use_count, slots, 0);
  if (cache->stage_of_row) {
    TBE_LAUNCH("cache_init", s, cache_fill_i32_kernel, dim3(grid_for(cache->total_rows, kBlockThreads, 4096)), block,
               cache->stage_of_row, cache->total_rows, -1);
    TBE_LAUNCH("cache_init", s, cache_fill_i32_kernel,
               dim3(grid_for(2 * cache->stage_slots + 1, kBlockThreads, 4096)), block, cache->stage_keys,
               2 * cache->stage_slots, -1);
  }
  return check_launch("tbe_cache_init");
}

extern "C" int tbe_cache_prepare(const tbe_cache_t *cache, int32_t dtype, int64_t total_rows,
                                 int64_t max_table_rows, int32_t D, const int32_t *table_offsets, int32_t T,
                                 const int32_t *indices, int64_t num_indices,
                                 const int32_t *offsets, int32_t B, int32_t step, void *workspace,
                                 uint64_t workspace_bytes, void *cache_workspace,
                                 uint64_t cache_workspace_bytes, void *stream, void *side_stream) {
  using namespace tbe;
  const char *name = "tbe_cache_prepare";
  if (int rc = validate_cache(name, cache)) return rc;
  TBE_REQUIRE(T > 0 && B > 0, "%s: T and B must be positive (got %d, %d)", name, T, B);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(step > 0, "%s: steps are numbered from 1 (got %d)", name, step);
  TBE_REQUIRE(table_offsets && offsets && (indices || num_indices == 0), "%s: null pointer argument", name);
  TBE_REQUIRE(stream != side_stream, "%s: side_stream must differ from stream", name);
  tbe_workspace_layout_t l;
  backward_layout(num_indices, D, dtype, T, &l);
  tbe_cache_workspace_layout_t cl;
  cache_layout(num_indices, cache->num_sets, &cl);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  if (!cache_workspace || cache_workspace_bytes < cl.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: cache workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)cl.total_bytes, (unsigned long long)cache_workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipStream_t side = static_cast<hipStream_t>(side_stream);
  char *ws = static_cast<char *>(workspace);
  char *cw = static_cast<char *>(cache_workspace);
  auto i32 = [](char *base, uint64_t off) { return reinterpret_cast<int32_t *>(base + off); };
  int32_t *stats = i32(cw, cl.stats);
  const dim3 block(kBlockThreads);
  TBE_LAUNCH("cache_zero", s, cache_fill_i32_kernel, dim3(1), block, stats, static_cast<int64_t>(8), 0);
  const int unit_count = static_cast<int>(static_cast<int64_t>(D) * dtype_size(dtype) / 8);
  if (cache->stage_of_row && cache->stage_slots > 0) {
    // deferred write-back: the area this step stages into must be empty.  It is, when steps are
    // numbered consecutively (the step before the last released it); otherwise its rows go back now.
    write_back_stage(cache, unit_count, step & 1, s);
    if (num_indices == 0) write_back_stage(cache, unit_count, 1 - (step & 1), s);
  }
  if (num_indices == 0) return check_launch(name);

  int rc = build_plan(l, workspace, table_offsets, T, indices, num_indices, offsets, B, total_rows, max_table_rows, s);
  if (rc) return rc;
  const int32_t *keys_sorted = i32(ws, l.keys_sorted);
  const int32_t *segment_starts = i32(ws, l.segment_starts);
  const int32_t *counters = i32(ws, l.num_unique);
  const int64_t num_sets = cache->num_sets;
  const int64_t num_slots = num_sets * kWays;
  // deferred write-back: two staging areas take turns; this step stages into one while the rows
  // the step before left in the other are fetched from there or written back
  const bool deferred = cache->stage_of_row != nullptr && cache->stage_slots > 0;
  const int64_t half = deferred ? (step & 1) : 0;
  const int64_t stage_base = num_slots + half * cache->stage_slots;
  const int64_t old_stage_base = num_slots + (1 - half) * cache->stage_slots;

  TBE_LAUNCH("cache_zero", s, cache_fill_i32_kernel, dim3(grid_for(2 * (num_sets + 1), kBlockThreads, 1024)),
             block, i32(cw, cl.set_counts), static_cast<int64_t>((cl.set_starts - cl.set_counts) / 4), 0);
  TBE_LAUNCH("cache_lookup", s, cache_lookup_kernel, dim3(grid_for(num_indices, kWavesPerBlock, 256 * 16)),
             block, cache->tags, cache->last_used, cache->use_count, static_cast<uint32_t>(num_sets), step,
             keys_sorted, segment_starts, counters, i32(cw, cl.unique_slots), i32(cw, cl.evicted_keys),
             i32(cw, cl.miss_sets), i32(cw, cl.set_counts), stats);
  TBE_LAUNCH("cache_scan_sets", s, cache_scan_sets_kernel, dim3(1), block, i32(cw, cl.set_counts), num_sets,
             i32(cw, cl.set_starts));
  // the missing rows grouped by set, each set's in ascending order of u: a stable sort of (set, u)
  // over the U unique rows (hits carry the key num_sets and end up behind every set).  The
  // sorted keys go to the slot-per-lookup array, which is written later; the sort's scratch is
  // the plan's, free since the plan was built.
  {
    int bits = 1;
    while ((int64_t{1} << bits) <= num_sets) ++bits;
    const int rc_sort = sort_pairs(i32(cw, cl.miss_sets), nullptr, i32(cw, cl.lookup_slots), i32(cw, cl.miss_list),
                                   num_indices, bits, ws + l.sort_scratch, s, nullptr, counters);
    if (rc_sort) return rc_sort;
  }
  TBE_LAUNCH("cache_insert", s, cache_insert_kernel, dim3(grid_for(num_sets, kWavesPerBlock, 256 * 16)), block,
             cache->tags, cache->last_used, cache->use_count, num_sets, cache->policy, step, keys_sorted,
             segment_starts, i32(cw, cl.set_starts), i32(cw, cl.miss_list), i32(cw, cl.unique_slots),
             i32(cw, cl.evicted_keys), stats, cache->stage_slots, stage_base);
  if (deferred)
    TBE_LAUNCH("cache_resolve", s, cache_resolve_kernel, dim3(grid_for(num_indices, kBlockThreads, 256 * 16)), block,
               keys_sorted, segment_starts, counters, i32(cw, cl.unique_slots), i32(cw, cl.evicted_keys),
               cache->stage_of_row, cache->stage_keys, i32(cw, cl.fetch_source), num_slots, stats);

  // Row traffic over the host link goes to the side stream while this stream builds the
  // per-lookup slot table; the side stream is joined before anything reads the cached rows.
  hipEvent_t ready = join_event(0), filled = join_event(1);
  if (!ready || !filled) return fail(TBE_ERR_HIP, "%s: could not create events", name);
  hipError_t e = hipEventRecord(ready, s);
  if (e == hipSuccess) e = hipStreamWaitEvent(side, ready, 0);
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "%s: %s", name, hipGetErrorString(e));
  const int row_units = static_cast<int>(static_cast<int64_t>(D) * dtype_size(dtype) / 8);
  int32_t *old_stage_keys = deferred ? cache->stage_keys + (1 - half) * cache->stage_slots : nullptr;
  TBE_LAUNCH("cache_fill", side, cache_fill_kernel,
             dim3((deferred ? 2 : 1) * grid_for(num_indices, kWavesPerBlock, 256 * 16)), block,
             static_cast<uint64_t *>(cache->rows), static_cast<uint64_t *>(cache->backing_rows), row_units,
             keys_sorted, segment_starts, counters, i32(cw, cl.unique_slots), i32(cw, cl.evicted_keys),
             deferred ? i32(cw, cl.fetch_source) : static_cast<int32_t *>(nullptr), old_stage_keys, old_stage_base,
             cache->stage_slots);
  if (deferred)
    TBE_LAUNCH("cache_retire_stage", side, cache_retire_stage_kernel,
               dim3(grid_for(cache->stage_slots, kBlockThreads, 1024)), block, cache->stage_of_row, old_stage_keys,
               old_stage_base, cache->stage_slots);
  TBE_LAUNCH("cache_locate", s, cache_locate_kernel, dim3(grid_for(num_indices, kBlockThreads, 256 * 16)), block,
             i32(ws, l.positions_sorted), i32(ws, l.segment_ids), i32(cw, cl.unique_slots), num_indices,
             i32(cw, cl.lookup_slots));
  e = hipEventRecord(filled, side);
  if (e == hipSuccess) e = hipStreamWaitEvent(s, filled, 0);
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "%s: %s", name, hipGetErrorString(e));
  return check_launch(name);
}

extern "C" int tbe_cache_flush(const tbe_cache_t *cache, int32_t dtype, int32_t D, void *stream) {
  using namespace tbe;
  if (int rc = validate_cache("tbe_cache_flush", cache)) return rc;
  TBE_REQUIRE(D > 0 && D % 4 == 0, "tbe_cache_flush: D must be a positive multiple of 4 (got %d)", D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "tbe_cache_flush: bad dtype %d", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t slots = cache->num_sets * kWays;
  const int row_units = static_cast<int>(static_cast<int64_t>(D) * dtype_size(dtype) / 8);
  if (cache->stage_of_row && cache->stage_slots > 0) {
    // the rows the last step staged (one of the two areas; the other is empty)
    write_back_stage(cache, row_units, 0, s);
    write_back_stage(cache, row_units, 1, s);
  }
  TBE_LAUNCH("cache_flush", s, cache_flush_kernel, dim3(grid_for(slots, kWavesPerBlock, 256 * 16)),
             dim3(kBlockThreads), cache->tags, static_cast<const uint64_t *>(cache->rows),
             static_cast<uint64_t *>(cache->backing_rows), row_units, slots);
  return check_launch("tbe_cache_flush");
}
