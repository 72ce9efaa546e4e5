// HBM-resident set-associative row cache in front of a host-resident table, for gfx950.
//
// 64 ways per set = one wavefront probes a set with one coalesced 256-byte tag load and a
// ballot.  The reference has no cache; the specification is the comment above tbe_cache_t in
// include/tbe_hip.h.  Per step:
//   lookup   one wavefront per unique row: ballot match -> slot, mark used; misses count per set
//   scan     exclusive scan of the per-set miss counts
//   group    misses written into their set's range of miss_list (a stable sort by set)
//   insert   one wavefront per set: for each missing row in ascending order, victim = lowest
//            (priority, way) among slots not used in this step (wavefront min + ballot)
//   locate   slot of every lookup position, for the forward gather
// Every decision is a function of integers only, so the tags after a step are reproducible.
//
// Row traffic.  Without deferred write-back one launch on the side stream writes back each evicted
// row and fetches each new row into its slot or staging row, and the staged rows go home after the
// update.  With deferred write-back (cache->stage_of_row) the decisions above touch no row, so the
// plan of step x+1 can be made, and most of its rows moved, while step x still computes:
//   resolve  where every fetched row comes from (the backing table, or a staging row that still
//            holds its newest value) and where it lands: a staged row in its staging row, an
//            inserted row in a *landing* row of the same area, because its slot may still serve the
//            step before
//   retire   the list of rows of the oldest of the three staging areas that nobody took over
//   fill     (link stream) the fetches whose source is final, and that list back to the host
//   commit   (caller's stream, after the update of the step before) the fetches whose source that
//            update wrote, and slot <-> landing row swaps: the new row enters its slot, the evicted
//            row waits in the landing row for the fill launch two steps later
// so nothing the host link carries waits for, or is waited for by, the kernels of a step.

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
       kStatFromStaging, kStatWrittenOut, kStatLate, kStatNoLanding, kStatCount = 16 };

// Deferred write-back: three staging areas take turns by the sequence number of the step.
constexpr int kAreas = 3;
__host__ __device__ inline int64_t area_of(int64_t sequence) { return ((sequence % kAreas) + kAreas) % kAreas; }
// stage_of_row value "the backing row is written by the caller's stream during step `sequence`"
__host__ __device__ inline int32_t host_written_mark(int32_t sequence) { return -(2 + sequence); }

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
    int64_t stage_base, int32_t *__restrict__ landing) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  int inserted = 0, written_back = 0, uncached = 0, staged = 0, no_landing = 0;
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
          if (landing) {
            // The set owns the staging indices [begin, end): its staged rows take the first ones (below),
            // its inserted rows the last `takers`, as landing rows.
            const int64_t index = static_cast<int64_t>(end) - takers + j0 + j;
            landing[u] = index < stage_slots ? static_cast<int32_t>(stage_base + index) : -1;
            if (index >= stage_slots) ++no_landing;
          }
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
    if (no_landing) atomicAdd(&stats[kStatNoLanding], no_landing);
  }
}

// ---------------------------------------------------------------- deferred write-back
// stage_keys[3 * stage_slots]: per staging row, -1 = free, key >= 0 = the row holds the newest value
// of that table row and has to go back to the backing table, -(key + 2) = it held that row until a
// later step took it over.  stage_of_row[total_rows]: the row of `rows` (>= num_slots) whose
// stage_keys entry names the table row, -1 = none (the backing table or a slot holds the newest
// value), or host_written_mark(s): none, and the caller's stream writes the backing row in step s.
//
// fetch_source[u] for a row that step x fetches: -1 the backing table, read by the fill launch;
// >= num_slots a staging row -- one of the area before last, whose rows are final, is read by the
// fill launch, one of the last step's area by the commit launch, after that step's update; -3 the
// backing table, read by the commit launch (the last step writes that row on the caller's stream).

// After the step's slots are decided: sources and destinations of the rows it fetches.
__global__ __launch_bounds__(kBlockThreads) void cache_resolve_kernel(
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    const int32_t *__restrict__ evicted_keys, const int32_t *__restrict__ landing,
    int32_t *__restrict__ stage_of_row, int32_t *__restrict__ stage_keys,
    int32_t *__restrict__ fetch_source, int64_t num_slots, int64_t stage_slots, int32_t sequence,
    int32_t *__restrict__ stats) {
  const int U = counters[0];
  const int64_t final_area = num_slots + area_of(sequence - 2) * stage_slots;  // rows nobody updates any more
  int from_staging = 0, late = 0;
  for (int64_t u = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; u < U;
       u += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int32_t evicted = evicted_keys[u];
    const int32_t slot = unique_slots[u];
    if (evicted == -2 && slot >= 0) continue;  // a hit
    const int32_t key = keys_sorted[segment_starts[u]];
    const int32_t held = stage_of_row[key];
    const bool held_final = held >= final_area && held < final_area + stage_slots;
    if (evicted == -2) {
      // Left in the backing table for this step: forward and update address the backing row.  Its
      // newest value may still sit in a staging row.  One of the oldest area goes home in this
      // step's fill launch anyway (the entry is left as it is); one of the last step's area is
      // copied home by the commit launch.
      fetch_source[u] = (held >= 0 && !held_final) ? held : -1;
      if (held >= 0 && !held_final) stage_keys[held - num_slots] = -(key + 2);
      stage_of_row[key] = host_written_mark(sequence);
      continue;
    }
    const bool staged = slot >= num_slots;
    const int32_t land = staged ? slot : landing[u];
    int32_t source = -1;
    if (held >= 0) {
      if (land < 0 && held_final) {
        // an inserted row without a landing row is fetched by the commit launch; by then the oldest
        // area may be in use again, so its row goes home with the fill launch and is read from there
        source = -3;
        ++late;
      } else {
        source = held;
        stage_keys[held - num_slots] = -(key + 2);
        ++from_staging;
        if (!held_final) ++late;
      }
    } else if (held == host_written_mark(sequence - 1) || land < 0) {
      source = -3;
      ++late;
    }
    fetch_source[u] = source;
    if (staged) {
      stage_of_row[key] = slot;
      stage_keys[slot - num_slots] = key;
    } else {
      stage_of_row[key] = -1;  // the row lives in a slot of the cache now
      if (evicted >= 0) {
        if (land >= 0) {  // the commit launch moves the evicted row into the landing row
          stage_of_row[evicted] = land;
          stage_keys[land - num_slots] = evicted;
        } else {          // or straight to the backing table
          stage_of_row[evicted] = host_written_mark(sequence);
        }
      }
    }
  }
  for (int m = kWave / 2; m > 0; m >>= 1) {
    from_staging += __shfl_xor(from_staging, m, kWave);
    late += __shfl_xor(late, m, kWave);
  }
  if ((threadIdx.x & (kWave - 1)) == 0) {
    if (from_staging) atomicAdd(&stats[kStatFromStaging], from_staging);
    if (late) atomicAdd(&stats[kStatLate], late);
  }
}

// The oldest staging area is released: what its rows still owe the backing table is listed for
// the fill launch (write_out[i] = key, or -1), its entries are emptied, and stage_of_row forgets
// the rows it held.
__global__ __launch_bounds__(kBlockThreads) void cache_retire_stage_kernel(
    int32_t *__restrict__ stage_of_row, int32_t *__restrict__ old_stage_keys, int64_t old_stage_base,
    int64_t stage_slots, int32_t *__restrict__ write_out, int32_t *__restrict__ stats) {
  int pending = 0;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < stage_slots;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const int32_t entry = old_stage_keys[i];
    if (write_out) write_out[i] = entry >= 0 ? entry : -1;
    if (entry == -1) continue;
    const int32_t key = entry >= 0 ? entry : -(entry + 2);
    if (stage_of_row[key] == old_stage_base + i) stage_of_row[key] = -1;
    old_stage_keys[i] = -1;
    if (entry >= 0) ++pending;
  }
  for (int m = kWave / 2; m > 0; m >>= 1) pending += __shfl_xor(pending, m, kWave);
  if (stats && (threadIdx.x & (kWave - 1)) == 0 && pending) atomicAdd(&stats[kStatWrittenOut], pending);
}

// Rows move as 8-byte units.  A row of the cache (slot, staging or landing row) has row_units of
// them: D * element size / 8, D the widest table's with tables of different widths.  Where a row
// of the backing table lies, and how many units it has: row `key` at key * row_units with uniform
// tables; else the table is found by bisecting the tables' first row ids.
struct BackingMap {
  uint64_t *rows;
  int row_units;
  const int64_t *table_offsets;  // tables of different widths (null otherwise): first element of each table,
  const int32_t *table_rows;     // first row id of each table, [T + 1],
  const int32_t *dim_offsets;    // first output column of each table, [T + 1]
  int T;
  int unit_shift;                // log2 of the elements per unit
};
struct BackingRow {
  uint64_t *row;
  int units;
};
__device__ __forceinline__ BackingRow backing_row(const BackingMap &m, int64_t key) {
  if (!m.table_offsets) return BackingRow{m.rows + key * m.row_units, m.row_units};
  int lo = 0, hi = m.T;  // table_rows[lo] <= key < table_rows[hi]
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (m.table_rows[mid] <= key) lo = mid;
    else hi = mid;
  }
  const int64_t D = m.dim_offsets[lo + 1] - m.dim_offsets[lo];
  const int64_t element = m.table_offsets[lo] + (key - m.table_rows[lo]) * D;
  return BackingRow{m.rows + (element >> m.unit_shift), static_cast<int>(D >> m.unit_shift)};
}

// One wavefront per row.
// Without deferred write-back: the evicted row goes to the backing table, the new row comes into
// the slot or the staging row.
__global__ __launch_bounds__(kBlockThreads) void cache_fill_kernel(
    uint64_t *__restrict__ cache_rows, BackingMap backing,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    const int32_t *__restrict__ evicted_keys) {
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t i = wave_id; i < U; i += stride) {
    const int32_t evicted = evicted_keys[i];
    if (evicted == -2) continue;
    const int64_t key = keys_sorted[segment_starts[i]];
    uint64_t *slot_row = cache_rows + static_cast<int64_t>(unique_slots[i]) * backing.row_units;
    const BackingRow fresh = backing_row(backing, key);
    if (evicted >= 0) {
      const BackingRow old = backing_row(backing, evicted);
      for (int k = lane; k < old.units; k += kWave) old.row[k] = slot_row[k];
    }
    for (int k = lane; k < fresh.units; k += kWave) slot_row[k] = fresh.row[k];
  }
}

// Deferred write-back, the launch on the link stream.  A wavefront takes kFillBatch rows of the
// oldest staging area that may be owed to the backing table (write_out) and kFillBatch unique rows
// of this step whose source may be final (the backing table, or a row of that same area) at a time:
// one lane per row works out source and destination, then the whole wavefront moves the 2 *
// kFillBatch rows with all loads issued before the first store.  (Packing only rows that move into
// a batch, instead of consecutive list entries with their gaps, made the launch itself 1.5 %
// faster and the step beside it 4 % slower.)  Both directions of the host link
// are busy at once in every wavefront, and a wavefront keeps several kilobytes in flight, so that a
// grid of a few hundred workgroups fills the link and leaves the compute units to the kernels of
// the step that runs beside this launch.  (A grid that occupies every wavefront slot, each
// wavefront with one row in flight, moved the same bytes in the same time when alone, but the
// step's own kernels then waited for its wavefronts to retire.)
// Nothing here touches a slot or a row that the step before may still read or update.
constexpr int kFillBatch = 4;
__global__ __launch_bounds__(kBlockThreads) void cache_fill_deferred_kernel(
    uint64_t *__restrict__ cache_rows, BackingMap backing,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    const int32_t *__restrict__ evicted_keys, const int32_t *__restrict__ landing,
    const int32_t *__restrict__ fetch_source, const int32_t *__restrict__ write_out, int64_t old_stage_base,
    int64_t stage_slots, int64_t num_slots) {
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  const int row_units = backing.row_units;
  const int64_t items = U > stage_slots ? U : stage_slots;
  for (int64_t base = wave_id * kWave; base < items; base += stride * kWave) {
    // 64 entries of each list at a time are screened first, one per lane: a step whose rows are
    // nearly all resident passes over its lists without taking them apart
    const int64_t mine = base + lane;
    const bool owes = mine < stage_slots && write_out[mine] >= 0;
    const bool fetches = mine < U && evicted_keys[mine] != -2;
    const unsigned long long busy = __ballot(owes || fetches);
    if (busy == 0ull) continue;
    for (int sub = 0; sub < kWave; sub += kFillBatch) {
      if (((busy >> sub) & ((1ull << kFillBatch) - 1ull)) == 0ull) continue;
      const int64_t i0 = base + sub;
      // lanes 0 .. kFillBatch-1: a row of the released area each; the next kFillBatch lanes: a unique row each
      const uint64_t *my_src = cache_rows;  // a harmless source for the lanes without a row to move
      uint64_t *my_dst = nullptr;
      int my_units = 0;
      if (lane < kFillBatch) {
        const int64_t i = i0 + lane;
        if (i < stage_slots) {
          const int64_t key = write_out[i];
          if (key >= 0) {
            const BackingRow home = backing_row(backing, key);
            my_src = cache_rows + (old_stage_base + i) * row_units;
            my_dst = home.row;
            my_units = home.units;
          }
        }
      } else if (lane < 2 * kFillBatch) {
        const int64_t i = i0 + lane - kFillBatch;
        if (i < U && evicted_keys[i] != -2) {
          const int64_t slot = unique_slots[i];
          const int64_t land = slot >= num_slots ? slot : landing[i];
          const int64_t source = fetch_source[i];
          if (land >= 0) {
            const BackingRow home = backing_row(backing, keys_sorted[segment_starts[i]]);
            if (source == -1) {
              my_src = home.row;
              my_dst = cache_rows + land * row_units;
              my_units = home.units;
            } else if (source >= old_stage_base && source < old_stage_base + stage_slots) {
              my_src = cache_rows + source * row_units;
              my_dst = cache_rows + land * row_units;
              my_units = home.units;
            }  // else: the commit launch fetches it
          }
        }
      }
      const uint64_t *src[2 * kFillBatch];
      uint64_t *dst[2 * kFillBatch];
      int units[2 * kFillBatch];  // (0 for a lane without a row to move)
      int most = 0;
#pragma unroll
      for (int j = 0; j < 2 * kFillBatch; ++j) {
        src[j] = reinterpret_cast<const uint64_t *>(__shfl(reinterpret_cast<unsigned long long>(my_src), j, kWave));
        dst[j] = reinterpret_cast<uint64_t *>(__shfl(reinterpret_cast<unsigned long long>(my_dst), j, kWave));
        units[j] = __shfl(my_units, j, kWave);
        most = max(most, units[j]);
      }
      for (int k = lane; k < most; k += kWave) {
        uint64_t v[2 * kFillBatch];
#pragma unroll
        for (int j = 0; j < 2 * kFillBatch; ++j) v[j] = k < units[j] ? src[j][k] : 0;
#pragma unroll
        for (int j = 0; j < 2 * kFillBatch; ++j)
          if (k < units[j]) dst[j][k] = v[j];
      }
    }
  }
}

// Deferred write-back, the launch on the caller's stream, after the fill launch and after the
// update of the step before: the fetches that had to wait for that update, the slot <-> landing
// row swap of every inserted row (the new row into the slot, the evicted one into the landing
// row, or, without one, straight to the backing table), and the newest value of a row that this
// step leaves in the backing table, if the last step's staging area still held it.
__global__ __launch_bounds__(kBlockThreads) void cache_commit_kernel(
    uint64_t *__restrict__ cache_rows, BackingMap backing,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ unique_slots,
    const int32_t *__restrict__ evicted_keys, const int32_t *__restrict__ landing,
    const int32_t *__restrict__ fetch_source, int64_t old_stage_base, int64_t stage_slots, int64_t num_slots) {
  const int lane = threadIdx.x & (kWave - 1);
  const int U = counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  // 64 unique rows at a time, one per lane: most rows of a step are hits, or were fetched by the fill
  // launch; a lane whose row has work to do here describes it as one copy, or two for a swap (the
  // new row into the slot, the slot's old content to the landing row or the backing table).  The
  // wavefront then moves kCommitBatch rows at a time with every load issued before the first store,
  // which is also what makes a swap through the same landing row correct.
  constexpr int kCommitBatch = 4;
  const int row_units = backing.row_units;
  for (int64_t base = wave_id * kWave; base < U; base += stride * kWave) {
    const int64_t mine = min(base + lane, static_cast<int64_t>(U) - 1);
    const int32_t evicted = evicted_keys[mine];
    const int64_t slot = unique_slots[mine];
    const int64_t source = fetch_source[mine];
    const bool by_fill = source == -1 || (source >= old_stage_base && source < old_stage_base + stage_slots);
    const bool idle = (evicted == -2 && (slot >= 0 || source < 0))        // a hit, or a row left in the table
                      || (evicted != -2 && slot >= num_slots && by_fill);  // staged, and fetched already
    const bool busy = base + lane < U && !idle;
    const uint64_t *src0 = cache_rows, *src1 = cache_rows;  // (harmless sources for lanes without a copy)
    uint64_t *dst0 = nullptr, *dst1 = nullptr;
    int units0 = 0, units1 = 0;
    if (busy) {
      const BackingRow home = backing_row(backing, keys_sorted[segment_starts[mine]]);
      units0 = home.units;
      if (evicted == -2) {
        // a row that stays in the backing table, whose newest value the last step left in a staging row
        src0 = cache_rows + source * row_units;
        dst0 = home.row;
      } else {
        const uint64_t *late_src = source >= 0 ? cache_rows + source * row_units : home.row;
        if (slot >= num_slots) {
          src0 = late_src;  // a staged row that the fill launch could not fetch yet
          dst0 = cache_rows + slot * row_units;
        } else {
          const int64_t land = landing[mine];
          uint64_t *slot_row = cache_rows + slot * row_units;
          src0 = (by_fill && land >= 0) ? cache_rows + land * row_units : late_src;
          dst0 = slot_row;
          if (evicted >= 0) {
            // (the evicted row may belong to a table of another width than the row that replaces it)
            const BackingRow old_home = backing_row(backing, evicted);
            src1 = slot_row;
            dst1 = land >= 0 ? cache_rows + land * row_units : old_home.row;
            units1 = old_home.units;
          }
        }
      }
    }
    unsigned long long todo = __ballot(busy);
    while (todo != 0ull) {
      const uint64_t *src[2 * kCommitBatch];
      uint64_t *dst[2 * kCommitBatch];
      int units[2 * kCommitBatch];  // (0: no copy)
      int most = 0;
#pragma unroll
      for (int j = 0; j < kCommitBatch; ++j) {
        const int which = todo ? __ffsll(static_cast<long long>(todo)) - 1 : -1;
        todo &= todo - (todo ? 1ull : 0ull);
        const int from = max(which, 0);
        src[2 * j] = reinterpret_cast<const uint64_t *>(__shfl(reinterpret_cast<unsigned long long>(src0), from, kWave));
        dst[2 * j] = reinterpret_cast<uint64_t *>(__shfl(reinterpret_cast<unsigned long long>(dst0), from, kWave));
        units[2 * j] = which >= 0 ? __shfl(units0, from, kWave) : 0;
        src[2 * j + 1] = reinterpret_cast<const uint64_t *>(__shfl(reinterpret_cast<unsigned long long>(src1), from, kWave));
        dst[2 * j + 1] = reinterpret_cast<uint64_t *>(__shfl(reinterpret_cast<unsigned long long>(dst1), from, kWave));
        units[2 * j + 1] = which >= 0 ? __shfl(units1, from, kWave) : 0;
        most = max(most, max(units[2 * j], units[2 * j + 1]));
      }
      for (int k = lane; k < most; k += kWave) {
        uint64_t v[2 * kCommitBatch];
#pragma unroll
        for (int j = 0; j < 2 * kCommitBatch; ++j) v[j] = k < units[j] ? src[j][k] : 0;
#pragma unroll
        for (int j = 0; j < 2 * kCommitBatch; ++j)
          if (k < units[j]) dst[j][k] = v[j];
      }
    }
  }
}

// Deferred write-back, outside a step (flush): the rows of the staging areas that hold a key go
// to the backing table.  A wavefront reads 64 entries at a time and copies the rows of those that
// hold one, so an empty area costs one pass over its entries.
__global__ __launch_bounds__(kBlockThreads) void cache_unstage_area_kernel(
    const uint64_t *__restrict__ cache_rows, BackingMap backing,
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
      const uint64_t *src = cache_rows + (stage_base + i0 + j) * backing.row_units;
      const BackingRow home = backing_row(backing, key);
      for (int k = lane; k < home.units; k += kWave) home.row[k] = src[k];
    }
  }
}

// After the update: staged rows (slot >= first_stage_slot) go back to the backing table.
__global__ __launch_bounds__(kBlockThreads) void cache_unstage_kernel(
    const uint64_t *__restrict__ cache_rows, BackingMap backing,
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
    const uint64_t *src = cache_rows + slot * backing.row_units;
    const BackingRow home = backing_row(backing, key);
    for (int i = lane; i < home.units; i += kWave) home.row[i] = src[i];
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
    const int32_t *__restrict__ tags, const uint64_t *__restrict__ cache_rows, BackingMap backing,
    int64_t num_slots) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t slot = wave_id; slot < num_slots; slot += stride) {
    const int64_t key = tags[slot];
    if (key < 0) continue;
    const uint64_t *src = cache_rows + slot * backing.row_units;
    const BackingRow home = backing_row(backing, key);
    for (int i = lane; i < home.units; i += kWave) home.row[i] = src[i];
  }
}

void cache_layout(int64_t n, int64_t num_sets, int64_t stage_slots, tbe_cache_workspace_layout_t *l) {
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
  l->landing = off; off += ints;
  l->write_out = off; off += align_up(static_cast<uint64_t>(stage_slots > 0 ? stage_slots : 1) * 4, 256);
  l->total_bytes = off;
}

inline unsigned grid_for(int64_t work_items, int64_t per_block, int64_t cap) {
  return static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(ceil_div(work_items, per_block), cap)));
}

inline bool deferred(const tbe_cache_t *cache) { return cache->stage_of_row != nullptr && cache->stage_slots > 0; }
inline bool mixed_tables(const tbe_cache_t *cache) { return cache->mixed_table_offsets != nullptr; }

// D: elements of a cache row (with tables of different widths: of the widest table's rows)
BackingMap backing_map(const tbe_cache_t *cache, int32_t D, int32_t dtype) {
  const int element = static_cast<int>(dtype_size(dtype));
  return BackingMap{static_cast<uint64_t *>(cache->backing_rows),
                    static_cast<int>(static_cast<int64_t>(D) * element / 8),
                    cache->mixed_table_offsets,
                    cache->mixed_table_rows,
                    cache->mixed_dim_offsets,
                    cache->mixed_T,
                    element == 2 ? 2 : element == 4 ? 1 : 0};
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
    TBE_REQUIRE(cache->num_sets * kWays + kAreas * cache->stage_slots < INT32_MAX, "%s: stage_slots out of range",
                name);
  }
  if (cache->mixed_table_offsets || cache->mixed_table_rows || cache->mixed_dim_offsets || cache->mixed_T) {
    TBE_REQUIRE(cache->mixed_table_offsets && cache->mixed_table_rows && cache->mixed_dim_offsets && cache->mixed_T > 0,
                "%s: tables of different widths need mixed_table_offsets, mixed_table_rows, mixed_dim_offsets and mixed_T",
                name);
  }
  return TBE_OK;
}

// Deferred write-back, outside a step: the rows of staging area `area` that still wait for their
// write-back go to the backing table, and the area is released -- unless a planned batch still
// works on it (`keep`): then its rows stay listed, since that batch's update changes them again.
void write_back_stage(const tbe_cache_t *cache, const BackingMap &backing, int64_t area, bool keep, hipStream_t stream) {
  const int64_t base = cache->num_sets * kWays + area * cache->stage_slots;
  int32_t *keys = cache->stage_keys + area * cache->stage_slots;
  TBE_LAUNCH("cache_unstage", stream, cache_unstage_area_kernel,
             dim3(grid_for(cache->stage_slots, kWavesPerBlock, 256 * 16)), dim3(kBlockThreads),
             static_cast<const uint64_t *>(cache->rows), backing, keys, base, cache->stage_slots);
  if (keep) return;
  TBE_LAUNCH("cache_retire_stage", stream, cache_retire_stage_kernel,
             dim3(grid_for(cache->stage_slots, kBlockThreads, 1024)), dim3(kBlockThreads), cache->stage_of_row, keys,
             base, cache->stage_slots, static_cast<int32_t *>(nullptr), static_cast<int32_t *>(nullptr));
}

// One event per calling thread and purpose, used to order two streams: it is waited for right
// after it is recorded, so recording it again later does not disturb the earlier wait.
hipEvent_t join_event(int which) {
  thread_local hipEvent_t events[2] = {nullptr, nullptr};
  if (!events[which]) {
    if (hipEventCreateWithFlags(&events[which], hipEventDisableTiming) != hipSuccess) return nullptr;
  }
  return events[which];
}

int order_after(const char *name, hipStream_t later, hipStream_t earlier, int which) {
  if (later == earlier) return TBE_OK;
  hipEvent_t event = join_event(which);
  if (!event) return fail(TBE_ERR_HIP, "%s: could not create an event", name);
  hipError_t e = hipEventRecord(event, earlier);
  if (e == hipSuccess) e = hipStreamWaitEvent(later, event, 0);
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "%s: %s", name, hipGetErrorString(e));
  return TBE_OK;
}

struct PlanArgs {
  const tbe_cache_t *cache;
  int32_t dtype;
  int64_t total_rows, max_table_rows;
  int32_t D;
  const int32_t *table_offsets;
  int32_t T;
  const int32_t *indices;
  int64_t num_indices;
  const int32_t *offsets;
  int32_t B, step, sequence;
  void *workspace;
  uint64_t workspace_bytes;
  void *cache_workspace;
  uint64_t cache_workspace_bytes;
};

int validate_plan(const char *name, const PlanArgs &a, tbe_workspace_layout_t *l, tbe_cache_workspace_layout_t *cl) {
  if (int rc = validate_cache(name, a.cache)) return rc;
  TBE_REQUIRE(a.T > 0 && a.B > 0, "%s: T and B must be positive (got %d, %d)", name, a.T, a.B);
  TBE_REQUIRE(a.D > 0 && a.D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, a.D);
  TBE_REQUIRE(a.dtype >= TBE_DTYPE_F32 && a.dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, a.dtype);
  TBE_REQUIRE(a.total_rows > 0 && a.total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(a.max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(a.num_indices >= 0 && a.num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(a.T) * a.B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(a.step > 0, "%s: steps are numbered from 1 (got %d)", name, a.step);
  TBE_REQUIRE(a.sequence >= 0 && a.sequence < INT32_MAX - 4, "%s: sequence out of range (got %d)", name, a.sequence);
  TBE_REQUIRE(a.table_offsets && a.offsets && (a.indices || a.num_indices == 0), "%s: null pointer argument", name);
  TBE_REQUIRE(!mixed_tables(a.cache) || a.T == a.cache->mixed_T, "%s: T = %d, but the cache describes %d tables", name,
              a.T, a.cache->mixed_T);
  backward_layout(a.num_indices, mixed_tables(a.cache) ? mixed_layout_dim(a.dtype) : a.D, a.dtype, a.T, l);
  cache_layout(a.num_indices, a.cache->num_sets, a.cache->stage_slots, cl);
  if (!a.workspace || a.workspace_bytes < l->total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l->total_bytes, (unsigned long long)a.workspace_bytes);
  if (!a.cache_workspace || a.cache_workspace_bytes < cl->total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: cache workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)cl->total_bytes, (unsigned long long)a.cache_workspace_bytes);
  return TBE_OK;
}

inline int32_t *i32_at(void *base, uint64_t off) { return reinterpret_cast<int32_t *>(static_cast<char *>(base) + off); }

// The decisions of a step on `s` (they touch no row), then the row traffic that does not depend
// on the step before on `link`.
int plan_step(const char *name, const PlanArgs &a, const tbe_workspace_layout_t &l,
              const tbe_cache_workspace_layout_t &cl, hipStream_t s, hipStream_t link) {
  const tbe_cache_t *cache = a.cache;
  void *ws = a.workspace, *cw = a.cache_workspace;
  const int64_t n = a.num_indices;
  int32_t *stats = i32_at(cw, cl.stats);
  const dim3 block(kBlockThreads);
  const int64_t num_sets = cache->num_sets;
  const int64_t num_slots = num_sets * kWays;
  const bool defer = deferred(cache);
  const BackingMap backing = backing_map(cache, a.D, a.dtype);
  // deferred write-back: this step stages into one of three areas; the area of the step before may
  // still be updated; the one before that is final and is released by this step
  const int64_t stage_base = num_slots + (defer ? area_of(a.sequence) * cache->stage_slots : 0);
  const int64_t old_area = area_of(a.sequence - 2);
  const int64_t old_stage_base = num_slots + old_area * cache->stage_slots;
  const int32_t *keys_sorted = i32_at(ws, l.keys_sorted);
  const int32_t *segment_starts = i32_at(ws, l.segment_starts);
  int32_t *counters = i32_at(ws, l.num_unique);

  TBE_LAUNCH("cache_zero", s, cache_fill_i32_kernel, dim3(1), block, stats, static_cast<int64_t>(kStatCount), 0);
  if (n == 0) {
    if (!defer) return check_launch(name);
    TBE_LAUNCH("cache_zero", s, cache_fill_i32_kernel, dim3(1), block, counters, static_cast<int64_t>(1), 0);
  } else {
    int rc = build_plan(l, ws, a.table_offsets, a.T, a.indices, n, a.offsets, a.B, a.total_rows, a.max_table_rows, s);
    if (rc) return rc;
    TBE_LAUNCH("cache_zero", s, cache_fill_i32_kernel, dim3(grid_for(2 * (num_sets + 1), kBlockThreads, 1024)),
               block, i32_at(cw, cl.set_counts), static_cast<int64_t>((cl.set_starts - cl.set_counts) / 4), 0);
    TBE_LAUNCH("cache_lookup", s, cache_lookup_kernel, dim3(grid_for(n, kWavesPerBlock, 256 * 16)), block,
               cache->tags, cache->last_used, cache->use_count, static_cast<uint32_t>(num_sets), a.step, keys_sorted,
               segment_starts, counters, i32_at(cw, cl.unique_slots), i32_at(cw, cl.evicted_keys),
               i32_at(cw, cl.miss_sets), i32_at(cw, cl.set_counts), stats);
    TBE_LAUNCH("cache_scan_sets", s, cache_scan_sets_kernel, dim3(1), block, i32_at(cw, cl.set_counts), num_sets,
               i32_at(cw, cl.set_starts));
    // the missing rows grouped by set, each set's in ascending order of u: a stable sort of (set, u)
    // over the U unique rows (hits carry the key num_sets and end up behind every set).  The
    // sorted keys go to the slot-per-lookup array, which is written later; the sort's scratch is
    // the plan's, free since the plan was built.
    int bits = 1;
    while ((int64_t{1} << bits) <= num_sets) ++bits;
    rc = sort_pairs(i32_at(cw, cl.miss_sets), nullptr, i32_at(cw, cl.lookup_slots), i32_at(cw, cl.miss_list), n, bits,
                    static_cast<char *>(ws) + l.sort_scratch, s, nullptr, counters);
    if (rc) return rc;
    TBE_LAUNCH("cache_insert", s, cache_insert_kernel, dim3(grid_for(num_sets, kWavesPerBlock, 256 * 16)), block,
               cache->tags, cache->last_used, cache->use_count, num_sets, cache->policy, a.step, keys_sorted,
               segment_starts, i32_at(cw, cl.set_starts), i32_at(cw, cl.miss_list), i32_at(cw, cl.unique_slots),
               i32_at(cw, cl.evicted_keys), stats, cache->stage_slots, stage_base,
               defer ? i32_at(cw, cl.landing) : static_cast<int32_t *>(nullptr));
    if (defer)
      TBE_LAUNCH("cache_resolve", s, cache_resolve_kernel, dim3(grid_for(n, kBlockThreads, 256 * 16)), block,
                 keys_sorted, segment_starts, counters, i32_at(cw, cl.unique_slots), i32_at(cw, cl.evicted_keys),
                 i32_at(cw, cl.landing), cache->stage_of_row, cache->stage_keys, i32_at(cw, cl.fetch_source),
                 num_slots, cache->stage_slots, a.sequence, stats);
  }
  if (defer)
    TBE_LAUNCH("cache_retire_stage", s, cache_retire_stage_kernel,
               dim3(grid_for(cache->stage_slots, kBlockThreads, 1024)), block, cache->stage_of_row,
               cache->stage_keys + old_area * cache->stage_slots, old_stage_base, cache->stage_slots,
               i32_at(cw, cl.write_out), stats);
  if (n > 0)
    TBE_LAUNCH("cache_locate", s, cache_locate_kernel, dim3(grid_for(n, kBlockThreads, 256 * 16)), block,
               i32_at(ws, l.positions_sorted), i32_at(ws, l.segment_ids), i32_at(cw, cl.unique_slots), n,
               i32_at(cw, cl.lookup_slots));

  // Row traffic over the host link goes to the link stream, behind the decisions.
  if (int rc = order_after(name, link, s, 0)) return rc;
  if (defer) {
    const int64_t work = std::max<int64_t>(n, cache->stage_slots);
    // One workgroup per compute unit.  Measured on 35.6 GB of host-resident tables with 6.6 M rows in and
    // 3.9 M rows out per step: 64 / 128 / 256 / 512 / 2048 workgroups move a step's rows in 59 / 51 / 48 / 48 /
    // 49 ms when alone, but from 384 workgroups on the kernels of the step that runs beside the launch
    // crawl behind its outstanding host reads, and the step takes 62 / 55 / 50 / 55 / 58 ms.
    TBE_LAUNCH("cache_fill", link, cache_fill_deferred_kernel,
               dim3(grid_for(work, kWavesPerBlock * kFillBatch, 256)),
               block, static_cast<uint64_t *>(cache->rows), backing,
               keys_sorted, segment_starts, counters, i32_at(cw, cl.unique_slots), i32_at(cw, cl.evicted_keys),
               i32_at(cw, cl.landing), i32_at(cw, cl.fetch_source), i32_at(cw, cl.write_out), old_stage_base,
               cache->stage_slots, num_slots);
  } else {
    TBE_LAUNCH("cache_fill", link, cache_fill_kernel, dim3(grid_for(n, kWavesPerBlock, 256 * 16)), block,
               static_cast<uint64_t *>(cache->rows), backing,
               keys_sorted, segment_starts, counters, i32_at(cw, cl.unique_slots), i32_at(cw, cl.evicted_keys));
  }
  return check_launch(name);
}

int commit_step(const char *name, const PlanArgs &a, const tbe_workspace_layout_t &l,
                const tbe_cache_workspace_layout_t &cl, hipStream_t s) {
  const tbe_cache_t *cache = a.cache;
  if (!deferred(cache) || a.num_indices == 0) return TBE_OK;
  void *ws = a.workspace, *cw = a.cache_workspace;
  const int64_t num_slots = cache->num_sets * kWays;
  TBE_LAUNCH("cache_commit", s, cache_commit_kernel, dim3(grid_for(a.num_indices, kWavesPerBlock, 256 * 16)),
             dim3(kBlockThreads), static_cast<uint64_t *>(cache->rows), backing_map(cache, a.D, a.dtype),
             i32_at(ws, l.keys_sorted), i32_at(ws, l.segment_starts), i32_at(ws, l.num_unique),
             i32_at(cw, cl.unique_slots), i32_at(cw, cl.evicted_keys), i32_at(cw, cl.landing),
             i32_at(cw, cl.fetch_source), num_slots + area_of(a.sequence - 2) * cache->stage_slots, cache->stage_slots,
             num_slots);
  return check_launch(name);
}

}  // namespace

int cache_unstage(const tbe_cache_t *cache, int32_t dtype, int32_t D, const int32_t *keys_sorted,
                  const int32_t *segment_starts, const int32_t *counters,
                  const int32_t *unique_slots, int64_t num_indices, hipStream_t stream) {
  if (cache->stage_slots <= 0 || num_indices == 0) return TBE_OK;
  if (cache->stage_of_row) return TBE_OK;  // deferred: a later fill launch (or a flush) writes them back
  TBE_LAUNCH("cache_unstage", stream, cache_unstage_kernel,
             dim3(grid_for(num_indices, kWavesPerBlock, 256 * 16)), dim3(kBlockThreads),
             static_cast<const uint64_t *>(cache->rows), backing_map(cache, D, dtype), keys_sorted, segment_starts, counters, unique_slots,
             cache->num_sets * static_cast<int64_t>(kWays));
  return check_launch("tbe_backward_cached");
}

}  // namespace tbe

extern "C" int tbe_cache_workspace_layout(int64_t num_indices, int64_t num_sets, int64_t stage_slots,
                                          tbe_cache_workspace_layout_t *layout) {
  using namespace tbe;
  TBE_REQUIRE(layout, "tbe_cache_workspace_layout: null layout");
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "tbe_cache_workspace_layout: num_indices out of range");
  TBE_REQUIRE(num_sets > 0 && num_sets * kWays < INT32_MAX, "tbe_cache_workspace_layout: num_sets out of range");
  TBE_REQUIRE(stage_slots >= 0 && stage_slots < INT32_MAX, "tbe_cache_workspace_layout: stage_slots out of range");
  cache_layout(num_indices, num_sets, stage_slots, layout);
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
               dim3(grid_for(kAreas * cache->stage_slots + 1, kBlockThreads, 4096)), block, cache->stage_keys,
               kAreas * cache->stage_slots, -1);
  }
  return check_launch("tbe_cache_init");
}

extern "C" int tbe_cache_plan(const tbe_cache_t *cache, int32_t dtype, int64_t total_rows,
                              int64_t max_table_rows, int32_t D, const int32_t *table_offsets, int32_t T,
                              const int32_t *indices, int64_t num_indices, const int32_t *offsets, int32_t B,
                              int32_t step, int32_t sequence, void *workspace, uint64_t workspace_bytes,
                              void *cache_workspace, uint64_t cache_workspace_bytes, void *plan_stream,
                              void *link_stream) {
  using namespace tbe;
  const char *name = "tbe_cache_plan";
  const PlanArgs a{cache, dtype, total_rows, max_table_rows, D, table_offsets, T, indices, num_indices, offsets, B,
                   step, sequence, workspace, workspace_bytes, cache_workspace, cache_workspace_bytes};
  tbe_workspace_layout_t l;
  tbe_cache_workspace_layout_t cl;
  if (int rc = validate_plan(name, a, &l, &cl)) return rc;
  TBE_REQUIRE(deferred(cache), "%s: planning ahead needs deferred write-back (stage_of_row, stage_slots > 0)", name);
  return plan_step(name, a, l, cl, static_cast<hipStream_t>(plan_stream), static_cast<hipStream_t>(link_stream));
}

extern "C" int tbe_cache_commit(const tbe_cache_t *cache, int32_t dtype, int32_t D, int32_t T,
                                int64_t num_indices, int32_t sequence, void *workspace, uint64_t workspace_bytes,
                                void *cache_workspace, uint64_t cache_workspace_bytes, void *stream) {
  using namespace tbe;
  const char *name = "tbe_cache_commit";
  if (int rc = validate_cache(name, cache)) return rc;
  TBE_REQUIRE(deferred(cache), "%s: needs deferred write-back (stage_of_row, stage_slots > 0)", name);
  TBE_REQUIRE(D > 0 && D % 4 == 0 && T > 0, "%s: bad D or T (got %d, %d)", name, D, T);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(sequence >= 0, "%s: sequence out of range (got %d)", name, sequence);
  tbe_workspace_layout_t l;
  tbe_cache_workspace_layout_t cl;
  backward_layout(num_indices, mixed_tables(cache) ? mixed_layout_dim(dtype) : D, dtype, T, &l);
  cache_layout(num_indices, cache->num_sets, cache->stage_slots, &cl);
  TBE_REQUIRE(workspace && workspace_bytes >= l.total_bytes && cache_workspace &&
                  cache_workspace_bytes >= cl.total_bytes,
              "%s: the workspaces of the plan being committed are missing or too small", name);
  const PlanArgs a{cache, dtype, 0, 0, D, nullptr, T, nullptr, num_indices, nullptr, 0, 0, sequence, workspace,
                   workspace_bytes, cache_workspace, cache_workspace_bytes};
  return commit_step(name, a, l, cl, static_cast<hipStream_t>(stream));
}

extern "C" int tbe_cache_prepare(const tbe_cache_t *cache, int32_t dtype, int64_t total_rows,
                                 int64_t max_table_rows, int32_t D, const int32_t *table_offsets, int32_t T,
                                 const int32_t *indices, int64_t num_indices,
                                 const int32_t *offsets, int32_t B, int32_t step, int32_t sequence, void *workspace,
                                 uint64_t workspace_bytes, void *cache_workspace,
                                 uint64_t cache_workspace_bytes, void *stream, void *side_stream) {
  using namespace tbe;
  const char *name = "tbe_cache_prepare";
  const PlanArgs a{cache, dtype, total_rows, max_table_rows, D, table_offsets, T, indices, num_indices, offsets, B,
                   step, sequence, workspace, workspace_bytes, cache_workspace, cache_workspace_bytes};
  tbe_workspace_layout_t l;
  tbe_cache_workspace_layout_t cl;
  if (int rc = validate_plan(name, a, &l, &cl)) return rc;
  TBE_REQUIRE(stream != side_stream, "%s: side_stream must differ from stream", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  hipStream_t side = static_cast<hipStream_t>(side_stream);
  if (int rc = plan_step(name, a, l, cl, s, side)) return rc;
  // the side stream is joined before anything reads the cached rows
  if (int rc = order_after(name, s, side, 1)) return rc;
  return commit_step(name, a, l, cl, s);
}

extern "C" int tbe_cache_flush(const tbe_cache_t *cache, int32_t dtype, int32_t D, uint32_t live_sequences,
                               int32_t last_sequence, void *stream) {
  using namespace tbe;
  if (int rc = validate_cache("tbe_cache_flush", cache)) return rc;
  TBE_REQUIRE(D > 0 && D % 4 == 0, "tbe_cache_flush: D must be a positive multiple of 4 (got %d)", D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "tbe_cache_flush: bad dtype %d", dtype);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t slots = cache->num_sets * kWays;
  const BackingMap backing = backing_map(cache, D, dtype);
  TBE_REQUIRE(live_sequences <= static_cast<uint32_t>(kAreas), "tbe_cache_flush: at most %d planned batches can be live",
              kAreas);
  if (deferred(cache)) {
    bool keep[kAreas] = {false, false, false};
    for (uint32_t back = 0; back < live_sequences; ++back) keep[area_of(static_cast<int64_t>(last_sequence) - back)] = true;
    for (int64_t area = 0; area < kAreas; ++area) write_back_stage(cache, backing, area, keep[area], s);
  }
  TBE_LAUNCH("cache_flush", s, cache_flush_kernel, dim3(grid_for(slots, kWavesPerBlock, 256 * 16)),
             dim3(kBlockThreads), cache->tags, static_cast<const uint64_t *>(cache->rows), backing, slots);
  return check_launch("tbe_cache_flush");
}
