// Tiles, chunk records and lists of long segments: what the update kernels of uniform tables
// (tbe_update.hip) and of tables of different row widths (tbe_mixed.hip) share.
#pragma once

#include "tbe_common.h"
#include "tbe_stages.h"

namespace tbe {

// The short-segment kernels cut their work by sorted position: a wavefront takes a tile of
// tile_positions() consecutive sorted positions and owns every segment that starts inside it.
// Tile size in sorted positions: 16 per lane group, so narrow rows (many groups per wavefront)
// get larger tiles and the per-tile bookkeeping is amortised over the same number of rows.
// (at most 256 positions; 64 for the variant whose row width is only known at run time.  Measured
// with segments of up to 128 occurrences reduced here: 8 / 16 / 32 / 64 positions per lane group
// take 616 / 605 / 616 / 632 us for 64 tables of fp32 rows of 128 and 206 / 188 / 203 / 203 us for
// 32 tables of fp16 rows of 64 with per-sample weights, 5.2 M lookups each.)
// Small batches (fewer than kSmallBatchTiles such tiles: not enough wavefronts to fill the chip)
// take tiles a quarter that size.
constexpr int kSmallBatchTiles = 4096;
constexpr int tile_positions(int chunks_template, bool small = false) {
  if (chunks_template == 0) return small ? 16 : 64;
  const int positions = (small ? 8 : 16) * (kWave / chunks_template);
  return positions > 256 ? 256 : positions;
}

struct ChunkRecord {   // 32 bytes
  int32_t begin, end;  // sorted positions [begin, end)
  int32_t key;         // row
  int32_t u;           // index of the unique row (for the cache slot table)
  int32_t partial;     // index of the partial row to write, -1 = the chunk is the whole segment
  int32_t pad[3];
};
struct LongRecord {    // 16 bytes: a segment cut into several chunks
  int32_t u, key, begin, end;  // unique-row number, row, sorted positions [begin, end)
};

// The segments of several chunks are listed per XCD (long_records[x][...], lengths in the high word
// of each XCD's counter line).  A wavefront walks the concatenation of the eight lists.
struct LongLists {
  int len[kNumXcd];
  int64_t total;
  int64_t capacity;  // records per list
};
__device__ __forceinline__ LongLists long_lists(const int32_t *__restrict__ counters, int64_t max_long) {
  LongLists l;
  l.total = 0;
  l.capacity = max_long / kNumXcd;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) {
    l.len[x] = counters[xcd_counter(x) + 1];
    l.total += l.len[x];
  }
  return l;
}
__device__ __forceinline__ LongRecord long_record_at(const LongRecord *__restrict__ long_records, const LongLists &l,
                                                     int64_t slot) {
  // (straight-line: a list picked by a run-time index would put the eight lengths into scratch memory)
  int64_t at = 0;
  bool found = false;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) {
    if (!found && slot < l.len[x]) {
      at = x * l.capacity + slot;
      found = true;
    }
    slot -= l.len[x];
  }
  return long_records[at];
}

}  // namespace tbe
