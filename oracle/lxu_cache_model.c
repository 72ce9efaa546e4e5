/*
 * lxu_cache_model.c -- TEST INFRASTRUCTURE, NOT A PRODUCT PATH.
 *
 * Scalar CPU model of the set-associative row cache specified above tbe_cache_t in
 * include/tbe_hip.h.  The reference repository has no cache (its host-resident tables are
 * plain managed / mapped memory, table_batched_embeddings_cuda.cu:795-880), so this model
 * restates this repository's own specification; no reference vectors exist for it.
 * PARITY UNPINNED against the reference.  It is pinned against the specification by
 * tests/test_oracle.py: a brute-force Python model on tiny inputs, invariants (no duplicate
 * tags, residents <= slots, every key resident or flagged uncached, rows used in a step are
 * never evicted in it) and the LRU / LFU textbook behaviour on hand-made traces.
 */
#include <stdint.h>
#include <stdlib.h>

#define WAYS 64

/* lowbias32 hash and multiplicative range reduction; must equal cache_set_of in the library */
uint32_t lxu_set_of(uint32_t key, uint32_t num_sets) {
  uint32_t h = key;
  h ^= h >> 16;
  h *= 0x7feb352du;
  h ^= h >> 15;
  h *= 0x846ca68bu;
  h ^= h >> 16;
  return (uint32_t)(((uint64_t)h * num_sets) >> 32);
}

/*
 * One step over the batch's unique keys (strictly ascending).  policy 0 = LRU, 1 = LFU.
 * Phase 1: every key probes its set; a hit records the slot and marks it used in this step.
 * Phase 2: missing keys, in ascending order, take the slot with the smallest (priority, way)
 *          among slots with last_used < step; none -> the key stays uncached (-1).
 * Outputs per key: unique_slots (slot or -1), evicted_keys (-2 untouched, -1 filled an empty
 * slot, >= 0 key that was written back).  stats[6]: unique, hits, misses, inserted,
 * written back, uncached.
 */
void lxu_cache_step(int32_t *tags, int32_t *last_used, int32_t *use_count, int64_t num_sets,
                    int32_t policy, int32_t step, const int32_t *unique_keys, int64_t U,
                    int32_t *unique_slots, int32_t *evicted_keys, int32_t *stats) {
  for (int k = 0; k < 6; ++k) stats[k] = 0;
  stats[0] = (int32_t)U;
  for (int64_t u = 0; u < U; ++u) {
    const int32_t key = unique_keys[u];
    const int64_t slot0 = (int64_t)lxu_set_of((uint32_t)key, (uint32_t)num_sets) * WAYS;
    unique_slots[u] = -1;
    evicted_keys[u] = -2;
    for (int w = 0; w < WAYS; ++w) {
      if (tags[slot0 + w] == key) {
        unique_slots[u] = (int32_t)(slot0 + w);
        last_used[slot0 + w] = step;
        if (use_count[slot0 + w] != INT32_MAX) ++use_count[slot0 + w];
        break;
      }
    }
    if (unique_slots[u] >= 0) ++stats[1];
    else ++stats[2];
  }
  for (int64_t u = 0; u < U; ++u) {
    if (unique_slots[u] >= 0) continue;
    const int32_t key = unique_keys[u];
    const int64_t slot0 = (int64_t)lxu_set_of((uint32_t)key, (uint32_t)num_sets) * WAYS;
    int victim = -1;
    uint32_t best = 0xffffffffu;
    for (int w = 0; w < WAYS; ++w) {
      if (last_used[slot0 + w] >= step) continue;
      const uint32_t priority = (uint32_t)(policy == 1 ? use_count[slot0 + w] : last_used[slot0 + w]);
      if (priority < best) { /* strict: ties keep the lower way */
        best = priority;
        victim = w;
      }
    }
    if (victim < 0) {
      ++stats[5];
      continue;
    }
    const int32_t old = tags[slot0 + victim];
    evicted_keys[u] = old >= 0 ? old : -1;
    if (old >= 0) ++stats[4];
    ++stats[3];
    tags[slot0 + victim] = key;
    last_used[slot0 + victim] = step;
    use_count[slot0 + victim] = 1;
    unique_slots[u] = (int32_t)(slot0 + victim);
  }
}
