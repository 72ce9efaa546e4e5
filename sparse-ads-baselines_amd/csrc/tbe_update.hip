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
// Work decomposition.  `chunks` lanes (one 16-byte vector each) own a row and a
// wavefront holds 64/chunks such lane groups.  Three classes of segment:
//   short  (<= kShortSegment occurrences)  reduced serially by one lane group inside a
//          position-balanced tile (update_short_kernel);
//   medium (<= kChunkLen)  one wavefront, lane groups split the occurrences, update applied
//          at once (update_chunks_kernel);
//   long   cut into kChunkLen-occurrence chunks reduced by separate wavefronts into partial
//          rows, added in chunk order and applied by update_long_finish_kernel.
// Rows wider than 64 vectors take a multi-pass wavefront-per-segment path.

#include <algorithm>

#include "tbe_queues.h"
#include "tbe_rowwise.h"
#include "tbe_stages.h"

namespace tbe {
namespace {

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
// this lane's vector of the row; `state_old` is *state_row, read by the caller ahead of the
// gradient sum so that its latency is off the row's critical path (unused for SGD).
template <typename T, int VEC, int CHUNKS, int OPT, bool STREAMING = false>
__device__ __forceinline__ void apply_update(T *wrow, const RowVec<T, VEC> &w_old,
                                             const RowVec<T, VEC> &G,
                                             typename AccOf<T>::type *state_row,
                                             typename AccOf<T>::type state_old, float lr,
                                             float eps, int chunks, int group_base, int c,
                                             const StochasticRounding &sr, int64_t element) {
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
    const A s_new = state_old + gss;
    if (c == 0) *state_row = s_new;
    const A mult = adagrad_multiplier<A>(s_new, lr, eps);
#pragma unroll
    for (int i = 0; i < VEC; ++i) w_new.v[i] = w_old.v[i] - G.v[i] * mult;
  }
  store_row<T, VEC, STREAMING>(wrow, w_new, sr, element);
}

// ------------------------------------------------------------ short segments
// Work is cut by sorted position, not by segment: a wavefront takes a tile of tile_positions()
// consecutive sorted positions and owns every segment that STARTS inside it, so each tile costs
// about the same however skewed the keys are.  The tile's bookkeeping is fetched 64 wide into
// LDS (segment bounds, keys, and the gradient row of every occurrence; positions too when
// weighted), after which the only global loads on a segment's critical path are rows.  Lane
// group r walks segments r, r + groups, ...  Segments longer than kShortSegment are not
// reduced here: the owning group appends chunk records (at most kChunkLen occurrences each)
// to a queue that update_chunks_kernel drains with one wavefront per chunk.
// (tile sizes: tile_positions() of tbe_queues.h)

// APPROX (row-wise Adagrad only): the approximate optimizer's per-lookup update
// (batched_embedding_backward_adagrad_approx_kernel_1, tbe.cu:648-704) instead of one update with the
// summed gradient -- every occurrence, in position order, adds its bag's ||grad||^2 (times its
// squared weight) to the state and moves the row by its own multiplier.  Segments longer than
// kApproxShortSegment are then queued as unique-row numbers for tbe_approx.hip's wavefront-per-row kernel.
// APPROX_SUM (with APPROX, rows without per-sample weights in fp32 / fp64): longer segments take the
// chunk queue like the exact update's, for update_chunks_kernel's per-lookup form.
template <typename T, int VEC, int CHUNKS, int OPT, bool WEIGHTED, int UNROLL, bool APPROX = false,
          bool APPROX_SUM = false, bool SMALL = false>
__global__ __launch_bounds__(kBlockThreads) void update_short_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int32_t *__restrict__ keys_sorted,
    const int32_t *__restrict__ positions_sorted, const int32_t *__restrict__ grad_rows,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ segment_ids,
    int32_t *__restrict__ counters, LongRecord *__restrict__ long_records,
    ChunkRecord *__restrict__ chunk_records, int64_t max_chunks, int64_t max_long, int64_t n,
    int64_t num_tiles, int64_t tiles_per_xcd, int D_rt, int chunks_rt, float lr, float eps,
    const int32_t *__restrict__ unique_slots, T *__restrict__ cache_rows, StochasticRounding sr,
    int32_t *__restrict__ approx_long_queue) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  // (a compile-time row width turns every row address into a shift)
  const int D = CHUNKS > 0 ? CHUNKS * VEC : D_rt;
  using R = typename V::R;
  static_assert(!APPROX || OPT == kOptAdagrad, "the approximate update is a row-wise Adagrad");

  constexpr int kTilePositions = tile_positions(CHUNKS, SMALL);
  constexpr int kShort = APPROX ? kApproxShortSegment : kShortSegment;  // longest segment reduced here
  constexpr int kStageCap = kTilePositions + kShort;  // occurrences staged in LDS per wavefront
  __shared__ int32_t s_bounds[kWavesPerBlock][kTilePositions + 1];
  __shared__ int32_t s_keys[kWavesPerBlock][kTilePositions];
  __shared__ int32_t s_grow[kWavesPerBlock][kStageCap];
  __shared__ int32_t s_pos[WEIGHTED ? kWavesPerBlock : 1][WEIGHTED ? kStageCap : 1];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  const int64_t tile = xcd_contiguous(blockIdx.x, tiles_per_xcd) * kWavesPerBlock + wave;
  if (tile >= num_tiles) return;
  // The workgroups of an XCD walk one eighth of the sorted positions in order, so the chunk
  // records they queue are in (table, row) order: each XCD keeps its own queue, which
  // update_chunks_kernel drains on the same XCD in that order (the gradient rows of a table then
  // stay in that XCD's L2 while its hot rows are reduced).
  const int xcd = blockIdx.x % kNumXcd;
  ChunkRecord *chunk_queue = chunk_records + xcd * (max_chunks / kNumXcd);
  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const int group_base = r * chunks;
  const int64_t col = static_cast<int64_t>(c) * VEC;

  // Segments that start in [p0, p1): the segment containing p0 belongs to this tile only if
  // p0 is its head, i.e. if the position before it lies in another segment.  Three segment
  // numbers, fetched together, say it all: a tile inside one long row (most tiles of a skewed
  // batch) is done after one round trip.
  const int64_t p0 = tile * kTilePositions;
  const int64_t p1 = min(n, p0 + kTilePositions);
  const int id_before = segment_ids[max(p0 - 1, int64_t{0})];
  const int id0 = segment_ids[p0];
  const int id_last = segment_ids[p1 - 1];
  const int u_first = id0 + ((p0 > 0 && id_before == id0) ? 1 : 0);
  const int u_limit = id_last + 1;
  const int nseg = u_limit - u_first;  // <= kTilePositions
  if (nseg <= 0) return;

  // Bookkeeping into LDS.  All loads of one level are issued before the first dependent load:
  // the segment bounds, then -- both only need the bounds -- the keys and the tile's sorted
  // positions, then the gradient row of every position.  Three memory round trips however many
  // positions the tile holds.  (The first and the last bound reach all lanes by lane shuffles, not
  // through LDS, so that the positions are requested together with the keys.)
  constexpr int kBoundIters = (kTilePositions + 1 + kWave - 1) / kWave;
  constexpr int kStageIters = (kStageCap + kWave - 1) / kWave;
  int sb[kBoundIters];
#pragma unroll
  for (int q = 0; q < kBoundIters; ++q) {
    const int k = q * kWave + lane;
    sb[q] = segment_starts[u_first + min(k, nseg)];  // clamped, not predicated: no branch per load
  }
  const int tile_begin = shfl_idx(sb[0], 0);
  int tile_end = 0;  // bound number nseg: where the tile's last segment ends
#pragma unroll
  for (int q = 0; q < kBoundIters; ++q) {
    const int v = shfl_idx(sb[q], nseg & (kWave - 1));
    if (q == (nseg >> 6)) tile_end = v;
  }
  const int staged = min(tile_end - tile_begin, kStageCap);
  {
    int kv[kBoundIters];
#pragma unroll
    for (int q = 0; q < kBoundIters; ++q) kv[q] = keys_sorted[min(static_cast<int64_t>(sb[q]), n - 1)];
    int pos[kStageIters], grow[kStageIters];
#pragma unroll
    for (int q = 0; q < kStageIters; ++q) {
      const int i = q * kWave + lane;
      pos[q] = positions_sorted[tile_begin + min(i, staged - 1)];
    }
#pragma unroll
    for (int q = 0; q < kBoundIters; ++q) {
      const int k = q * kWave + lane;
      if (k <= nseg) s_bounds[wave][k] = sb[q];
      if (k < nseg) s_keys[wave][k] = kv[q];
    }
#pragma unroll
    for (int q = 0; q < kStageIters; ++q) grow[q] = grad_rows[pos[q]];
#pragma unroll
    for (int q = 0; q < kStageIters; ++q) {
      const int i = q * kWave + lane;
      if (i < staged) {
        s_grow[wave][i] = grow[q];
        if constexpr (WEIGHTED) s_pos[wave][i] = pos[q];
      }
    }
  }
  __builtin_amdgcn_wave_barrier();

  for (int j = (r < groups) ? r : nseg; j < nseg; j += groups) {
    const int u = u_first + j;
    const int seg_begin = s_bounds[wave][j];
    const int seg_end = s_bounds[wave][j + 1];
    const int len = seg_end - seg_begin;
    const int32_t key = s_keys[wave][j];
    if constexpr (APPROX && !APPROX_SUM) {
      if (len > kShort) {
        // (one queue per XCD, like the chunk records: `max_chunks` is the room of all eight)
        // and one behind them for the rows of very many occurrences
        if (c == 0) {
          if (len > kApproxHuge) approx_long_queue[max_chunks + atomicAdd(&counters[1], 1)] = u;
          else approx_long_queue[xcd * (max_chunks / kNumXcd) + atomicAdd(&counters[xcd_counter(xcd)], 1)] = u;
        }
        continue;
      }
    }
    if (len > kShort) {
      // Hand the segment to the chunk queue.
      const int nch = (len + kChunkLen - 1) / kChunkLen;
      int first_chunk = 0;
      if (c == 0) {
        // one atomic add on the XCD's own line: its low word hands out the queue slots, its high
        // word the place in the XCD's list of segments of several chunks
        const unsigned long long taken = atomicAdd(
            reinterpret_cast<unsigned long long *>(counters + xcd_counter(xcd)),
            static_cast<unsigned long long>(nch) | (nch > 1 ? 1ull << 32 : 0ull));
        first_chunk = static_cast<int>(taken & 0xffffffffull);
        if (nch > 1)
          long_records[xcd * (max_long / kNumXcd) + static_cast<int64_t>(taken >> 32)] =
              LongRecord{u, key, seg_begin, seg_end};
      }
      first_chunk = shfl_idx(first_chunk, group_base);
      for (int k = c; k < nch; k += chunks) {
        ChunkRecord rec;
        rec.begin = seg_begin + k * kChunkLen;
        rec.end = min(seg_end, rec.begin + kChunkLen);
        rec.key = key;
        rec.u = u;
        rec.partial = nch > 1 ? partial_row_of_chunk(seg_begin, seg_end, k, nch) : -1;
        rec.pad[0] = rec.pad[1] = rec.pad[2] = 0;
        chunk_queue[first_chunk + k] = rec;
      }
      continue;
    }
    T *wrow = resolve_row(weights, cache_rows, unique_slots, u, static_cast<int64_t>(key), D) + col;
    // each row is touched once per step: streaming accesses keep L2 for gradient rows.  The
    // row is requested right after the first gradient rows and stays packed until it is used,
    // so that converting it (fp16) does not put its latency in front of theirs.
    R w_raw;
    A state_old = A(0);
    V w_old;
    V G;
    G.zero();
    for (int i0 = seg_begin; i0 < seg_end; i0 += UNROLL) {
      R raw[UNROLL];
      int pos[UNROLL];
      T pw_raw[UNROLL];
#pragma unroll
      for (int q = 0; q < UNROLL; ++q) {
        const int i = i0 + q;
        if (i < seg_end) {
          // a short segment starts inside the tile and has at most kShort occurrences,
          // so all of them are among the staged ones
          const int rel = i - tile_begin;
          const int64_t grow = s_grow[wave][rel];
          if constexpr (WEIGHTED) pos[q] = s_pos[wave][rel];
          raw[q] = V::load_raw(grad_output + grow * D + col);
          if constexpr (WEIGHTED) pw_raw[q] = psw[pos[q]];
        }
      }
      if (i0 == seg_begin) {  // requested after the first gradient rows, see above
        w_raw = V::load_raw_streaming(wrow);
        if constexpr (OPT == kOptAdagrad) state_old = state[key];
      }
      if constexpr (APPROX) {
        // w_old is the row as the occurrences so far have left it, state_old the running state
        if (i0 == seg_begin) w_old.unpack(w_raw);
#pragma unroll
        for (int q = 0; q < UNROLL; ++q) {
          if (i0 + q < seg_end) {
            V x;
            x.unpack(raw[q]);
            A local = A(0);
#pragma unroll
            for (int i = 0; i < VEC; ++i) local += x.v[i] * x.v[i];
            const A gss = group_sum<CHUNKS, A>(local, chunks, group_base);
            A pw = A(1);
            if constexpr (WEIGHTED) pw = to_acc(pw_raw[q]);
            state_old = state_old + (WEIGHTED ? gss * pw * pw : gss);
            const A mult = approx_multiplier<A>(state_old, pw, WEIGHTED, lr, eps);
            if constexpr (WEIGHTED) {
              A dot = lane_dot<VEC, A>(w_old.v, x.v);
              dot = group_sum<CHUNKS, A>(dot, chunks, group_base);
              if (c == 0) grad_psw[pos[q]] = from_acc<T, A>(dot);
            }
#pragma unroll
            for (int i = 0; i < VEC; ++i) w_old.v[i] = w_old.v[i] - x.v[i] * mult;
            round_trip<T, VEC>(w_old, rounding_of_update(sr, i0 + q - seg_begin), static_cast<int64_t>(key) * D + col);
          }
        }
        continue;
      }
      if constexpr (WEIGHTED) w_old.unpack(w_raw);
#pragma unroll
      for (int q = 0; q < UNROLL; ++q) {
        if (i0 + q < seg_end) {
          V x;
          x.unpack(raw[q]);
          if constexpr (WEIGHTED) {
            const A pw = opaque(to_acc(pw_raw[q]));  // converted once; the gradient's conversions fold into the sums
            A dot = lane_dot<VEC, A>(w_old.v, x.v);
            dot = group_sum<CHUNKS, A>(dot, chunks, group_base);
            if (c == 0) grad_psw[pos[q]] = from_acc<T, A>(dot);
#pragma unroll
            for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * pw;
          } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i];
          }
        }
      }
    }
    if constexpr (APPROX) {
      // (fp16: the last update already rounded the row to the stored type, this conversion is exact)
      if (c == 0) state[key] = state_old;
      w_old.store_streaming(wrow);
      continue;
    }
    w_old.unpack(w_raw);
    apply_update<T, VEC, CHUNKS, OPT, true>(wrow, w_old, G, state ? state + key : nullptr, state_old, lr,
                                            eps, chunks, group_base, c, sr,
                                            static_cast<int64_t>(key) * D + col);
  }
}

// ------------------------------------------------ medium / long segments: chunks
// One wavefront per chunk record.  The wavefronts of an XCD take the records of that XCD's
// queue, consecutive records at the same time (see below for queues of unequal length).  Lane
// group r adds occurrences r, r + groups, ... of the chunk; the groups are combined in a fixed
// tree.
// A chunk that is a whole segment is applied to its row at once; a chunk of a longer
// segment stores its sum as a partial row for update_long_finish_kernel.
// APPROX (instantiated as SGD without per-sample weights, fp32 / fp64 rows): the approximate
// Adagrad of a row without per-sample weights is row_0 - sum_k mult_k * g_k with
// mult_k = lr / (sqrt(state_0 + sum_{j<=k} wss_j) + eps), so its long rows are summed in chunks like
// the exact update's.  `psw` then holds wss of every lookup by position (approx_lookup_norms_kernel);
// a chunk adds up the addends of the row's earlier occurrences, forms the multipliers of its own
// 64 at a time (a wavefront prefix sum) and adds mult * g.  A chunk that is a whole segment writes
// the row and its state; the state of a row of several chunks is left to approx_long_state_kernel
// (every chunk of the row reads the old one).
template <typename T, int VEC, int CHUNKS, int OPT, bool WEIGHTED, int UNROLL, bool APPROX = false>
__global__ __launch_bounds__(kBlockThreads) void update_chunks_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw,
    T *__restrict__ grad_psw, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ counters,
    const ChunkRecord *__restrict__ chunk_records, int64_t max_chunks,
    typename AccOf<T>::type *__restrict__ partial_sums, int D_rt, int chunks_rt, float lr, float eps,
    const int32_t *__restrict__ unique_slots, T *__restrict__ cache_rows, StochasticRounding sr,
    const int32_t *__restrict__ segment_starts) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  // (a compile-time row width turns every row address into a shift)
  const int D = CHUNKS > 0 ? CHUNKS * VEC : D_rt;
  using R = typename V::R;
  static_assert(!APPROX || (OPT == kOptSgd && !WEIGHTED && sizeof(T) == sizeof(A)),
                "the per-lookup form sums fp32 / fp64 rows without per-sample weights");

  const int lane = threadIdx.x & (kWave - 1);
  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const int group_base = r * chunks;
  const bool active = r < groups;
  const int64_t col = static_cast<int64_t>(c) * VEC;
  // An XCD drains its own queue up to one and a half times the average queue length; what the
  // longer queues hold beyond that is dealt to the wavefronts of all XCDs, so that a batch whose
  // hot rows sit in one table still uses the whole machine.  All of it is index arithmetic on
  // the eight queue lengths: no wavefront waits for another.
  const int xcd = blockIdx.x % kNumXcd;
  const int64_t queue_capacity = max_chunks / kNumXcd;
  int queue_len[kNumXcd];
  int64_t total = 0;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) {
    queue_len[x] = counters[xcd_counter(x)];
    total += queue_len[x];
  }
  const int fair = static_cast<int>(total / kNumXcd + total / 16 + 1);
  int64_t shared_total = 0;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) shared_total += max(0, queue_len[x] - fair);
  const int own = min(queue_len[xcd], fair);
  int64_t q = static_cast<int64_t>(blockIdx.x / kNumXcd) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x / kNumXcd) * kWavesPerBlock;
  int64_t g = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t shared_stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;

  while (true) {
    const ChunkRecord *next;
    if (q < own) {
      next = chunk_records + xcd * queue_capacity + q;
      q += stride;
    } else if (g < shared_total) {
      int64_t before = 0;
      int x = 0;
      while (g >= before + max(0, queue_len[x] - fair)) {
        before += max(0, queue_len[x] - fair);
        ++x;
      }
      next = chunk_records + x * queue_capacity + fair + (g - before);
      g += shared_stride;
    } else {
      break;
    }
    const ChunkRecord rec = *next;
    T *wrow = resolve_row(weights, cache_rows, unique_slots, rec.u, static_cast<int64_t>(rec.key), D) + col;
    V w_old;
    w_old.zero();
    if (active && (WEIGHTED || rec.partial < 0)) w_old.load(wrow);
    A state_old = A(0);
    if constexpr (OPT == kOptAdagrad) {
      if (rec.partial < 0) state_old = state[rec.key];
    }
    V G;
    G.zero();
    // APPROX: the row's state before the chunk's first occurrence
    A running = A(0);
    if constexpr (APPROX) {
      constexpr int kAhead = 16;
      const int seg_begin = segment_starts[rec.u];
      A earlier = A(0);
      for (int i0 = seg_begin; i0 < rec.begin; i0 += kAhead * kWave) {
        int p[kAhead];
        A x[kAhead];
#pragma unroll
        for (int k = 0; k < kAhead; ++k) p[k] = positions_sorted[min(i0 + k * kWave + lane, rec.begin - 1)];
#pragma unroll
        for (int k = 0; k < kAhead; ++k) x[k] = to_acc(psw[p[k]]);
#pragma unroll
        for (int k = 0; k < kAhead; ++k) earlier += (i0 + k * kWave + lane < rec.begin) ? x[k] : A(0);
      }
#pragma unroll
      for (int m = kWave / 2; m > 0; m >>= 1) earlier += shfl_x(earlier, m);
      running = state[rec.key] + earlier;
    }
    // The positions of a 64-position batch are requested two batches ahead, its gradient row ids
    // and weights one batch ahead (lanes past the chunk's end ask for its first position: any
    // valid index will do), so a batch waits for gradient rows only.
    auto position_at = [&](int64_t i) { return positions_sorted[i < rec.end ? i : rec.begin]; };
    int pos_now = position_at(static_cast<int64_t>(rec.begin) + lane);
    int pos_next = position_at(static_cast<int64_t>(rec.begin) + kWave + lane);
    int grow_now = grad_rows[pos_now];
    A w_now = A(0);
    if constexpr (WEIGHTED || APPROX) w_now = to_acc(psw[pos_now]);
    for (int base = rec.begin; base < rec.end; base += kWave) {
      const int n = min(kWave, rec.end - base);
      const int my_pos = pos_now, my_grow = grow_now;
      A my_w = w_now;
      pos_now = pos_next;
      pos_next = position_at(static_cast<int64_t>(base) + 2 * kWave + lane);
      grow_now = grad_rows[pos_now];
      if constexpr (WEIGHTED || APPROX) w_now = to_acc(psw[pos_now]);
      if constexpr (APPROX) {
        // lane j holds occurrence base + j: its state is the running one plus the addends up to it
        const A incl = wave_inclusive_sum<A>(lane < n ? my_w : A(0));
        my_w = lane < n ? approx_multiplier<A>(running + incl, A(1), false, lr, eps) : A(0);
        running = running + shfl_idx(incl, n - 1);
      }
      // Straight-line code: every lane loads (a lane without an occurrence loads what occurrence
      // 0 loads and drops it), so that the UNROLL loads of a step are issued back to back.
      for (int j0 = 0; j0 < n; j0 += groups * UNROLL) {
        R raw[UNROLL];
        bool ok[UNROLL];
        int src[UNROLL];
#pragma unroll
        for (int k = 0; k < UNROLL; ++k) {
          const int j = j0 + k * groups + r;
          ok[k] = active && j < n;
          src[k] = j < n ? j : 0;
        }
#pragma unroll
        for (int k = 0; k < UNROLL; ++k) {
          const int64_t grow = shfl_idx(my_grow, src[k]);
          raw[k] = V::load_raw(grad_output + grow * D + col);
        }
#pragma unroll
        for (int k = 0; k < UNROLL; ++k) {
          A pw = A(0);
          int pos = 0;
          if constexpr (WEIGHTED) {
            pw = shfl_idx(my_w, src[k]);
            pos = shfl_idx(my_pos, src[k]);
          }
          if constexpr (APPROX) pw = shfl_idx(my_w, src[k]);
          keep_if(raw[k], ok[k]);
          V x;
          x.unpack(raw[k]);
          if constexpr (APPROX) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * pw;
          } else if constexpr (WEIGHTED) {
            A dot = lane_dot<VEC, A>(w_old.v, x.v);
            dot = group_sum<CHUNKS, A>(dot, chunks, group_base);
            if (ok[k] && c == 0) grad_psw[pos] = from_acc<T, A>(dot);
#pragma unroll
            for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i] * pw;
          } else {
#pragma unroll
            for (int i = 0; i < VEC; ++i) G.v[i] += x.v[i];
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
      if (rec.partial >= 0) {
        A *dst = partial_sums + static_cast<int64_t>(rec.partial) * D + col;
#pragma unroll
        for (int i = 0; i < VEC; ++i) dst[i] = G.v[i];
      } else if constexpr (APPROX) {
        V w_new;
#pragma unroll
        for (int i = 0; i < VEC; ++i) w_new.v[i] = w_old.v[i] - G.v[i];
        w_new.store(wrow);
        if (c == 0) state[rec.key] = running;
      } else {
        apply_update<T, VEC, CHUNKS, OPT>(wrow, w_old, G, state ? state + rec.key : nullptr, state_old,
                                          lr, eps, chunks, 0, c, sr,
                                          static_cast<int64_t>(rec.key) * D + col);
      }
    }
  }
}

// The approximate Adagrad's rows that were summed in several chunks: their state takes the addends
// of all their lookups (one wavefront per row; update_long_finish_kernel writes the row itself).
template <typename A>
__global__ __launch_bounds__(kBlockThreads) void approx_long_state_kernel(
    A *__restrict__ state, const A *__restrict__ lookup_wss, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ segment_starts, const int32_t *__restrict__ counters,
    const LongRecord *__restrict__ long_records, int64_t max_long) {
  constexpr int kAhead = 16;
  const int lane = threadIdx.x & (kWave - 1);
  const LongLists lists = long_lists(counters, max_long);
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  for (int64_t slot = wave_id; slot < lists.total; slot += stride) {
    const LongRecord rec = long_record_at(long_records, lists, slot);
    const int seg_begin = rec.begin;
    const int seg_end = rec.end;
    A sum = A(0);
    for (int i0 = seg_begin; i0 < seg_end; i0 += kAhead * kWave) {
      int p[kAhead];
      A x[kAhead];
#pragma unroll
      for (int k = 0; k < kAhead; ++k) p[k] = positions_sorted[min(i0 + k * kWave + lane, seg_end - 1)];
#pragma unroll
      for (int k = 0; k < kAhead; ++k) x[k] = lookup_wss[p[k]];
#pragma unroll
      for (int k = 0; k < kAhead; ++k) sum += (i0 + k * kWave + lane < seg_end) ? x[k] : A(0);
    }
#pragma unroll
    for (int m = kWave / 2; m > 0; m >>= 1) sum += shfl_x(sum, m);
    if (lane == 0) state[rec.key] += sum;
  }
}

// --------------------------------------------- long segments: combine + update
// One wavefront per long row: lane group r adds partial rows r, r + groups, ..., the groups are
// combined in a fixed tree and group 0 applies the update.
template <typename T, int VEC, int CHUNKS, int OPT>
__global__ __launch_bounds__(kBlockThreads) void update_long_finish_kernel(
    T *__restrict__ weights, typename AccOf<T>::type *__restrict__ state,
    const int32_t *__restrict__ counters, const LongRecord *__restrict__ long_records,
    const typename AccOf<T>::type *__restrict__ partial_sums, int D_rt, int chunks_rt, float lr,
    float eps, const int32_t *__restrict__ unique_slots, T *__restrict__ cache_rows,
    StochasticRounding sr, int64_t max_long) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  // (a compile-time row width turns every row address into a shift)
  const int D = CHUNKS > 0 ? CHUNKS * VEC : D_rt;

  const int lane = threadIdx.x & (kWave - 1);
  const int chunks = CHUNKS > 0 ? CHUNKS : chunks_rt;
  const int groups = kWave / chunks;
  const int r = lane / chunks;
  const int c = lane - r * chunks;
  const bool active = r < groups;
  const LongLists lists = long_lists(counters, max_long);
  const int64_t col = static_cast<int64_t>(c) * VEC;
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;

  for (int64_t slot = wave_id; slot < lists.total; slot += stride) {
    const LongRecord rec = long_record_at(long_records, lists, slot);
    const int num_chunks = (rec.end - rec.begin + kChunkLen - 1) / kChunkLen;
    T *wrow = resolve_row(weights, cache_rows, unique_slots, rec.u, static_cast<int64_t>(rec.key), D) + col;
    V w_old;
    w_old.zero();
    if (r == 0) w_old.load(wrow);
    A state_old = A(0);
    if constexpr (OPT == kOptAdagrad) state_old = state[rec.key];
    V G;
    G.zero();
    if (active) {
      // eight partial rows are requested before the first is added (same order of additions)
      constexpr int kAhead = 8;
      for (int k0 = r; k0 < num_chunks; k0 += groups * kAhead) {
        A part[kAhead][VEC];
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
          const int k = min(k0 + a * groups, num_chunks - 1);  // clamped: no branch per load
          const A *src =
              partial_sums + static_cast<int64_t>(partial_row_of_chunk(rec.begin, rec.end, k, num_chunks)) * D + col;
#pragma unroll
          for (int i = 0; i < VEC; ++i) part[a][i] = src[i];
        }
#pragma unroll
        for (int a = 0; a < kAhead; ++a) {
          const bool real = k0 + a * groups < num_chunks;
#pragma unroll
          for (int i = 0; i < VEC; ++i) G.v[i] += real ? part[a][i] : A(0);
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
      apply_update<T, VEC, CHUNKS, OPT>(wrow, w_old, G, state ? state + rec.key : nullptr, state_old, lr,
                                        eps, chunks, 0, c, sr, static_cast<int64_t>(rec.key) * D + col);
    }
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
    T *__restrict__ cache_rows, StochasticRounding sr) {
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
      store_row<T, VEC, false>(wrow + static_cast<int64_t>(cb) * VEC, w, sr, row * D + static_cast<int64_t>(cb) * VEC);
    }
  }
}

constexpr int kShortUnroll = 4;
constexpr int kLongUnroll = 8;  // 4 for weighted 8-element fp16 vectors: registers, hence occupancy

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
  LongRecord *long_records = reinterpret_cast<LongRecord *>(a.long_segments);
  ChunkRecord *chunk_records = reinterpret_cast<ChunkRecord *>(a.chunk_segments);
  const int groups = kWave / g.chunks;
  const dim3 block(kBlockThreads);

  const bool small = ceil_div(a.num_indices, tile_positions(CHUNKS)) < kSmallBatchTiles;
  const int64_t num_tiles = ceil_div(a.num_indices, tile_positions(CHUNKS, small));
  const int64_t tiles_per_xcd = ceil_div(ceil_div(num_tiles, kWavesPerBlock), kNumXcd);
  const dim3 grid_short(static_cast<unsigned>(tiles_per_xcd * kNumXcd));
#define TBE_UPDATE_SHORT(SMALL)                                                                             \
  TBE_LAUNCH("update_short", stream,                                                                        \
             (update_short_kernel<T, VEC, CHUNKS, OPT, WEIGHTED, kShortUnroll, false, false, SMALL>),       \
             grid_short, block, go, w, st, psw, gpsw, a.keys_sorted, a.positions_sorted, a.grad_rows,       \
             a.segment_starts, a.segment_ids, a.counters, long_records, chunk_records, a.max_chunks,        \
             a.max_long, a.num_indices, num_tiles, tiles_per_xcd, a.D, g.chunks, a.learning_rate, a.eps,                \
             a.unique_slots, cr, a.stochastic_rounding, static_cast<int32_t *>(nullptr))
  if (small) { TBE_UPDATE_SHORT(true); }
  else { TBE_UPDATE_SHORT(false); }
#undef TBE_UPDATE_SHORT

  const int64_t want_chunks = ceil_div(a.max_chunks, kWavesPerBlock);
  // a multiple of the XCD count, so that every XCD gets as many workgroups (a small batch, whose
  // queues are mostly empty room, gets few: starting workgroups that find nothing is its cost)
  const dim3 grid_chunks(static_cast<unsigned>(
      kNumXcd * std::max<int64_t>(1, std::min<int64_t>(ceil_div(want_chunks, kNumXcd), small ? 64 : 1024))));
  TBE_LAUNCH("update_chunks", stream,
             (update_chunks_kernel<T, VEC, CHUNKS, OPT, WEIGHTED, (WEIGHTED && VEC == 8) ? 4 : kLongUnroll>),
             grid_chunks, block,
             go, w, st, psw, gpsw, a.positions_sorted, a.grad_rows, a.counters, chunk_records,
             a.max_chunks, partial, a.D, g.chunks, a.learning_rate, a.eps, a.unique_slots, cr,
             a.stochastic_rounding, static_cast<const int32_t *>(nullptr));

  const int64_t want_long = ceil_div(a.max_long, kWavesPerBlock);
  const dim3 grid_finish(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_long, 256 * 4))));
  TBE_LAUNCH("update_long_finish", stream, (update_long_finish_kernel<T, VEC, CHUNKS, OPT>),
             grid_finish, block, w, st, a.counters, long_records, partial, a.D, g.chunks,
             a.learning_rate, a.eps, a.unique_slots, cr, a.stochastic_rounding, a.max_long);
}

// The short-row kernel alone, in its per-lookup (approximate Adagrad) form; rows of more than
// kApproxShortSegment occurrences are left in `queue`: eight queues of approx_long_queue_capacity() row
// numbers, one per XCD, their lengths in counters[xcd_counter(x)].
template <typename T, int VEC, int CHUNKS, bool WEIGHTED>
void launch_approx_short(const UpdateArgs &a, const RowGeometry &g, int32_t *queue, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  const bool small = ceil_div(a.num_indices, tile_positions(CHUNKS)) < kSmallBatchTiles;
  const int64_t num_tiles = ceil_div(a.num_indices, tile_positions(CHUNKS, small));
  const int64_t tiles_per_xcd = ceil_div(ceil_div(num_tiles, kWavesPerBlock), kNumXcd);
  const dim3 grid_short(static_cast<unsigned>(tiles_per_xcd * kNumXcd));
  if constexpr (!WEIGHTED && sizeof(T) == sizeof(A)) {
    if (queue == nullptr) {
      // fp32 / fp64 rows without per-sample weights: longer rows go to the chunk queues
#define TBE_APPROX_SUM_SHORT(SMALL)                                                                             \
  TBE_LAUNCH("update_approx_short", stream,                                                                     \
             (update_short_kernel<T, VEC, CHUNKS, kOptAdagrad, false, kShortUnroll, true, true, SMALL>),        \
             grid_short, dim3(kBlockThreads), static_cast<const T *>(a.grad_output),                            \
             static_cast<T *>(a.weights), static_cast<A *>(a.optimizer_state), static_cast<const T *>(nullptr), \
             static_cast<T *>(nullptr), a.keys_sorted, a.positions_sorted, a.grad_rows, a.segment_starts,       \
             a.segment_ids, a.counters, reinterpret_cast<LongRecord *>(a.long_segments),                        \
             reinterpret_cast<ChunkRecord *>(a.chunk_segments), a.max_chunks, a.max_long, a.num_indices,        \
             num_tiles,                                                                                         \
             tiles_per_xcd, a.D, g.chunks, a.learning_rate, a.eps, a.unique_slots,                              \
             static_cast<T *>(a.cache_rows), a.stochastic_rounding, static_cast<int32_t *>(nullptr))
      if (small) { TBE_APPROX_SUM_SHORT(true); }
      else { TBE_APPROX_SUM_SHORT(false); }
#undef TBE_APPROX_SUM_SHORT
      return;
    }
  }
#define TBE_APPROX_SHORT(SMALL)                                                                                 \
  TBE_LAUNCH("update_approx_short", stream,                                                                     \
             (update_short_kernel<T, VEC, CHUNKS, kOptAdagrad, WEIGHTED, kShortUnroll, true, false, SMALL>),    \
             grid_short, dim3(kBlockThreads), static_cast<const T *>(a.grad_output),                            \
             static_cast<T *>(a.weights), static_cast<A *>(a.optimizer_state),                                  \
             static_cast<const T *>(a.per_sample_weights), static_cast<T *>(a.grad_per_sample_weights),         \
             a.keys_sorted, a.positions_sorted, a.grad_rows, a.segment_starts, a.segment_ids, a.counters,       \
             static_cast<LongRecord *>(nullptr), static_cast<ChunkRecord *>(nullptr),                           \
             kNumXcd * approx_long_queue_capacity(a.num_indices), int64_t{0}, a.num_indices, num_tiles,         \
             tiles_per_xcd,                                                                                     \
             a.D, g.chunks, a.learning_rate, a.eps, a.unique_slots, static_cast<T *>(a.cache_rows),             \
             a.stochastic_rounding, queue)
  if (small) { TBE_APPROX_SHORT(true); }
  else { TBE_APPROX_SHORT(false); }
#undef TBE_APPROX_SHORT
}

template <typename T, int VEC, bool WEIGHTED>
void launch_approx_short_geometry(const UpdateArgs &a, const RowGeometry &g, int32_t *queue, hipStream_t stream) {
  switch (g.tmpl) {
    case 64: launch_approx_short<T, VEC, 64, WEIGHTED>(a, g, queue, stream); break;
    case 32: launch_approx_short<T, VEC, 32, WEIGHTED>(a, g, queue, stream); break;
    case 16: launch_approx_short<T, VEC, 16, WEIGHTED>(a, g, queue, stream); break;
    case 8: launch_approx_short<T, VEC, 8, WEIGHTED>(a, g, queue, stream); break;
    case 4: launch_approx_short<T, VEC, 4, WEIGHTED>(a, g, queue, stream); break;
    default: launch_approx_short<T, VEC, 0, WEIGHTED>(a, g, queue, stream); break;
  }
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
               a.unique_slots, static_cast<T *>(a.cache_rows), a.stochastic_rounding);
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

bool approx_short_serves(int32_t dtype, int32_t D) { return !row_geometry(dtype, D).wide; }

int segment_update_approx_short(const UpdateArgs &a, int32_t *queue, hipStream_t stream) {
  if (a.num_indices == 0) return TBE_OK;
  const RowGeometry g = row_geometry(a.dtype, a.D);
  const bool weighted = a.per_sample_weights != nullptr;
#define TBE_APPROX_SHORT(TYPE, VECTOR)                                                        \
  do {                                                                                       \
    if (weighted) launch_approx_short_geometry<TYPE, VECTOR, true>(a, g, queue, stream);     \
    else launch_approx_short_geometry<TYPE, VECTOR, false>(a, g, queue, stream);             \
  } while (0)
  switch (a.dtype) {
    case TBE_DTYPE_F32: TBE_APPROX_SHORT(float, 4); break;
    case TBE_DTYPE_F16:
      if (g.vec == 8) TBE_APPROX_SHORT(__half, 8);
      else TBE_APPROX_SHORT(__half, 4);
      break;
    default: TBE_APPROX_SHORT(double, 2); break;
  }
#undef TBE_APPROX_SHORT
  return check_launch("tbe approximate Adagrad update (short rows)");
}

namespace {
template <typename T, int VEC, int CHUNKS>
void launch_approx_sum_long(const UpdateArgs &a, const RowGeometry &g, const void *lookup_wss, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  if constexpr (sizeof(T) == sizeof(A)) {
    T *w = static_cast<T *>(a.weights);
    A *st = static_cast<A *>(a.optimizer_state);
    A *partial = static_cast<A *>(a.partial_sums);
    LongRecord *long_records = reinterpret_cast<LongRecord *>(a.long_segments);
    ChunkRecord *chunk_records = reinterpret_cast<ChunkRecord *>(a.chunk_segments);
    const dim3 block(kBlockThreads);
    const int64_t want_chunks = ceil_div(a.max_chunks, kWavesPerBlock);
    const bool small = ceil_div(a.num_indices, tile_positions(CHUNKS)) < kSmallBatchTiles;
    const dim3 grid_chunks(static_cast<unsigned>(
        kNumXcd * std::max<int64_t>(1, std::min<int64_t>(ceil_div(want_chunks, kNumXcd), small ? 64 : 1024))));
    TBE_LAUNCH("update_approx_chunks", stream,
               (update_chunks_kernel<T, VEC, CHUNKS, kOptSgd, false, kLongUnroll, true>), grid_chunks, block,
               static_cast<const T *>(a.grad_output), w, st, static_cast<const T *>(lookup_wss),
               static_cast<T *>(nullptr), a.positions_sorted, a.grad_rows, a.counters, chunk_records, a.max_chunks,
               partial, a.D, g.chunks, a.learning_rate, a.eps, a.unique_slots, static_cast<T *>(a.cache_rows),
               a.stochastic_rounding, a.segment_starts);
    const int64_t want_long = ceil_div(a.max_long, kWavesPerBlock);
    const dim3 grid_finish(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want_long, 256 * 4))));
    // (the partial rows already carry the multipliers: the row takes their sum as it is)
    TBE_LAUNCH("update_long_finish", stream, (update_long_finish_kernel<T, VEC, CHUNKS, kOptSgd>), grid_finish,
               block, w, st, a.counters, long_records, partial, a.D, g.chunks, 1.0f, a.eps, a.unique_slots,
               static_cast<T *>(a.cache_rows), a.stochastic_rounding, a.max_long);
    TBE_LAUNCH("update_approx_state", stream, (approx_long_state_kernel<A>), grid_finish, block, st,
               static_cast<const A *>(lookup_wss), a.positions_sorted, a.segment_starts, a.counters, long_records,
               a.max_long);
  }
}

template <typename T, int VEC>
void launch_approx_sum_long_geometry(const UpdateArgs &a, const RowGeometry &g, const void *wss, hipStream_t stream) {
  switch (g.tmpl) {
    case 64: launch_approx_sum_long<T, VEC, 64>(a, g, wss, stream); break;
    case 32: launch_approx_sum_long<T, VEC, 32>(a, g, wss, stream); break;
    case 16: launch_approx_sum_long<T, VEC, 16>(a, g, wss, stream); break;
    case 8: launch_approx_sum_long<T, VEC, 8>(a, g, wss, stream); break;
    case 4: launch_approx_sum_long<T, VEC, 4>(a, g, wss, stream); break;
    default: launch_approx_sum_long<T, VEC, 0>(a, g, wss, stream); break;
  }
}
}  // namespace

bool approx_sums_long_rows(int32_t dtype, int32_t D, bool weighted) {
  return !weighted && dtype != TBE_DTYPE_F16 && approx_short_serves(dtype, D);
}

// The long rows of the approximate update in its chunked form (approx_sums_long_rows()): the short-row
// kernel, called with a null queue, has left them in the chunk queues of `a`; `lookup_wss` holds
// ||grad||^2 of every lookup by position.
int segment_update_approx_sum_long(const UpdateArgs &a, const void *lookup_wss, hipStream_t stream) {
  if (a.num_indices == 0) return TBE_OK;
  const RowGeometry g = row_geometry(a.dtype, a.D);
  if (a.dtype == TBE_DTYPE_F32) launch_approx_sum_long_geometry<float, 4>(a, g, lookup_wss, stream);
  else launch_approx_sum_long_geometry<double, 2>(a, g, lookup_wss, stream);
  return check_launch("tbe approximate Adagrad update (summed rows)");
}

int segment_update(const UpdateArgs &a, hipStream_t stream) {
  if (a.num_indices == 0) return TBE_OK;
  const RowGeometry g = row_geometry(a.dtype, a.D);
  // the queue counters were zeroed when the plan's segments were found
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
