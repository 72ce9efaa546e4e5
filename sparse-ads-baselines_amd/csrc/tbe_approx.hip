// Approximate row-wise Adagrad for gfx950: the reference's per-lookup update
// (batched_embedding_backward_adagrad_approx_kernel_1, table_batched_embeddings_cuda.cu:648-704,
// with AdaGradFunctor / WeightedAdaGradFunctor, :437-471, :483-553; mixed-D twin :1006-1074),
// made deterministic.
//
// The reference gives every bag a warp that, for each of the bag's lookups, adds the bag's
// ||grad||^2 to the row's state with a plain load and store, derives one multiplier per lookup
// from the state it found, and subtracts multiplier * grad from the row.  Bags run concurrently,
// so a row that occurs in two bags is raced for; the result is defined only when no row repeats.
// Here the same per-lookup arithmetic runs ONE LOOKUP AT A TIME per row, in position order:
// the batch is sorted by (table, row) as for the exact update, and the lane group that owns a
// row walks its occurrences in ascending position,
//     wss  = ||grad_output[b][t]||^2 (* psw[p]^2)
//     s   += wss;  mult = (psw[p] *) lr * (1.0 / (sqrt(s) + eps))
//     grad_psw[p] = <row, grad_output[b][t]>          (weighted; the row as it is at that moment)
//     row -= mult * grad_output[b][t]                 (rounded to the weights' type every time)
// Rows are independent, so this is the reference's kernel executed serially in position order:
// identical to it when no row repeats, and the serial outcome when rows do.  No atomics, fixed
// order, bit-identical reruns.
//
// Geometry: `group` lanes (a power of two, the row's vector count rounded up, at most 64) own
// one row; a wavefront holds 64 / group rows.  A row of at most `group` vectors stays in
// registers from its first to its last occurrence; wider rows (and the mixed-D tables, which use
// the whole wavefront per row) are read and written per occurrence in column blocks.  Gradient
// rows of up to 8 occurrences are requested together.
//
// A row with more than kApproxLong occurrences would keep one lane group busy for a long serial
// walk (three dependent loads per 8 occurrences, a double-precision division per occurrence).
// Such rows are queued and get a wavefront each (approx_adagrad_long_kernel), which takes 64
// occurrences at a time: bookkeeping one occurrence per lane, ||grad||^2 by all lane groups in
// parallel, the running state by a wavefront prefix sum and the 64 multipliers side by side;
// only `row -= mult * grad` (and its rounding) remains a serial chain, fed by prefetched rows.

#include <algorithm>
#include <type_traits>

#include "tbe_rowwise.h"
#include "tbe_stages.h"

namespace tbe {
namespace {

// Value of `v` in lane `src`, for a lane number that is the same in every lane (a scalar read
// instead of a trip through LDS).
__device__ __forceinline__ int broadcast_lane(int v, int src) { return __builtin_amdgcn_readlane(v, src); }
__device__ __forceinline__ float broadcast_lane(float v, int src) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), src));
}
__device__ __forceinline__ int64_t broadcast_lane(int64_t v, int src) {
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v), src));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readlane(static_cast<int>(v >> 32), src));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}
__device__ __forceinline__ double broadcast_lane(double v, int src) {
  return __longlong_as_double(broadcast_lane(static_cast<int64_t>(__double_as_longlong(v)), src));
}

// A value that is the same in every lane, moved to scalar registers.
__device__ __forceinline__ int uniform(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ int64_t uniform(int64_t v) {
  const uint32_t lo = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v)));
  const uint32_t hi = static_cast<uint32_t>(__builtin_amdgcn_readfirstlane(static_cast<int>(v >> 32)));
  return static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo);
}

// Sum over the `group` lanes (a power of two) around the caller; every lane gets the result.
template <typename A> __device__ __forceinline__ A group_sum_pow2(A v, int group) {
  for (int m = group >> 1; m > 0; m >>= 1) v += shfl_x(v, m);
  return v;
}


constexpr int kBatch = 8;  // occurrences whose gradient rows are requested together
constexpr int kApproxLong = 64;  // a register-held row with more occurrences gets a wavefront of its own

// Geometry of the row behind a unique key and of its gradient rows.
struct RowPlace {
  int row_D;            // elements in the row
  int64_t row_element;  // first element of the row inside `weights`
  int64_t grad_stride;  // elements between consecutive gradient rows ...
  int grad_column;      // ... and the first column of this table inside one
};

template <bool MIXED>
__device__ __forceinline__ RowPlace place_row(int64_t key, int first_grad_row, int D, const MixedTables &mt) {
  RowPlace p{D, key * D, D, 0};
  if constexpr (MIXED) {
    const int table = first_grad_row % mt.T;
    const int column0 = mt.dim_offsets[table];
    p.row_D = mt.dim_offsets[table + 1] - column0;
    p.row_element = mt.table_offsets[table] + (key - mt.table_dim_offsets[table]) * p.row_D;
    p.grad_column = column0;
    p.grad_stride = mt.total_D;
  }
  return p;
}

template <bool MIXED>
__device__ __forceinline__ int64_t grad_row_offset(int grad_row, const RowPlace &p, const MixedTables &mt) {
  if constexpr (MIXED) return static_cast<int64_t>(grad_row / mt.T) * p.grad_stride + p.grad_column;
  else return static_cast<int64_t>(grad_row) * p.grad_stride;
}

template <typename T, int VEC, bool WEIGHTED, bool MIXED>
__global__ __launch_bounds__(kBlockThreads) void approx_adagrad_kernel(
    const T *__restrict__ grad_output, T *__restrict__ weights,
    typename AccOf<T>::type *__restrict__ state, const T *__restrict__ psw, T *__restrict__ grad_psw,
    const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ positions_sorted,
    const int32_t *__restrict__ grad_rows, const int32_t *__restrict__ segment_starts,
    int32_t *__restrict__ counters, int32_t *__restrict__ long_queue, int D, int group, float lr,
    float eps, MixedTables mt, StochasticRounding sr, const int32_t *__restrict__ only_rows,
    const int32_t *__restrict__ unique_slots, T *__restrict__ cache_rows, int slot_D) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  using R = typename V::R;

  const int lane = threadIdx.x & (kWave - 1);
  const int r = lane / group;
  const int c = lane - r * group;
  const int group_base = r * group;
  const int groups = kWave / group;
  // every unique row, or (only_rows) the rows another kernel has left in a queue of counters[2] entries
  const int U = only_rows ? counters[2] : counters[0];
  const int64_t wave_id = static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6);
  const int64_t wave_stride = static_cast<int64_t>(gridDim.x) * kWavesPerBlock;
  const int batch = group < kBatch ? group : kBatch;  // one lane of the group fetches one occurrence's bookkeeping

  // A wavefront takes strips of 64 unique rows.  First one row per LANE: segment bounds, key,
  // state, position / gradient row / weight of the first occurrence -- the dependent loads are
  // paid once per strip, 64 wide.  Then one row per lane GROUP, handed out by lane shuffles.
  // (Every lane of the wavefront runs the same trip counts: the shuffles need all of them.)
  for (int64_t strip = wave_id * kWave; strip < U; strip += wave_stride * kWave) {
    const int rows_here = static_cast<int>(min(static_cast<int64_t>(kWave), U - strip));
    int lane_begin = 0, lane_end = 0, lane_key = 0, lane_pos0 = 0, lane_grow0 = 0;
    A lane_state = A(0), lane_pw0 = A(1);
    int lane_u = static_cast<int>(strip) + lane;
    if (lane < rows_here) {
      if (only_rows) lane_u = only_rows[strip + lane];
      lane_begin = segment_starts[lane_u];
      lane_end = segment_starts[lane_u + 1];
      lane_key = keys_sorted[lane_begin];
      lane_pos0 = positions_sorted[lane_begin];
      lane_state = state[lane_key];
      lane_grow0 = grad_rows[lane_pos0];
      if constexpr (WEIGHTED) lane_pw0 = to_acc(psw[lane_pos0]);
    }
  for (int i0 = 0; i0 < rows_here; i0 += groups) {
    const bool valid = i0 + r < rows_here;
    const int src = valid ? i0 + r : 0;
    const int64_t u = shfl_idx(lane_u, src);
    const int seg_begin = shfl_idx(lane_begin, src);
    int seg_end = shfl_idx(lane_end, src);
    if (!valid) seg_end = seg_begin;
    const int64_t key = shfl_idx(lane_key, src);
    const int first_pos = shfl_idx(lane_pos0, src);
    const int first_grow = shfl_idx(lane_grow0, src);
    const A first_pw = shfl_idx(lane_pw0, src);
    const A state_in = shfl_idx(lane_state, src);
    // where the row and its gradient rows live
    const RowPlace place = place_row<MIXED>(key, first_grow, D, mt);
    const int row_D = valid ? place.row_D : 0;
    const int64_t row_element = place.row_element;
    const int64_t grad_stride = place.grad_stride;
    const int grad_column = place.grad_column;
    const int row_chunks = valid ? row_D / VEC : 0;
    const bool in_registers = row_chunks <= group;   // one vector per lane holds the row
    const bool mine = c < row_chunks;                // this lane owns a vector of a register-held row
    if (valid && in_registers && seg_end - seg_begin > kApproxLong) {
      // a long walk: the row gets a wavefront of its own in approx_adagrad_long_kernel
      if (c == 0) long_queue[atomicAdd(&counters[1], 1)] = static_cast<int32_t>(u);
      seg_end = seg_begin;  // nothing to do here
    }
    const bool handled_here = seg_end > seg_begin;
    // (cache-fronted tables: the row lives in its cache slot, slot_D elements wide, when it has one;
    // its random words still go by its place in the table)
    T *wrow = weights + row_element;
    if (unique_slots) {
      const int slot = unique_slots[u];
      if (slot >= 0) wrow = cache_rows + static_cast<int64_t>(slot) * slot_D;
    }
    A s = state_in;
    V w;
    w.zero();
    if (handled_here && in_registers && mine) w.load(wrow + static_cast<int64_t>(c) * VEC);

    for (int k0 = seg_begin; __any(k0 < seg_end); k0 += batch) {
      // bookkeeping of up to `batch` occurrences, one per lane of the group
      int my_pos = first_pos, my_grow = first_grow;  // the segment's first occurrence is known already
      A my_pw = first_pw;
      if (c < batch && k0 + c < seg_end && k0 + c > seg_begin) {
        my_pos = positions_sorted[k0 + c];
        my_grow = grad_rows[my_pos];
        if constexpr (WEIGHTED) my_pw = to_acc(psw[my_pos]);
      }
      // the gradient vectors of a register-held row, requested together
      R raw[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        const int src = group_base + (j < batch ? j : 0);
        const int grow = shfl_idx(my_grow, src);
        const int64_t gbase = MIXED ? static_cast<int64_t>(grow / mt.T) * grad_stride + grad_column
                                    : static_cast<int64_t>(grow) * grad_stride;
        if (in_registers && mine && j < batch && k0 + j < seg_end)
          raw[j] = V::load_raw(grad_output + gbase + static_cast<int64_t>(c) * VEC);
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        if (j >= batch) break;
        if (!__any(k0 + j < seg_end)) break;
        const bool live = k0 + j < seg_end;
        const int src = group_base + j;
        const int pos = shfl_idx(my_pos, src);
        const int grow = shfl_idx(my_grow, src);
        const A pw = shfl_idx(my_pw, src);
        const int64_t gbase = MIXED ? static_cast<int64_t>(grow / mt.T) * grad_stride + grad_column
                                    : static_cast<int64_t>(grow) * grad_stride;
        const T *grow_ptr = grad_output + gbase;
        // the k-th update of a row in this call rounds with its own random words
        const StochasticRounding sr_k = rounding_of_update(sr, k0 + j - seg_begin);

        // ||grad||^2 of the bag (the reference computes it once per bag, tbe.cu:668-675)
        A local = A(0);
        V g;
        g.zero();
        if (in_registers) {
          if (live && mine) g.unpack(raw[j]);
#pragma unroll
          for (int i = 0; i < VEC; ++i) local += g.v[i] * g.v[i];
        } else if (live) {
          for (int cb = c; cb < row_chunks; cb += group) {
            V x;
            x.load(grow_ptr + static_cast<int64_t>(cb) * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) local += x.v[i] * x.v[i];
          }
        }
        const A gss = group_sum_pow2<A>(local, group);
        A mult = A(0);
        if (live) {
          const A wss = WEIGHTED ? gss * pw * pw : gss;
          s = s + wss;
          mult = approx_multiplier<A>(s, pw, WEIGHTED, lr, eps);
        }
        A dot = A(0);
        if (in_registers) {
          if (live && mine) {
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WEIGHTED) dot += w.v[i] * g.v[i];
              w.v[i] = w.v[i] - g.v[i] * mult;
            }
            round_trip<T, VEC>(w, sr_k, row_element + static_cast<int64_t>(c) * VEC);
          }
        } else if (live) {
          for (int cb = c; cb < row_chunks; cb += group) {
            V x, y;
            x.load(grow_ptr + static_cast<int64_t>(cb) * VEC);
            y.load(wrow + static_cast<int64_t>(cb) * VEC);
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
              if constexpr (WEIGHTED) dot += y.v[i] * x.v[i];
              y.v[i] = y.v[i] - x.v[i] * mult;
            }
            store_row<T, VEC, false>(wrow + static_cast<int64_t>(cb) * VEC, y, sr_k,
                                     row_element + static_cast<int64_t>(cb) * VEC);
          }
        }
        if constexpr (WEIGHTED) {
          dot = group_sum_pow2<A>(dot, group);
          if (live && c == 0) grad_psw[pos] = from_acc<T, A>(dot);
        }
      }
    }
    if (handled_here && c == 0) state[key] = s;
    // (fp16: the last update already rounded the row to the stored type, this conversion is exact)
    if (handled_here && in_registers && mine) w.store(wrow + static_cast<int64_t>(c) * VEC);
  }
  }
}

// ||grad||^2 (times the squared per-sample weight) of every lookup, by position: the addend of the
// row state that the lookup's update starts with.  One lane group per bag reads the bag's gradient
// row once and writes the value to the bag's positions, so the kernel below neither gathers a
// gradient row twice nor forms a norm inside its serial walk.  Nothing reads the values when no
// row was queued, and the kernel returns at once.
template <typename T, int VEC, bool WEIGHTED, bool MIXED>
__global__ __launch_bounds__(kBlockThreads) void approx_lookup_norms_kernel(
    const T *__restrict__ grad_output, const T *__restrict__ psw, const int32_t *__restrict__ offsets,
    const int32_t *__restrict__ counters, typename AccOf<T>::type *__restrict__ lookup_wss, int B,
    int T_tables, int D, int group, MixedTables mt) {
  using V = RowVec<T, VEC>;
  using A = typename V::A;
  int queued = counters[1];  // (one queue, or one per XCD)
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) queued += counters[xcd_counter(x)];
  if (queued == 0) return;
  const int lane = threadIdx.x & (kWave - 1);
  const int r = lane / group;
  const int c = lane - r * group;
  const int groups = kWave / group;
  const int64_t bags = static_cast<int64_t>(B) * T_tables;
  const int64_t bag = (static_cast<int64_t>(blockIdx.x) * kWavesPerBlock + (threadIdx.x >> 6)) * groups + r;
  const bool valid = bag < bags;
  const int t = valid ? static_cast<int>(bag / B) : 0;
  const int b = valid ? static_cast<int>(bag - static_cast<int64_t>(t) * B) : 0;
  const int begin = valid ? offsets[bag] : 0;
  const int end = valid ? offsets[bag + 1] : 0;
  int row_D = D;
  int64_t goff = (static_cast<int64_t>(b) * T_tables + t) * D;
  if constexpr (MIXED) {
    const int column0 = mt.dim_offsets[t];
    row_D = mt.dim_offsets[t + 1] - column0;
    goff = static_cast<int64_t>(b) * mt.total_D + column0;
  }
  const int row_chunks = end > begin ? row_D / VEC : 0;  // a bag without lookups needs no norm
  A local = A(0);
  for (int cb = c; cb < row_chunks; cb += group) {
    V x;
    x.load(grad_output + goff + static_cast<int64_t>(cb) * VEC);
#pragma unroll
    for (int i = 0; i < VEC; ++i) local += x.v[i] * x.v[i];
  }
  const A gss = group_sum_pow2<A>(local, group);
  for (int p = begin + c; p < end; p += group) {
    A wss = gss;
    if constexpr (WEIGHTED) {
      const A pw = to_acc(psw[p]);
      wss = gss * pw * pw;
    }
    lookup_wss[p] = wss;
  }
}

// E consecutive elements of a row, loaded with one instruction of E * sizeof(T) bytes.
template <typename T, int E> struct alignas(E * sizeof(T)) LanePack { T x[E]; };

// The E values of a lane after they were stored in the weights' type and read again: nothing for
// fp32 / fp64; fp16: round to nearest even, or, with stochastic rounding, element e takes word
// e % 4 of the Philox block of elements 4 * (e / 4) ... (the rule of pack_rounded).
template <typename T, int E, bool STOCHASTIC, typename A>
__device__ __forceinline__ void round_lane_elements(A (&v)[E], const StochasticRounding &sr, int64_t element) {
  if constexpr (sizeof(T) == 2) {
    if constexpr (STOCHASTIC) {
      constexpr int kBlocks = E >= 4 ? E / 4 : 1;
#pragma unroll
      for (int q = 0; q < kBlocks; ++q) {
        const uint64_t block = static_cast<uint64_t>(element) / 4 + q;
        const uint4 rnd = philox4x32_10(
            make_uint4(static_cast<uint32_t>(block), static_cast<uint32_t>(block >> 32),
                       static_cast<uint32_t>(sr.offset), static_cast<uint32_t>(sr.offset >> 32)),
            make_uint2(static_cast<uint32_t>(sr.seed), static_cast<uint32_t>(sr.seed >> 32)));
        const uint32_t word[4] = {rnd.x, rnd.y, rnd.z, rnd.w};
        constexpr int kHere = E >= 4 ? 4 : E;
        const int first = E >= 4 ? 0 : static_cast<int>(element & 3);  // (a multiple of E)
#pragma unroll
        for (int i = 0; i < kHere; ++i) {
          uint32_t bits = word[0];
#pragma unroll
          for (int x = 1; x < 4; ++x) bits = (first + i == x) ? word[x] : bits;
          A &value = v[4 * q + i];
          value = round_trip_stochastic(value, bits);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < E; ++i) v[i] = __half2float(__float2half_rn(v[i]));
    }
  }
}

// Stochastic rounding of a lane's E < 4 elements with Philox blocks shared inside a quad of lanes.
// The 4 / E lanes whose elements fall into one block of four would each draw the same block for
// an occurrence; instead they draw it for 4 / E consecutive occurrences, one each (`rnd`, drawn
// with the occurrence's key), and for occurrence number SLOT of those a lane reads its words from
// the quad's lane that drew them.  The words and the rounding are those of round_lane_elements.
template <int E, int SLOT> __device__ __forceinline__ uint32_t quad_word(uint32_t v) {
  // lanes of a quad read from lane SLOT (E == 1), or lanes 0, 1 from lane SLOT and lanes 2, 3 from lane 2 + SLOT
  constexpr int kPattern = E == 1 ? (SLOT | SLOT << 2 | SLOT << 4 | SLOT << 6)
                                  : (SLOT | SLOT << 2 | (2 + SLOT) << 4 | (2 + SLOT) << 6);
  return static_cast<uint32_t>(__builtin_amdgcn_mov_dpp(static_cast<int>(v), kPattern, 0xf, 0xf, true));
}
template <int E, int SLOT, typename A>
__device__ __forceinline__ void round_with_shared_draw(A (&v)[E], const uint4 &rnd, int lane) {
  static_assert(E == 1 || E == 2, "lanes that hold less than a block of four elements");
  const uint32_t word[4] = {quad_word<E, SLOT>(rnd.x), quad_word<E, SLOT>(rnd.y), quad_word<E, SLOT>(rnd.z),
                            quad_word<E, SLOT>(rnd.w)};
  const int first = (lane * E) & 3;  // the lane's first element inside its block (rows start on a block)
#pragma unroll
  for (int i = 0; i < E; ++i) {
    uint32_t bits = word[0];
#pragma unroll
    for (int x = 1; x < 4; ++x) bits = (first + i == x) ? word[x] : bits;
    v[i] = round_trip_stochastic(v[i], bits);
  }
}
__device__ __forceinline__ uint4 draw_block(const StochasticRounding &sr, int64_t element) {
  const uint64_t block = static_cast<uint64_t>(element) / 4;
  return philox4x32_10(make_uint4(static_cast<uint32_t>(block), static_cast<uint32_t>(block >> 32),
                                  static_cast<uint32_t>(sr.offset), static_cast<uint32_t>(sr.offset >> 32)),
                       make_uint2(static_cast<uint32_t>(sr.seed), static_cast<uint32_t>(sr.seed >> 32)));
}

// Cooperative walk of a very long fp16 row with stochastic rounding: the random bits are most of
// the work per occurrence, and they do not depend on the values, so three wavefronts of the
// workgroup draw them for the next 32 occurrences into LDS while the first wavefront walks the
// current 32.  words[2][kCoopStep][kCoopD]: the 13 random bits of every element of the row for
// every occurrence of a step, two steps deep.
constexpr int kCoopD = 128;    // widest row walked this way (two elements per lane)
static_assert(kCoopD == kApproxCoopD, "the width up to which rows are listed for a workgroup's walk");
constexpr int kCoopStep = 32;  // occurrences per step
// The barrier between the steps of the cooperative walk: LDS traffic of the wavefront is complete
// (the bits written, or the bits of the finished step read), but the walking wavefront's gradient
// rows stay in flight -- __syncthreads() would wait for them too and drain the ring at every step.
__device__ __forceinline__ void step_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void draw_step_bits(const StochasticRounding &sr, int64_t row_element, int row_D,
                                               int first_occurrence, int count, uint16_t *words, int thread,
                                               int threads) {
  // A thread keeps one block of four elements and takes every (threads >> shift)-th occurrence,
  // 2^shift being the blocks of a row rounded up to a power of two (threads is a multiple of
  // 32): no division, and the occurrence's key advances by an addition.  The words are those of
  // draw_block(rounding_of_update(sr, occurrence), row_element + 4 * block).
  const int blocks_per_row = row_D / 4;
  int shift = 0;
  while ((1 << shift) < blocks_per_row) ++shift;
  const int block = thread & ((1 << shift) - 1);
  if (block >= blocks_per_row) return;
  const int per_round = threads >> shift;
  const uint64_t kKeyStep = 0x9E3779B97F4A7C15ull;  // (rounding_of_update)
  int o = thread >> shift;
  uint64_t key_term = static_cast<uint64_t>(first_occurrence + o) * kKeyStep;
  const uint64_t round_term = static_cast<uint64_t>(per_round) * kKeyStep;
  const uint64_t counter = static_cast<uint64_t>(row_element) / 4 + static_cast<uint64_t>(block);
  for (; o < count; o += per_round, key_term += round_term) {
    const uint64_t seed = sr.seed ^ key_term;
    const uint4 r = philox4x32_10(
        make_uint4(static_cast<uint32_t>(counter), static_cast<uint32_t>(counter >> 32),
                   static_cast<uint32_t>(sr.offset), static_cast<uint32_t>(sr.offset >> 32)),
        make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)));
    uint2 packed;
    packed.x = (r.x >> 19) | ((r.y >> 19) << 16);
    packed.y = (r.z >> 19) | ((r.w >> 19) << 16);
    *reinterpret_cast<uint2 *>(words + o * kCoopD + 4 * block) = packed;
  }
}

template <typename T> struct LongRowArgs {
  using A = typename AccOf<T>::type;
  const T *grad_output;
  T *weights;
  A *state;
  const T *psw;
  T *grad_psw;
  const int32_t *positions_sorted;
  const int32_t *grad_rows;
  const A *lookup_wss;
  float lr, eps;
  MixedTables mt;  // (T == 0: uniform tables)
  StochasticRounding sr;
  uint64_t grad_bytes;  // size of grad_output
  const int32_t *unique_slots;  // cache-fronted tables: slot of each unique row (-1: not resident), or null
  T *cache_rows;
  int slot_D;  // elements of a cache row
};

// First element of gradient row `grad_row` for a row at `p` (mixed-D tables: mt.T > 0).
__device__ __forceinline__ int64_t long_row_grad_offset(int grad_row, const RowPlace &p, const MixedTables &mt) {
  if (mt.T > 0) return static_cast<int64_t>(grad_row / mt.T) * p.grad_stride + p.grad_column;
  return static_cast<int64_t>(grad_row) * p.grad_stride;
}

// A LanePack read through a buffer descriptor: scalar byte offset of the row plus the lane's
// byte offset, so that a row request is two instructions (a lane read and the load).
template <typename P>
__device__ __forceinline__ P buffer_load_pack(__amdgpu_buffer_rsrc_t rsrc, uint32_t lane_bytes, uint32_t row_bytes) {
  P out;
  if constexpr (sizeof(P) == 2) {
    const uint16_t v = __builtin_amdgcn_raw_buffer_load_b16(rsrc, lane_bytes, row_bytes, 0);
    __builtin_memcpy(&out, &v, 2);
  } else if constexpr (sizeof(P) == 4) {
    const uint32_t v = __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_bytes, row_bytes, 0);
    __builtin_memcpy(&out, &v, 4);
  } else if constexpr (sizeof(P) == 8) {
    const auto v = __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_bytes, row_bytes, 0);
    __builtin_memcpy(&out, &v, 8);
  } else {
    const auto v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, row_bytes, 0);
    __builtin_memcpy(&out, &v, 16);
  }
  return out;
}

// The walk over one queued row by a whole wavefront: lane l owns elements [l * E, l * E + E) of
// the row from the first to the last occurrence.  Occurrences are taken 64 at a time: their
// bookkeeping (position, gradient row, per-sample weight, state addend) sits one per lane and is
// requested two batches (positions: three) ahead; the running state of the 64 comes from a
// wavefront prefix sum and their multipliers (a double-precision division each) are formed side
// by side.  What remains serial is `row -= mult * grad` (and its rounding) per occurrence.  Its
// gradient rows are requested well ahead, across batch boundaries, so that the chain does not
// wait for memory: into a ring of 64 registers (64, 32 or 16 rows, by the bytes of a row that a
// lane holds), each slot refilled as soon as it has been applied; with stochastic rounding, where the random bits
// are most of the work per occurrence, 16 ahead into one of two sets of 16.
// COOP (with STOCHASTIC, E <= 2): the wavefront is the first of a workgroup whose other wavefronts
// draw the random bits (draw_step_bits) into `words`; it meets them at a barrier after every
// kCoopStep occurrences.
template <typename T, int E, bool WEIGHTED, bool STOCHASTIC, bool BIG, bool COOP = false>
__device__ __forceinline__ void walk_long_row(const LongRowArgs<T> &a, int seg_begin, int seg_end, int64_t key,
                                              const RowPlace &place, T *storage, int lane,
                                              const uint16_t *words = nullptr) {
  using A = typename AccOf<T>::type;
  using P = LanePack<T, E>;
  static_assert(!COOP || (STOCHASTIC && E <= 2), "the cooperative walk is for stochastic rounding of narrow rows");
  constexpr int kAhead = 16;
  static_assert(kWave % kCoopStep == 0, "a batch is a whole number of steps");
  int step = 0;  // (COOP) steps walked so far
  // (the cooperative walk does not draw random words itself: it is as light per occurrence as the
  // walk without stochastic rounding and needs as many rows in flight)
  constexpr bool kInBlocks = STOCHASTIC && !COOP;
  constexpr int kRing = kInBlocks ? 2 * kAhead : (E * sizeof(T) <= 4 ? kWave : E * sizeof(T) <= 8 ? kWave / 2 : kWave / 4);
  const bool active = lane * E < place.row_D;
  const int lane_off = active ? lane * E : 0;  // (idle lanes shadow lane 0 and store nothing)
  T *wrow = storage + lane_off;  // (the row's first element where it lives: table or cache slot)
  A w[E];
  {
    const P p = *reinterpret_cast<const P *>(wrow);
#pragma unroll
    for (int i = 0; i < E; ++i) w[i] = to_acc(p.x[i]);
  }
  A s = a.state[key];

  // Bookkeeping, one occurrence per lane: this batch's and the next one's complete, the positions
  // of the batch after that on their way.  Everything a batch needs was requested at least a
  // whole batch earlier, so waiting for it never waits for the row requests behind it.
  const int last = seg_end - 1;
  int cur_pos = a.positions_sorted[min(seg_begin + lane, last)];
  int nxt_pos = a.positions_sorted[min(seg_begin + kWave + lane, last)];
  int aft_pos = a.positions_sorted[min(seg_begin + 2 * kWave + lane, last)];
  // where a gradient row starts: its first element, or (grad_output below 4 GiB) its first byte
  using Off = typename std::conditional<BIG, int64_t, int>::type;
  auto offset_of = [&](int grad_row) {
    const int64_t element = long_row_grad_offset(grad_row, place, a.mt);
    if constexpr (BIG) return element;
    else return static_cast<int>(static_cast<uint32_t>(element) * static_cast<uint32_t>(sizeof(T)));
  };
  Off cur_goff = offset_of(a.grad_rows[cur_pos]);
  Off nxt_goff = offset_of(a.grad_rows[nxt_pos]);
  A cur_pw = A(1), nxt_pw = A(1);
  if constexpr (WEIGHTED) {
    cur_pw = to_acc(a.psw[cur_pos]);
    nxt_pw = to_acc(a.psw[nxt_pos]);
  }
  A cur_wss = a.lookup_wss[cur_pos];
  A nxt_wss = a.lookup_wss[nxt_pos];
  // (waited for here, before the first row requests)
  asm volatile("" : "+v"(aft_pos), "+v"(nxt_goff), "+v"(nxt_pw), "+v"(nxt_wss) : : "memory");

  const uint32_t lane_bytes = static_cast<uint32_t>(lane_off) * static_cast<uint32_t>(sizeof(T));
  // (a raw buffer over grad_output: no stride, its size in bytes, 32-bit data format -- reads past
  // the end return zero)
  const __amdgpu_buffer_rsrc_t grad_buffer = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<T *>(a.grad_output), 0, static_cast<int>(static_cast<uint32_t>(BIG ? 0 : a.grad_bytes)), 0x00020000);
  auto row_of = [&](Off goffs, int src_lane) {
    if constexpr (BIG) return *reinterpret_cast<const P *>(a.grad_output + lane_off + broadcast_lane(goffs, src_lane));
    else return buffer_load_pack<P>(grad_buffer, lane_bytes, static_cast<uint32_t>(broadcast_lane(goffs, src_lane)));
  };
  P ring[kRing];
  {
    const int nb = min(kWave, seg_end - seg_begin);
    constexpr int kFirst = kInBlocks ? kAhead : kRing;
#pragma unroll
    for (int c = 0; c < kFirst; c += kAhead) {
      if (c < nb) {
#pragma unroll
        for (int b = 0; b < kAhead; ++b) ring[c + b] = row_of(cur_goff, min(c + b, nb - 1));
      }
    }
  }

  for (int k0 = seg_begin; k0 < seg_end; k0 += kWave) {
    const int nb = min(kWave, seg_end - k0);
    const int nb_next = min(kWave, seg_end - k0 - kWave);  // <= 0: this is the last batch
    // requested now, used from the next iteration on
    const int aft_grow = a.grad_rows[aft_pos];
    A aft_pw = A(1);
    if constexpr (WEIGHTED) aft_pw = to_acc(a.psw[aft_pos]);
    const A aft_wss = a.lookup_wss[aft_pos];
    const int fut_pos = a.positions_sorted[min(k0 + 3 * kWave + lane, last)];

    // running state and multiplier of every occurrence, one per lane
    const A incl = wave_inclusive_sum<A>(lane < nb ? cur_wss : A(0));
    const A my_mult = lane < nb ? approx_multiplier<A>(s + incl, cur_pw, WEIGHTED, a.lr, a.eps) : A(0);
    s = s + broadcast_lane(incl, nb - 1);

    // occurrence j of the batch, its gradient row in `grad`; with stochastic rounding and fewer
    // than four elements per lane, `shared_draw` holds the random words that this lane drew for
    // one of the kShare occurrences around j and `slot` tells which of them j is
    constexpr int kShare = (STOCHASTIC && E < 4) ? 4 / E : 1;
    // (COOP) the 13 random bits of this lane's elements for occurrence j of the batch, from the
    // buffer of the current step
    auto bits_of = [&](int j) {
      if constexpr (COOP) {
        const uint16_t *mine = words + (step & 1) * (kCoopStep * kCoopD) + (j & (kCoopStep - 1)) * kCoopD + lane_off;
        if constexpr (E == 1) return make_uint4(mine[0], 0u, 0u, 0u);
        else {
          const uint32_t two = *reinterpret_cast<const uint32_t *>(mine);
          return make_uint4(two & 0xffffu, two >> 16, 0u, 0u);
        }
      } else {
        return make_uint4(0u, 0u, 0u, 0u);
      }
    };
    auto apply = [&](const P &grad, int j, const uint4 &shared_draw, int slot) {
      const A mult = broadcast_lane(my_mult, j);
      A dot = A(0);
#pragma unroll
      for (int i = 0; i < E; ++i) {
        const A g = to_acc(grad.x[i]);
        if constexpr (WEIGHTED) dot += w[i] * g;
        w[i] = w[i] - g * mult;
      }
      if constexpr (COOP) {
        // (shared_draw.x, .y: the 13 bits of the lane's elements)
        w[0] = round_trip_with_bits(w[0], shared_draw.x);
        if constexpr (E == 2) w[1] = round_trip_with_bits(w[1], shared_draw.y);
      } else if constexpr (STOCHASTIC && E < 4) {
        if (slot == 0) round_with_shared_draw<E, 0, A>(w, shared_draw, lane);
        else if (slot == 1) round_with_shared_draw<E, 1, A>(w, shared_draw, lane);
        else if constexpr (E == 1) {
          if (slot == 2) round_with_shared_draw<E, 2, A>(w, shared_draw, lane);
          else round_with_shared_draw<E, 3, A>(w, shared_draw, lane);
        }
      } else if constexpr (STOCHASTIC) {
        round_lane_elements<T, E, true, A>(w, rounding_of_update(a.sr, k0 + j - seg_begin),
                                           place.row_element + lane_off);
      } else {
        round_lane_elements<T, E, false, A>(w, a.sr, place.row_element + lane_off);
      }
      if constexpr (WEIGHTED) {
        // (the wavefront's sum by lane moves: lane shuffles go through LDS and would wait one round
        // trip each, per occurrence)
        dot = wave_sum_in_last_row<A>(active ? dot : A(0));
        const int pos = broadcast_lane(cur_pos, j);
        if (lane == kWave - 1) a.grad_psw[pos] = from_acc<T, A>(dot);
      }
    };

    if constexpr (kInBlocks) {
      // one block of 16 occurrences: request the block after it into `fill`, then apply `use`
      auto block = [&](P *use, P *fill, int j0) {
        Off src = cur_goff;
        int first = 0, limit = 0;
        if (j0 + kAhead < nb) {
          first = j0 + kAhead;
          limit = nb - 1;
        } else if (nb_next > 0) {
          src = nxt_goff;
          limit = nb_next - 1;
        }
#pragma unroll
        for (int b = 0; b < kAhead; ++b) fill[b] = row_of(src, min(first + b, limit));
        uint4 draw = make_uint4(0u, 0u, 0u, 0u);
#pragma unroll
        for (int b = 0; b < kAhead; ++b) {
          if (j0 + b < nb) {
            if constexpr (kShare > 1) {
              // one draw per lane serves kShare occurrences: this lane's is for occurrence b + lane % kShare
              if (b % kShare == 0)
                draw = draw_block(rounding_of_update(a.sr, k0 + j0 + b + (lane % kShare) - seg_begin),
                                  place.row_element + lane_off);
            }
            apply(use[b], j0 + b, draw, b % kShare);
          }
        }
      };
      // blocks are taken in pairs so that the two register sets swap roles in place; the second
      // block of a pair may find nothing left to apply and then only renews the request for the
      // next batch's first rows
      int j0 = 0;
      do {  // (nb > 0)
        block(ring, ring + kAhead, j0);
        block(ring + kAhead, ring, j0 + kAhead);
        j0 += 2 * kAhead;
      } while (j0 < nb);
    } else if (nb == kWave && nb_next == kWave) {
      // a full batch followed by a full batch: straight-line code
      uint4 bits = bits_of(0);
#pragma unroll
      for (int j = 0; j < kWave; ++j) {
        const uint4 now = bits;
        if ((j + 1) % kCoopStep != 0) bits = bits_of(j + 1);
        apply(ring[j % kRing], j, now, 0);
        if (j + kRing < kWave) ring[j % kRing] = row_of(cur_goff, j + kRing);
        else ring[j % kRing] = row_of(nxt_goff, j + kRing - kWave);
        if constexpr (COOP) {
          if ((j + 1) % kCoopStep == 0) {
            step_barrier();  // the next step's bits are there, this step's buffer may be refilled
            ++step;
            if (j + 1 < kWave) bits = bits_of(j + 1);
          }
        }
      }
    } else {
      uint4 bits = bits_of(0);
#pragma unroll
      for (int j = 0; j < kWave; ++j) {
        if (j < nb) {
          const uint4 now = bits;
          if ((j + 1) % kCoopStep != 0) bits = bits_of(j + 1);
          apply(ring[j % kRing], j, now, 0);
          const int target = (j + kRing) % kWave;  // occurrence j + kRing of the row ...
          if (j + kRing < kWave) {                 // ... is in this batch
            if (target < nb) ring[j % kRing] = row_of(cur_goff, target);
          } else if (nb_next > 0) {                // ... or in the next one
            ring[j % kRing] = row_of(nxt_goff, min(target, nb_next - 1));
          }
          if constexpr (COOP) {
            if ((j + 1) % kCoopStep == 0 || j == nb - 1) {
              step_barrier();
              ++step;
              if (j + 1 < kWave) bits = bits_of(j + 1);
            }
          }
        }
      }
    }
    cur_pos = nxt_pos;
    cur_goff = nxt_goff;
    cur_pw = nxt_pw;
    cur_wss = nxt_wss;
    nxt_pos = aft_pos;
    nxt_goff = offset_of(aft_grow);
    nxt_pw = aft_pw;
    nxt_wss = aft_wss;
    aft_pos = fut_pos;
  }
  if (lane == 0) a.state[key] = s;
  if (active) {
    P p;
#pragma unroll
    for (int i = 0; i < E; ++i) p.x[i] = from_acc<T, A>(w[i]);  // (fp16: already rounded, exact)
    *reinterpret_cast<P *>(wrow) = p;
  }
}

// Staged walk of a very long fp16 row without stochastic rounding.  What is
// serial in such a row is one multiply-add and one rounding per occurrence and element; fetching
// the occurrence's gradient row and multiplier through lane reads and row requests costs the walking
// wavefront several times that.  So a workgroup takes the row: its first wavefront only walks --
// gradient rows and multipliers of a step's occurrences come out of LDS, at addresses known when
// the kernel is compiled -- while the third and fourth wavefront gather the next step's gradient
// rows into the other half of the LDS buffers (requested two steps before they are written
// there) and the second wavefront keeps the row's running state (the prefix sums over batches of
// 64 occurrences of walk_long_row: the same additions in the same order), forms the multipliers
// and looks up where the gradient rows are.  One barrier per step.  With per-sample weights the
// walking wavefront also starts <row, gradient row> of every occurrence -- the products summed over
// quads of lanes, off the chain of dependent updates -- and leaves the sixteen partial sums in LDS;
// a gathering thread per occurrence finishes them during the next step.
// Rows of up to 64 elements: one element per lane, 128 occurrences a step; rows of up to 128
// elements: two elements per lane, 64 occurrences a step (the same 16 KB of gradient rows).
constexpr int kStageStep = 128;  // most occurrences per step
constexpr int kStageD = 128;     // widest row walked this way
static_assert(kStageD == kApproxCoopD, "the width up to which rows are listed for a workgroup's walk");
constexpr int kStageElements = 128 * 64;  // elements of the gradient rows of one step
template <typename T, bool WEIGHTED> struct StageBuffers {
  alignas(16) T rows[2][kStageElements];  // [occurrence of the step][element of the row]
  alignas(16) float mult[2][kStageStep];
  // (per-sample weights) position of every occurrence -- where its grad_psw goes -- and the sixteen
  // sums over four lanes each of <row, gradient row>, left by the walk for the gathering wavefronts
  // ([occurrence][quad of lanes]: a thread reads its occurrence's sixteen sums as four 16-byte
  // pieces; measured faster than the transposed, padded layout whose reads are free of bank conflicts)
  alignas(16) int32_t pos[3][WEIGHTED ? kStageStep : 1];
  alignas(16) float partial[2][WEIGHTED ? kStageStep : 1][16];
  int64_t goff[4][kStageStep];  // first element of every occurrence's gradient row
};
template <typename T, int E, bool WEIGHTED>
__device__ __forceinline__ void staged_walk(const LongRowArgs<T> &a, int seg_begin, int seg_end, int64_t key,
                                            const RowPlace &place, T *storage, StageBuffers<T, WEIGHTED> &lds) {
  using A = typename AccOf<T>::type;
  static_assert(sizeof(T) == 2 && sizeof(A) == 4, "fp16 rows with fp32 arithmetic");
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = static_cast<int>(threadIdx.x >> 6);
  constexpr int kStep = kStageStep / E;  // occurrences per step
  constexpr int kRowD = kWave * E;       // elements of a staged row
  constexpr int kPerLane = kStep / kWave;  // occurrences of a step per lane of the bookkeeping wavefront
  const int len = seg_end - seg_begin;
  const int steps = (len + kStep - 1) / kStep;
  const int last = seg_end - 1;
  const bool active = lane * E < place.row_D;
  const int lane_off = active ? lane * E : 0;  // (idle lanes shadow lane 0 and store nothing)

  // ---- the second wavefront's bookkeeping: kPerLane occurrences of a step per lane
  A running = A(0);
  auto positions_of = [&](int step, int (&pos)[kPerLane]) {
#pragma unroll
    for (int h = 0; h < kPerLane; ++h) pos[h] = a.positions_sorted[min(seg_begin + step * kStep + h * kWave + lane, last)];
  };
  // (what a step's bookkeeping reads from memory is requested first, in one go, and used after the
  // step's gathering, so that a step costs the helpers one memory round trip)
  struct StepLoads {
    int grow[kPerLane];
    A wss[kPerLane];
    int pos[kPerLane];  // (WEIGHTED) the positions the multipliers belong to, and their per-sample weights
    A pw[kPerLane];
  };
  auto request_bookkeeping = [&](const int (&pos_offsets)[kPerLane], const int (&pos_multipliers)[kPerLane], StepLoads &l) {
#pragma unroll
    for (int h = 0; h < kPerLane; ++h) l.grow[h] = a.grad_rows[pos_offsets[h]];
#pragma unroll
    for (int h = 0; h < kPerLane; ++h) l.wss[h] = a.lookup_wss[pos_multipliers[h]];
#pragma unroll
    for (int h = 0; h < kPerLane; ++h) {
      l.pos[h] = pos_multipliers[h];
      l.pw[h] = A(1);
      if constexpr (WEIGHTED) l.pw[h] = to_acc(a.psw[pos_multipliers[h]]);
    }
  };
  auto write_offsets = [&](int step, const StepLoads &l) {
#pragma unroll
    for (int h = 0; h < kPerLane; ++h) lds.goff[step & 3][h * kWave + lane] = long_row_grad_offset(l.grow[h], place, a.mt);
  };
  auto write_multipliers = [&](int step, const StepLoads &l) {
#pragma unroll
    for (int h = 0; h < kPerLane; ++h) {
      const int nb = min(kWave, len - step * kStep - h * kWave);  // occurrences of this batch of 64
      if (nb > 0) {
        const A incl = wave_inclusive_sum<A>(lane < nb ? l.wss[h] : A(0));
        lds.mult[step & 1][h * kWave + lane] =
            lane < nb ? approx_multiplier<A>(running + incl, l.pw[h], WEIGHTED, a.lr, a.eps) : A(0);
        if constexpr (WEIGHTED) lds.pos[step % 3][h * kWave + lane] = l.pos[h];
        running = running + broadcast_lane(incl, nb - 1);
      }
    }
  };
  // ---- the gathering wavefronts (the third and fourth): 8-byte pieces of the rows, `pieces` (a
  // power of two) per row; a thread's pieces of a step are requested two steps before they are
  // written to LDS
  constexpr int kGatherThreads = kBlockThreads - 2 * kWave;
  const int helper = static_cast<int>(threadIdx.x) - 2 * kWave;
  int piece_shift = 0;
  while ((4 << piece_shift) < place.row_D) ++piece_shift;
  const int piece = helper & ((1 << piece_shift) - 1);
  const int rows_per_round = kGatherThreads >> piece_shift;  // at least 128 / (kRowD / 4)
  constexpr int kRounds = kStep / (kGatherThreads / (kRowD / 4));
  // (two sets of registers: the pieces of the steps b + 1 and b + 2 are on their way at a time)
  uint2 held_even[kRounds], held_odd[kRounds];
  auto request_rows = [&](int step, uint2 (&held)[kRounds]) {
    const int count = min(kStep, len - step * kStep);
    if (piece * 4 >= place.row_D || count <= 0) return;
    const int o0 = helper >> piece_shift;
#pragma unroll
    for (int k = 0; k < kRounds; ++k) {
      const int o = min(o0 + k * rows_per_round, count - 1);
      held[k] = *reinterpret_cast<const uint2 *>(a.grad_output + lds.goff[step & 3][o] + piece * 4);
    }
  };
  auto store_rows = [&](int step, const uint2 (&held)[kRounds]) {
    const int count = min(kStep, len - step * kStep);
    if (piece * 4 >= place.row_D) return;
    const int o0 = helper >> piece_shift;
#pragma unroll
    for (int k = 0; k < kRounds; ++k) {
      const int o = o0 + k * rows_per_round;
      if (o < count) *reinterpret_cast<uint2 *>(&lds.rows[step & 1][o * kRowD + piece * 4]) = held[k];
    }
  };

  // (per-sample weights) grad_psw of a walked step: a gathering thread per occurrence adds the sixteen
  // partial sums in order
  auto finish_dots = [&](int step) {
    if constexpr (WEIGHTED) {
      const int count = min(kStep, len - step * kStep);
      if (helper < count) {
        A dot = A(0);
#pragma unroll
        for (int q = 0; q < 16; ++q) dot += lds.partial[step & 1][helper][q];
        a.grad_psw[lds.pos[step % 3][helper]] = from_acc<T, A>(dot);
      }
    }
  };

  // Everything runs ahead of the walk by whole steps, and what comes from memory is requested two
  // steps before it is used (a step lasts about as long as one memory round trip), so that no
  // wavefront waits for memory inside a step.  While step b is walked: the rows of step b + 1
  // (requested during step b - 2) are written to LDS and those of step b + 3 requested; the
  // multipliers of step b + 1 and the row offsets of step b + 4 are formed from what was requested
  // during step b - 2; the state addends of step b + 3, the gradient row numbers of step b + 6 and
  // the positions of step b + 8 are requested.
  int pos3[kPerLane] = {}, pos4[kPerLane] = {}, pos5[kPerLane] = {}, pos6[kPerLane] = {}, pos7[kPerLane] = {};  // steps b + 3 .. b + 7
  StepLoads due{}, coming{};  // requested during the steps b - 2 and b - 1
  if (wave == 1) {
    int pos0[kPerLane], pos1[kPerLane], pos2[kPerLane];
    positions_of(0, pos0);
    positions_of(1, pos1);
    positions_of(2, pos2);
    positions_of(3, pos3);
    positions_of(4, pos4);
    positions_of(5, pos5);
    positions_of(6, pos6);
    positions_of(7, pos7);
    running = a.state[key];
    StepLoads first, second, third, fourth;
    request_bookkeeping(pos0, pos0, first);
    request_bookkeeping(pos1, pos1, second);
    request_bookkeeping(pos2, pos2, third);
    request_bookkeeping(pos3, pos3, fourth);
    write_offsets(0, first);
    write_multipliers(0, first);
    write_offsets(1, second);
    write_offsets(2, third);
    write_offsets(3, fourth);
    request_bookkeeping(pos4, pos1, due);     // (as if during step -2: offsets of step 4, multipliers of step 1)
    request_bookkeeping(pos5, pos2, coming);  // (as if during step -1)
  }
  __syncthreads();
  if (wave >= 2) {
    request_rows(0, held_even);
    store_rows(0, held_even);
    request_rows(1, held_odd);
    request_rows(2, held_even);
  }
  __syncthreads();

  A w[E];
#pragma unroll
  for (int i = 0; i < E; ++i) w[i] = to_acc(storage[lane_off + i]);
  // one step; `held`: the gathering threads' registers of step b + 1
  auto step_of_walk = [&](int b, uint2 (&held)[kRounds]) {
    if (wave == 0) {
      // eight occurrences at a time: the next eight are requested before the current eight are
      // applied (the barrier keeps the instruction scheduler from moving the requests back down).
      // The chain of dependent updates leaves the wavefront idle two thirds of the time, which is
      // where the ten LDS reads of eight occurrences go.
      const int count = min(kStep, len - b * kStep);
      const T *mine = &lds.rows[b & 1][lane_off];
      const float *mult = lds.mult[b & 1];
      float *my_partial = &lds.partial[b & 1][0][WEIGHTED ? lane >> 2 : 0];
      struct Eight {
        T g[8][E];
        float m[8];
      };
      auto fetch = [&](int first, Eight &e) {
#pragma unroll
        for (int k = 0; k < 8; ++k) __builtin_memcpy(&e.g[k][0], mine + (first + k) * kRowD, sizeof(T) * E);
        __builtin_memcpy(&e.m[0], mult + first, 16);
        __builtin_memcpy(&e.m[4], mult + first + 4, 16);
      };
      auto apply = [&](const Eight &e, int first, int limit) {
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          if (k < limit) {
            A dot = A(0);
#pragma unroll
            for (int i = 0; i < E; ++i) {
              const A g = to_acc(e.g[k][i]);
              if constexpr (WEIGHTED) dot += w[i] * g;  // (the row as the occurrences so far have left it)
              w[i] = w[i] - g * e.m[k];
              w[i] = __half2float(__float2half_rn(w[i]));
            }
            if constexpr (WEIGHTED) {
              // off the chain of dependent updates: the sum over the lane's quad by two lane moves,
              // left in LDS for a gathering thread to finish (the four lanes hold the same sum and
              // all write it: cheaper than masking three of them off)
              dot = active ? dot : A(0);
              dot += dpp_move<0xB1>(dot);
              dot += dpp_move<0x4E>(dot);
              my_partial[(first + k) * 16] = dot;
            }
          }
        }
      };
      Eight even, odd;
      fetch(0, even);
      if (count == kStep) {
#pragma unroll
        for (int first = 0; first < kStep; first += 16) {
          fetch(first + 8, odd);
          __builtin_amdgcn_sched_barrier(0);
          apply(even, first, 8);
          if (first + 16 < kStep) fetch(first + 16, even);
          __builtin_amdgcn_sched_barrier(0);
          apply(odd, first + 8, 8);
        }
      } else {
        for (int first = 0; first < count; first += 8) {
          apply(even, first, count - first);
          if (first + 8 < count) fetch(first + 8, even);
        }
      }
    } else {
      if (wave >= 2) {
        if (b + 1 < steps) store_rows(b + 1, held);
        request_rows(b + 3, held);
        if (b > 0) finish_dots(b - 1);
      } else {
        StepLoads requested{};
        request_bookkeeping(pos6, pos3, requested);  // (clamped positions: always valid)
        if (b + 1 < steps) write_multipliers(b + 1, due);
        if (b + 4 < steps) write_offsets(b + 4, due);
        due = coming;
        coming = requested;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          pos3[h] = pos4[h];
          pos4[h] = pos5[h];
          pos5[h] = pos6[h];
          pos6[h] = pos7[h];
        }
        positions_of(b + 8, pos7);
      }
    }
    // (the gathered rows are in LDS: a wavefront's reads have arrived before it writes them there)
    step_barrier();
  };
  for (int b = 0; b < steps; b += 2) {
    step_of_walk(b, held_odd);
    if (b + 1 < steps) step_of_walk(b + 1, held_even);
  }
  if (wave >= 2) finish_dots(steps - 1);  // (the last step's barrier is behind every wavefront)
  if (wave == 0 && active) {  // (already rounded: exact)
#pragma unroll
    for (int i = 0; i < E; ++i) storage[lane_off + i] = from_acc<T, A>(w[i]);
  }
  if (wave == 1 && lane == 0) a.state[key] = running;
}

// One wavefront per queued row (a row of at most 64 vectors with more occurrences than the kernel
// that queued it handles itself).  BIG: grad_output has 4 GiB or more, its rows are addressed
// with 64-bit offsets instead of through a buffer descriptor.
template <typename T, bool WEIGHTED, bool STOCHASTIC, bool BIG>
__global__ __launch_bounds__(kBlockThreads) void approx_adagrad_long_kernel(
    LongRowArgs<T> a, const int32_t *__restrict__ keys_sorted, const int32_t *__restrict__ segment_starts,
    const int32_t *__restrict__ counters, const int32_t *__restrict__ long_queue, int queue_capacity, int D,
    int mixed_huge_offset) {
  // (what is the same in every lane of the wavefront is told to the compiler, so that the walk's
  // control flow and addressing stay scalar)
  const int lane = threadIdx.x & (kWave - 1);
  const int wave_in_block = uniform(static_cast<int>(threadIdx.x >> 6));
  // queue_capacity == 0: one queue, its length in counters[1] (mixed-D tables: and, from
  // mixed_huge_offset on, the rows of more than kApproxHuge occurrences that a workgroup walks, their
  // number in counters[xcd_counter(0)]).  Otherwise, as the short-row kernel
  // leaves them: one queue per XCD (lengths in counters[xcd_counter(x)]) and behind them the
  // queue of the rows of more than kApproxHuge occurrences (counters[1]).  Those come first, one
  // per wavefront, so that the longest walks start when the kernel does.  Then the workgroups of
  // an XCD take their own queue in order -- it is in (table, row) order, so the gradient rows of a
  // table stay in that XCD's L2 while its rows are walked -- up to 1.5 times the average length;
  // what the longer queues hold beyond that is dealt to the wavefronts of all XCDs.  All of it is
  // index arithmetic on the queue lengths: no wavefront waits for another (outside the
  // cooperative walk below, whose wavefronts meet at workgroup barriers).
  // where a queued row is and what it looks like
  struct QueuedRow {
    int seg_begin, seg_end;
    int64_t key;
    RowPlace place;
    T *storage;
  };
  auto row_at = [&](int slot) {
    const int u = uniform(long_queue[slot]);
    QueuedRow r;
    r.seg_begin = uniform(segment_starts[u]);
    r.seg_end = uniform(segment_starts[u + 1]);
    r.key = uniform(keys_sorted[r.seg_begin]);
    const int first_grad_row = uniform(a.grad_rows[a.positions_sorted[r.seg_begin]]);
    r.place = a.mt.T > 0 ? place_row<true>(r.key, first_grad_row, D, a.mt)
                         : place_row<false>(r.key, first_grad_row, D, a.mt);
    r.place.row_D = uniform(r.place.row_D);
    r.place.row_element = uniform(r.place.row_element);
    r.place.grad_stride = uniform(r.place.grad_stride);
    r.place.grad_column = uniform(r.place.grad_column);
    r.storage = a.weights + r.place.row_element;
    if (a.unique_slots) {
      const int slot = uniform(a.unique_slots[u]);
      if (slot >= 0) r.storage = a.cache_rows + static_cast<int64_t>(slot) * a.slot_D;
    }
    return r;
  };
  int first_total = uniform(counters[1]);  // the rows every wavefront helps with first
  int block_index = static_cast<int>(blockIdx.x);
  int grid_blocks = static_cast<int>(gridDim.x);

  // Rows of more than kApproxHuge occurrences get a whole workgroup where that shortens the walk:
  // with stochastic rounding (rows at most kCoopD wide, see draw_step_bits), and for fp16 rows at
  // most kStageD wide without it (see staged_walk).  When the grid is large
  // enough, the first workgroups do nothing else -- as many as there are such rows, rounded up
  // to a multiple of the XCD count, at most half the grid -- and the others share the remaining
  // rows as if they were the whole grid.
  constexpr bool kStaged = !STOCHASTIC && sizeof(T) == 2;
  if constexpr (STOCHASTIC || kStaged) {
    using Shared = typename std::conditional<kStaged, StageBuffers<T, WEIGHTED>, uint16_t[2 * kCoopStep * kCoopD]>::type;
    __shared__ __align__(16) Shared s_shared;
    // (mixed-D tables: the strip kernel has listed the rows that qualify on their own)
    const bool mixed = a.mt.T > 0;
    const int huge_total = mixed ? uniform(counters[xcd_counter(0)]) : first_total;
    const int huge_base = mixed ? mixed_huge_offset : kNumXcd * queue_capacity;
    if ((mixed || (queue_capacity > 0 && D <= kApproxCoopD)) && huge_total > 0) {
      const bool dedicated = grid_blocks >= 2 * kNumXcd;
      const int coop_blocks =
          dedicated ? min((huge_total + kNumXcd - 1) / kNumXcd * kNumXcd, grid_blocks / (2 * kNumXcd) * kNumXcd) : 0;
      if (!dedicated || block_index < coop_blocks) {
        // these walks are the longest chains of the launch and share their SIMDs with the
        // wavefronts of other workgroups: they go first when both have an instruction ready
        __builtin_amdgcn_s_setprio(3);
        for (int h = block_index; h < huge_total; h += dedicated ? coop_blocks : grid_blocks) {
          const QueuedRow r = row_at(huge_base + h);
          if constexpr (kStaged) {
            if (r.place.row_D <= kWave) staged_walk<T, 1, WEIGHTED>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, s_shared);
            else staged_walk<T, 2, WEIGHTED>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, s_shared);
          } else {
            uint16_t *s_words = s_shared;
            const int len = r.seg_end - r.seg_begin;
            const int steps = (len + kCoopStep - 1) / kCoopStep;
            draw_step_bits(a.sr, r.place.row_element, r.place.row_D, 0, min(kCoopStep, len), s_words,
                           static_cast<int>(threadIdx.x), kBlockThreads);
            __syncthreads();
            if (wave_in_block == 0) {
              // (one barrier per step inside the walk)
              if (r.place.row_D <= kWave)
                walk_long_row<T, 1, WEIGHTED, true, BIG, true>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, lane, s_words);
              else
                walk_long_row<T, 2, WEIGHTED, true, BIG, true>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, lane, s_words);
            } else {
              for (int s = 1; s <= steps; ++s) {
                if (s < steps)
                  draw_step_bits(a.sr, r.place.row_element, r.place.row_D, s * kCoopStep,
                                 min(kCoopStep, len - s * kCoopStep), s_words + (s & 1) * (kCoopStep * kCoopD),
                                 static_cast<int>(threadIdx.x) - kWave, kBlockThreads - kWave);
                step_barrier();
              }
            }
          }
          __syncthreads();  // the buffers are free for the next row
        }
        if (dedicated) return;
        __builtin_amdgcn_s_setprio(0);
      }
      block_index -= coop_blocks;
      grid_blocks -= coop_blocks;
      if (!mixed) first_total = 0;
    }
  }

  const int xcd = block_index % kNumXcd;
  int queue_len[kNumXcd];
  int total = 0;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) {
    queue_len[x] = queue_capacity > 0 ? uniform(counters[xcd_counter(x)]) : 0;
    total += queue_len[x];
  }
  const int fair = total / kNumXcd + total / 16 + 1;
  int shared_total = 0;
#pragma unroll
  for (int x = 0; x < kNumXcd; ++x) shared_total += max(0, queue_len[x] - fair);
  const int own = min(queue_len[xcd], fair);
  int q = (block_index / kNumXcd) * kWavesPerBlock + wave_in_block;
  const int stride = (grid_blocks / kNumXcd) * kWavesPerBlock;
  const int all_stride = grid_blocks * kWavesPerBlock;
  int first = block_index * kWavesPerBlock + wave_in_block;
  int g = first;
  while (true) {
    int slot;
    if (first < first_total) {
      slot = kNumXcd * queue_capacity + first;
      first += all_stride;
    } else if (q < own) {
      slot = xcd * queue_capacity + q;
      q += stride;
    } else if (g < shared_total) {
      int before = 0, x = 0;
      while (g >= before + max(0, queue_len[x] - fair)) {
        before += max(0, queue_len[x] - fair);
        ++x;
      }
      slot = x * queue_capacity + fair + (g - before);
      g += all_stride;
    } else {
      break;
    }
    const QueuedRow r = row_at(slot);
    // elements per lane: the row spread over the 64 lanes, in loads of at most 16 bytes
    const int per_lane = (r.place.row_D + kWave - 1) / kWave;
    if (per_lane <= 1) walk_long_row<T, 1, WEIGHTED, STOCHASTIC, BIG>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, lane);
    else if (per_lane <= 2) walk_long_row<T, 2, WEIGHTED, STOCHASTIC, BIG>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, lane);
    else if constexpr (sizeof(T) <= 4) {
      if (per_lane <= 4) walk_long_row<T, 4, WEIGHTED, STOCHASTIC, BIG>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, lane);
      else if constexpr (sizeof(T) == 2) walk_long_row<T, 8, WEIGHTED, STOCHASTIC, BIG>(a, r.seg_begin, r.seg_end, r.key, r.place, r.storage, lane);
    }
  }
}

struct ApproxArgs {
  const void *grad_output;
  void *weights;
  void *state;
  const void *psw;
  void *grad_psw;
  int32_t dtype;
  int32_t vec;   // elements per vector (fp16: 8 or 4)
  int32_t D;     // uniform tables; 0 with mixed-D tables
  int64_t n;
  float lr, eps;
  MixedTables mt;
  StochasticRounding sr;
  const int32_t *offsets;  // [T * B + 1] first position of every bag
  int32_t B, T;
  // mixed-D tables: the rows of at most 64 vectors and kMixedShort occurrences are done and the
  // longer ones queued (update_mixed_approx_short); this queue holds the rows wider than 64 vectors
  const int32_t *wide_rows;
  // cache-fronted tables: slot of each unique row, the cache's rows (null otherwise) and their width
  const int32_t *unique_slots;
  void *cache_rows;
  int32_t slot_D;
};

template <typename T, int VEC>
void launch_approx(const ApproxArgs &a, const tbe_workspace_layout_t &l, char *ws, hipStream_t stream) {
  using A = typename AccOf<T>::type;
  auto i32 = [&](uint64_t off) { return reinterpret_cast<const int32_t *>(ws + off); };
  const bool mixed = a.D == 0;
  int group = kWave;
  if (!mixed) {
    const int chunks = a.D / VEC;
    group = 1;
    while (group < chunks && group < kWave) group <<= 1;
  }
  const int groups = kWave / group;
  const int64_t want = ceil_div(ceil_div(a.n, groups), kWavesPerBlock);
  const dim3 grid(static_cast<unsigned>(std::max<int64_t>(1, std::min<int64_t>(want, 256 * 64))));
  const dim3 block(kBlockThreads);
  // the queue of long rows borrows the exact update's chunk-record region (at least n / 17 records
  // of 32 bytes, against at most n / 17 queued rows of 4 bytes); its counter is word 1 of the
  // counter block, which the segment stage left at zero
  int32_t *counters = reinterpret_cast<int32_t *>(ws + l.num_unique);
  int32_t *long_queue = reinterpret_cast<int32_t *>(ws + l.chunk_segments);
  const int64_t most_long = a.n / (kApproxShortSegment + 1) + 1;  // (the short-row kernel queues rows of 17 and more)
  // (a multiple of the XCD count, so that every XCD has the same number of workgroups)
  const dim3 grid_long(static_cast<unsigned>(
      kNumXcd * std::max<int64_t>(1, std::min<int64_t>(ceil_div(most_long, kWavesPerBlock * kNumXcd), 256))));
  // uniform tables whose rows fit a wavefront: the short-row kernel fills one queue per XCD
  const int queue_capacity =
      (!mixed && approx_short_serves(a.dtype, a.D)) ? static_cast<int>(approx_long_queue_capacity(a.n)) : 0;

  const dim3 block_long(kBlockThreads);
  // the queued rows' kernel reads the state addend of every lookup from the sort's ping-pong
  // buffers (8 bytes per lookup, free once the batch is sorted)
  A *lookup_wss = reinterpret_cast<A *>(ws + l.sort_scratch);
  const int64_t bags = static_cast<int64_t>(a.B) * a.T;
  const dim3 grid_norms(static_cast<unsigned>(ceil_div(ceil_div(bags, groups), kWavesPerBlock)));
  const uint64_t grad_bytes = static_cast<uint64_t>(a.B) * (mixed ? a.mt.total_D : static_cast<int64_t>(a.T) * a.D) * sizeof(T);
  MixedTables long_tables = a.mt;
  if (!mixed) long_tables.T = 0;
  LongRowArgs<T> la{static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights), static_cast<A *>(a.state),
                    static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw), i32(l.positions_sorted),
                    i32(l.grad_rows), lookup_wss, a.lr, a.eps, long_tables, a.sr, grad_bytes, a.unique_slots,
                    static_cast<T *>(a.cache_rows), a.slot_D};
  const bool big = grad_bytes >= (1ull << 32);
  const bool stochastic = sizeof(T) == 2 && a.sr.enabled;
#define TBE_APPROX_LONG_KERNEL(WEIGHTED, STOCHASTIC, BIG)                                              \
  TBE_LAUNCH("update_approx_long", stream, (approx_adagrad_long_kernel<T, WEIGHTED, STOCHASTIC, BIG>), \
             grid_long, block_long, la, i32(l.keys_sorted), i32(l.segment_starts), counters,           \
             long_queue, queue_capacity, a.D, static_cast<int>(approx_mixed_huge_offset(a.n)))
#define TBE_APPROX_LONG(WEIGHTED, MIXED)                                                               \
  TBE_LAUNCH("update_approx_norms", stream, (approx_lookup_norms_kernel<T, VEC, WEIGHTED, MIXED>),     \
             grid_norms, block, static_cast<const T *>(a.grad_output), static_cast<const T *>(a.psw),  \
             a.offsets, counters, lookup_wss, a.B, a.T, a.D, group, a.mt);                             \
  if (stochastic) {                                                                                    \
    if (big) { TBE_APPROX_LONG_KERNEL(WEIGHTED, sizeof(T) == 2, true); }                               \
    else { TBE_APPROX_LONG_KERNEL(WEIGHTED, sizeof(T) == 2, false); }                                  \
  } else {                                                                                             \
    if (big) { TBE_APPROX_LONG_KERNEL(WEIGHTED, false, true); }                                        \
    else { TBE_APPROX_LONG_KERNEL(WEIGHTED, false, false); }                                           \
  }
#define TBE_APPROX(WEIGHTED, MIXED)                                                                    \
  TBE_LAUNCH("update_approx", stream, (approx_adagrad_kernel<T, VEC, WEIGHTED, MIXED>), grid, block,   \
             static_cast<const T *>(a.grad_output), static_cast<T *>(a.weights),                       \
             static_cast<A *>(a.state), static_cast<const T *>(a.psw), static_cast<T *>(a.grad_psw),   \
             i32(l.keys_sorted), i32(l.positions_sorted), i32(l.grad_rows), i32(l.segment_starts),     \
             counters, long_queue, a.D, group, a.lr, a.eps, a.mt, a.sr, a.wide_rows, a.unique_slots,   \
             static_cast<T *>(a.cache_rows), a.slot_D);                                                \
  TBE_APPROX_LONG(WEIGHTED, MIXED)
  if (mixed) {
    if (a.psw) { TBE_APPROX(true, true); }
    else { TBE_APPROX(false, true); }
  } else if (approx_short_serves(a.dtype, a.D)) {
    // uniform tables whose rows fit a wavefront: rows of up to kApproxShortSegment occurrences go through
    // the exact update's position-balanced short-row kernel in its per-lookup form, the others
    // (queued by it) get a wavefront each
    UpdateArgs ua{};
    ua.grad_output = a.grad_output;
    ua.weights = a.weights;
    ua.optimizer_state = a.state;
    ua.per_sample_weights = a.psw;
    ua.grad_per_sample_weights = a.grad_psw;
    ua.keys_sorted = i32(l.keys_sorted);
    ua.positions_sorted = i32(l.positions_sorted);
    ua.grad_rows = i32(l.grad_rows);
    ua.segment_starts = i32(l.segment_starts);
    ua.counters = counters;
    ua.segment_ids = i32(l.segment_ids);
    ua.num_indices = a.n;
    ua.dtype = a.dtype;
    ua.D = a.D;
    ua.optimizer = kOptAdagrad;
    ua.learning_rate = a.lr;
    ua.eps = a.eps;
    ua.stochastic_rounding = a.sr;
    ua.unique_slots = a.unique_slots;
    ua.cache_rows = a.cache_rows;
    if (approx_sums_long_rows(a.dtype, a.D, a.psw != nullptr)) {
      // fp32 / fp64 rows without per-sample weights: the update of a row is a weighted sum of its
      // gradient rows, so the longer rows are summed in chunks like the exact update's
      ua.long_segments = ws + l.long_segments;
      ua.chunk_segments = ws + l.chunk_segments;
      ua.partial_sums = ws + l.partial_sums;
      ua.max_long = l.max_long_segments;
      ua.max_chunks = l.max_chunks;
      (void)segment_update_approx_short(ua, nullptr, stream);
      TBE_LAUNCH("update_approx_norms", stream, (approx_lookup_norms_kernel<T, VEC, false, false>), grid_norms,
                 block, static_cast<const T *>(a.grad_output), static_cast<const T *>(nullptr), a.offsets, counters,
                 lookup_wss, a.B, a.T, a.D, group, a.mt);
      (void)segment_update_approx_sum_long(ua, lookup_wss, stream);
    } else {
      (void)segment_update_approx_short(ua, long_queue, stream);
      if (a.psw) { TBE_APPROX_LONG(true, false); }
      else { TBE_APPROX_LONG(false, false); }
    }
  } else {
    if (a.psw) { TBE_APPROX(true, false); }
    else { TBE_APPROX(false, false); }
  }
#undef TBE_APPROX_LONG
#undef TBE_APPROX_LONG_KERNEL
#undef TBE_APPROX
}

}  // namespace

// Runs the approximate update on a workspace that already holds the batch's plan
// (gradient rows, sorted keys and positions, run boundaries).
int approx_update(const void *grad_output, void *weights, void *state, const void *psw, void *grad_psw,
                  int32_t dtype, int32_t fp16_vector_width, int32_t D, int64_t n, float lr, float eps,
                  const int64_t *mixed_table_offsets, const int32_t *table_dim_offsets,
                  const int32_t *dim_offsets, int32_t total_D, int32_t T, const int32_t *offsets, int32_t B,
                  StochasticRounding sr, const tbe_workspace_layout_t &l, void *workspace, hipStream_t stream,
                  const int32_t *unique_slots, void *cache_rows, int32_t slot_D) {
  ApproxArgs a{grad_output, weights, state, psw, grad_psw, dtype, fp16_vector_width, D, n, lr, eps,
               MixedTables{mixed_table_offsets, table_dim_offsets, dim_offsets, total_D, T}, sr, offsets, B, T,
               D == 0 ? approx_mixed_wide_queue(l, workspace) : nullptr, unique_slots, cache_rows,
               D == 0 ? slot_D : D};
  char *ws = static_cast<char *>(workspace);
  // the queues of long rows borrow the chunk records' region: eight of approx_long_queue_capacity()
  // rows and one of the rows of more than kApproxHuge occurrences, or one queue of at most n / 9 rows
  const uint64_t queue_words = static_cast<uint64_t>(kNumXcd) * approx_long_queue_capacity(n) +
                               static_cast<uint64_t>(n) / (kApproxHuge + 1) + 1 + static_cast<uint64_t>(n) / 9;
  if (queue_words * 4 > static_cast<uint64_t>(l.max_chunks) * 32)
    return fail(TBE_ERR_WORKSPACE, "tbe approximate Adagrad update: queues of %llu rows do not fit the workspace",
                (unsigned long long)queue_words);
  switch (dtype) {
    case TBE_DTYPE_F32: launch_approx<float, 4>(a, l, ws, stream); break;
    case TBE_DTYPE_F16:
      if (a.vec == 8) launch_approx<__half, 8>(a, l, ws, stream);
      else launch_approx<__half, 4>(a, l, ws, stream);
      break;
    default: launch_approx<double, 2>(a, l, ws, stream); break;
  }
  return check_launch("tbe approximate Adagrad update");
}

}  // namespace tbe

extern "C" int tbe_backward_approx_adagrad(const void *grad_output, void *weights, int32_t dtype,
                                           int64_t total_rows, int64_t max_table_rows, int32_t D,
                                           const int32_t *table_offsets, int32_t T,
                                           const int32_t *indices, int64_t num_indices,
                                           const int32_t *offsets, int32_t B,
                                           const void *per_sample_weights, void *optimizer_state,
                                           float learning_rate, float eps,
                                           void *grad_per_sample_weights,
                                           int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                           void *workspace, uint64_t workspace_bytes, void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_approx_adagrad";
  TBE_REQUIRE(T > 0, "%s: T must be positive (got %d)", name, T);
  TBE_REQUIRE(B > 0, "%s: B must be positive (got %d)", name, B);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(max_table_rows >= 0, "%s: max_table_rows must not be negative", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "%s: T*B out of range", name);
  TBE_REQUIRE(grad_output && weights && table_offsets && offsets && optimizer_state, "%s: null pointer argument", name);
  TBE_REQUIRE(indices || num_indices == 0, "%s: indices is null but num_indices > 0", name);
  TBE_REQUIRE((per_sample_weights == nullptr) == (grad_per_sample_weights == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, D, dtype, T, &l);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (int rc = build_plan(l, workspace, table_offsets, T, indices, num_indices, offsets, B, total_rows,
                          max_table_rows, s))
    return rc;
  const RowGeometry g = row_geometry(dtype, D);
  return approx_update(grad_output, weights, optimizer_state, per_sample_weights, grad_per_sample_weights,
                       dtype, g.vec, D, num_indices, learning_rate, eps, nullptr, nullptr, nullptr, 0, T, offsets, B,
                       StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0},
                       l, workspace, s);
}

extern "C" int tbe_backward_approx_cached(const void *grad_output, const tbe_cache_t *cache, int32_t dtype,
                                          int64_t total_rows, int32_t D, int32_t T, int32_t B,
                                          int64_t num_indices, const int32_t *offsets,
                                          const void *per_sample_weights, void *optimizer_state,
                                          float learning_rate, float eps, void *grad_per_sample_weights,
                                          int32_t stochastic_rounding, uint64_t seed, uint64_t offset,
                                          void *workspace, uint64_t workspace_bytes,
                                          const int32_t *unique_slots, void *stream) {
  using namespace tbe;
  const char *name = "tbe_backward_approx_cached";
  TBE_REQUIRE(cache && cache->rows && cache->backing_rows, "%s: null cache", name);
  TBE_REQUIRE(T > 0 && B > 0, "%s: T and B must be positive (got %d, %d)", name, T, B);
  TBE_REQUIRE(D > 0 && D % 4 == 0, "%s: D must be a positive multiple of 4 (got %d)", name, D);
  TBE_REQUIRE(dtype >= TBE_DTYPE_F32 && dtype <= TBE_DTYPE_F64, "%s: bad dtype %d", name, dtype);
  TBE_REQUIRE(total_rows > 0 && total_rows < INT32_MAX, "%s: total_rows out of range", name);
  TBE_REQUIRE(num_indices >= 0 && num_indices < INT32_MAX, "%s: num_indices out of range", name);
  TBE_REQUIRE(grad_output && offsets && optimizer_state, "%s: null pointer argument", name);
  TBE_REQUIRE(unique_slots || num_indices == 0, "%s: null unique_slots", name);
  TBE_REQUIRE((per_sample_weights == nullptr) == (grad_per_sample_weights == nullptr),
              "%s: per_sample_weights and grad_per_sample_weights must both be given or both be null", name);
  if (num_indices == 0) return TBE_OK;
  tbe_workspace_layout_t l;
  backward_layout(num_indices, D, dtype, T, &l);
  if (!workspace || workspace_bytes < l.total_bytes)
    return fail(TBE_ERR_WORKSPACE, "%s: workspace of %llu bytes needed, %llu given", name,
                (unsigned long long)l.total_bytes, (unsigned long long)workspace_bytes);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RowGeometry g = row_geometry(dtype, D);
  if (int rc = approx_update(grad_output, cache->backing_rows, optimizer_state, per_sample_weights,
                             grad_per_sample_weights, dtype, g.vec, D, num_indices, learning_rate, eps, nullptr,
                             nullptr, nullptr, 0, T, offsets, B,
                             StochasticRounding{seed, offset, (stochastic_rounding && dtype == TBE_DTYPE_F16) ? 1 : 0},
                             l, workspace, s, unique_slots, cache->rows))
    return rc;
  if (cache->stage_slots <= 0) return TBE_OK;
  const char *ws = static_cast<const char *>(workspace);
  return cache_unstage(cache, dtype, D, reinterpret_cast<const int32_t *>(ws + l.keys_sorted),
                       reinterpret_cast<const int32_t *>(ws + l.segment_starts),
                       reinterpret_cast<const int32_t *>(ws + l.num_unique), unique_slots, num_indices, s);
}
