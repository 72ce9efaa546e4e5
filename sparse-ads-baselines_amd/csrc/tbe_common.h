// Shared device helpers and host-side plumbing for the gfx950 TBE kernels.
#pragma once

#include <hip/hip_fp16.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tbe_hip.h"

namespace tbe {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr int kBlockThreads = 256;  // 4 wavefronts per workgroup
constexpr int kWavesPerBlock = kBlockThreads / kWave;
constexpr int kNumXcd = 8;          // MI355X: 8 XCDs, workgroups are dealt round-robin

// ---------------------------------------------------------------- host side
// Records `msg` as this thread's last error and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
int check_launch(const char *what);

#define TBE_REQUIRE(cond, ...)                                  \
  do {                                                          \
    if (!(cond)) return ::tbe::fail(TBE_ERR_INVALID, __VA_ARGS__); \
  } while (0)

// Per-kernel timing for benchmarks: between tbe_profile_begin() and tbe_profile_end()
// every launch is bracketed by HIP events recorded on the launch stream.
struct LaunchTimer {
  LaunchTimer(const char *name, hipStream_t stream);
  ~LaunchTimer();
  int slot;
  hipStream_t stream;
};

#define TBE_LAUNCH(name, stream, kernel, grid, block, ...)                     \
  do {                                                                         \
    ::tbe::LaunchTimer tbe_launch_timer(name, stream);                         \
    hipLaunchKernelGGL(kernel, grid, block, 0, stream, __VA_ARGS__);           \
  } while (0)

inline uint64_t align_up(uint64_t x, uint64_t a) { return (x + a - 1) / a * a; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Geometry of one embedding row spread over the lanes of a wavefront.
// A row is `chunks` vectors of VEC elements (16 bytes where alignment allows);
// `chunks` consecutive lanes form a lane group that owns one row at a time, and
// a wavefront holds floor(64 / chunks) groups.  Rows wider than 64 vectors are
// handled by the whole wavefront looping over column blocks.
struct RowGeometry {
  int vec;        // elements per lane per access
  int chunks;     // D / vec
  int tmpl;       // chunks if it is a power of two <= 64 (compile-time variant), else 0
  bool wide;      // chunks > 64
};

inline RowGeometry row_geometry(int32_t dtype, int32_t D) {
  RowGeometry g;
  if (dtype == TBE_DTYPE_F16) g.vec = (D % 8 == 0) ? 8 : 4;
  else if (dtype == TBE_DTYPE_F32) g.vec = 4;
  else g.vec = 2;
  g.chunks = D / g.vec;
  g.wide = g.chunks > kWave;
  g.tmpl = (!g.wide && (g.chunks & (g.chunks - 1)) == 0) ? g.chunks : 0;
  return g;
}

inline size_t dtype_size(int32_t dtype) {
  return dtype == TBE_DTYPE_F16 ? 2 : dtype == TBE_DTYPE_F32 ? 4 : 8;
}
inline size_t acc_size(int32_t dtype) { return dtype == TBE_DTYPE_F64 ? 8 : 4; }

// -------------------------------------------------------------- device side
template <typename T> struct AccOf { using type = float; };
template <> struct AccOf<double> { using type = double; };

// Raw storage of VEC consecutive elements, loaded/stored with one instruction.
template <typename T, int VEC> struct Raw;
template <> struct Raw<float, 4> { using type = float4; };
template <> struct Raw<__half, 8> { using type = uint4; };
template <> struct Raw<__half, 4> { using type = uint2; };
template <> struct Raw<double, 2> { using type = double2; };

template <typename T, int VEC> struct RowVec {
  using A = typename AccOf<T>::type;
  using R = typename Raw<T, VEC>::type;
  A v[VEC];

  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < VEC; ++i) v[i] = A(0);
  }
  __device__ __forceinline__ static R load_raw(const T *p) {
    return *reinterpret_cast<const R *>(p);
  }
  // Streaming variants: the data is touched once, so it should not displace reusable lines.
  __device__ __forceinline__ static R load_raw_streaming(const T *p) {
    using Words = uint32_t __attribute__((ext_vector_type(sizeof(R) / 4)));
    const Words w = __builtin_nontemporal_load(reinterpret_cast<const Words *>(p));
    R r;
    __builtin_memcpy(&r, &w, sizeof(R));
    return r;
  }
  __device__ __forceinline__ void load_streaming(const T *p) { unpack(load_raw_streaming(p)); }
  __device__ __forceinline__ void store_streaming(T *p) const {
    using Words = uint32_t __attribute__((ext_vector_type(sizeof(R) / 4)));
    const R r = pack();
    Words w;
    __builtin_memcpy(&w, &r, sizeof(R));
    __builtin_nontemporal_store(w, reinterpret_cast<Words *>(p));
  }
  __device__ __forceinline__ void unpack(const R &r);
  __device__ __forceinline__ R pack() const;
  __device__ __forceinline__ void load(const T *p) { unpack(load_raw(p)); }
  __device__ __forceinline__ void store(T *p) const { *reinterpret_cast<R *>(p) = pack(); }
};

template <> __device__ __forceinline__ void RowVec<float, 4>::unpack(const float4 &r) {
  v[0] = r.x; v[1] = r.y; v[2] = r.z; v[3] = r.w;
}
template <> __device__ __forceinline__ float4 RowVec<float, 4>::pack() const {
  return make_float4(v[0], v[1], v[2], v[3]);
}
template <> __device__ __forceinline__ void RowVec<double, 2>::unpack(const double2 &r) {
  v[0] = r.x; v[1] = r.y;
}
template <> __device__ __forceinline__ double2 RowVec<double, 2>::pack() const {
  return make_double2(v[0], v[1]);
}

__device__ __forceinline__ void half2_to_floats(uint32_t bits, float &lo, float &hi) {
  __half2 h = *reinterpret_cast<const __half2 *>(&bits);
  float2 f = __half22float2(h);
  lo = f.x; hi = f.y;
}
// Round-to-nearest-even, the rounding the reference uses when it stores fp16
// (__float22half2_rn, table_batched_embeddings_cuda.cu:81-82).
__device__ __forceinline__ uint32_t floats_to_half2(float lo, float hi) {
  __half2 h = __floats2half2_rn(lo, hi);
  return *reinterpret_cast<const uint32_t *>(&h);
}
template <> __device__ __forceinline__ void RowVec<__half, 8>::unpack(const uint4 &r) {
  half2_to_floats(r.x, v[0], v[1]); half2_to_floats(r.y, v[2], v[3]);
  half2_to_floats(r.z, v[4], v[5]); half2_to_floats(r.w, v[6], v[7]);
}
template <> __device__ __forceinline__ uint4 RowVec<__half, 8>::pack() const {
  return make_uint4(floats_to_half2(v[0], v[1]), floats_to_half2(v[2], v[3]),
                    floats_to_half2(v[4], v[5]), floats_to_half2(v[6], v[7]));
}
template <> __device__ __forceinline__ void RowVec<__half, 4>::unpack(const uint2 &r) {
  half2_to_floats(r.x, v[0], v[1]); half2_to_floats(r.y, v[2], v[3]);
}
template <> __device__ __forceinline__ uint2 RowVec<__half, 4>::pack() const {
  return make_uint2(floats_to_half2(v[0], v[1]), floats_to_half2(v[2], v[3]));
}

// ------------------------------------------------------------ stochastic rounding
// Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3", SC'11), the
// generator behind curandStatePhilox4_32_10_t that the reference draws its rounding bits from
// (table_batched_embeddings_cuda.cu:595-599, 627-631).
__device__ __forceinline__ uint4 philox4x32_10(uint4 ctr, uint2 key) {
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    // (one 32 x 32 -> 64-bit multiplication per product instead of a high and a low one)
    const uint64_t p0 = static_cast<uint64_t>(0xD2511F53u) * ctr.x;
    const uint64_t p1 = static_cast<uint64_t>(0xCD9E8D57u) * ctr.z;
    const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
    const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
    ctr = make_uint4(hi1 ^ ctr.y ^ key.x, lo1, hi0 ^ ctr.w ^ key.y, lo0);
    key.x += 0x9E3779B9u;
    key.y += 0xBB67AE85u;
  }
  return ctr;
}

struct StochasticRounding {
  uint64_t seed;     // Philox key
  uint64_t offset;   // high half of the Philox counter: one value per backward call
  int32_t enabled;
};

// fp32 -> fp16 with stochastic rounding as in stochastic_rounding_vector
// (table_batched_embeddings_cuda.cu:564-578): 13 random bits are added to the fp32 pattern,
// then the value is truncated toward zero.
// fp32 -> fp16 toward zero: the hardware's packed conversion (v_cvt_pkrtz_f16_f32), which rounds
// toward zero whatever the rounding mode and returns, for every one of the 2^32 fp32 patterns,
// the bits of __float2half_rz (checked exhaustively): finite magnitudes beyond the largest fp16
// value stay at it, values below the smallest normal one become subnormals, infinities and NaNs
// convert as they are.
typedef __fp16 HalfPairRz __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t floats_to_half2_rz_bits(float lo, float hi) {
  const HalfPairRz h = __builtin_amdgcn_cvt_pkrtz(lo, hi);
  return __builtin_bit_cast(uint32_t, h);
}
__device__ __forceinline__ uint16_t float_to_half_rz_bits(float x) {
  return static_cast<uint16_t>(floats_to_half2_rz_bits(x, 0.0f) & 0xffffu);
}
// one value rounded stochastically to fp16 and back: `bits` are the 13 random bits of the element
// (the top 13 of its random word), added below the fp16 mantissa before the cut toward zero
__device__ __forceinline__ float round_trip_with_bits(float v, uint32_t bits) {
  return __half2float(__ushort_as_half(float_to_half_rz_bits(__uint_as_float(__float_as_uint(v) + bits))));
}
__device__ __forceinline__ float round_trip_stochastic(float v, uint32_t word) {
  return round_trip_with_bits(v, word >> 19);
}

__device__ __forceinline__ uint32_t floats_to_half2_stochastic(float lo, float hi, uint32_t r0, uint32_t r1) {
  return floats_to_half2_rz_bits(__uint_as_float(__float_as_uint(lo) + (r0 >> 19)),
                                 __uint_as_float(__float_as_uint(hi) + (r1 >> 19)));
}

// VEC accumulator values packed into the stored type: round to nearest even, or, for fp16 with
// stochastic rounding enabled, element e of the table (e = row * D + column, a multiple of 4)
// takes word (e % 4) of Philox(counter = {e / 4, offset}, key = seed), so the bits depend on the
// element and the call, not on the launch geometry.
template <typename T, int VEC>
__device__ __forceinline__ typename RowVec<T, VEC>::R pack_rounded(const RowVec<T, VEC> &v,
                                                                   const StochasticRounding &sr,
                                                                   int64_t element) {
  if constexpr (sizeof(T) == 2) {
    if (sr.enabled) {
      uint32_t words[VEC / 2];
#pragma unroll
      for (int q = 0; q < VEC / 4; ++q) {
        const uint64_t group = static_cast<uint64_t>(element) / 4 + q;
        const uint4 r = philox4x32_10(
            make_uint4(static_cast<uint32_t>(group), static_cast<uint32_t>(group >> 32),
                       static_cast<uint32_t>(sr.offset), static_cast<uint32_t>(sr.offset >> 32)),
            make_uint2(static_cast<uint32_t>(sr.seed), static_cast<uint32_t>(sr.seed >> 32)));
        words[2 * q] = floats_to_half2_stochastic(v.v[4 * q], v.v[4 * q + 1], r.x, r.y);
        words[2 * q + 1] = floats_to_half2_stochastic(v.v[4 * q + 2], v.v[4 * q + 3], r.z, r.w);
      }
      typename RowVec<T, VEC>::R raw;
      __builtin_memcpy(&raw, words, sizeof(raw));
      return raw;
    }
  }
  return v.pack();
}

// Stores VEC accumulator values at p, rounded as pack_rounded does.
template <typename T, int VEC, bool STREAMING>
__device__ __forceinline__ void store_row(T *p, const RowVec<T, VEC> &v, const StochasticRounding &sr,
                                          int64_t element) {
  if constexpr (sizeof(T) == 2) {
    if (sr.enabled) {
      *reinterpret_cast<typename RowVec<T, VEC>::R *>(p) = pack_rounded<T, VEC>(v, sr, element);
      return;
    }
  }
  if constexpr (STREAMING) v.store_streaming(p);
  else v.store(p);
}

__device__ __forceinline__ float to_acc(float x) { return x; }
__device__ __forceinline__ float to_acc(__half x) { return __half2float(x); }
__device__ __forceinline__ double to_acc(double x) { return x; }
template <typename T, typename A> __device__ __forceinline__ T from_acc(A x);
template <> __device__ __forceinline__ float from_acc<float, float>(float x) { return x; }
template <> __device__ __forceinline__ __half from_acc<__half, float>(float x) { return __float2half_rn(x); }
template <> __device__ __forceinline__ double from_acc<double, double>(double x) { return x; }

__device__ __forceinline__ float shfl_idx(float v, int src) { return __shfl(v, src, kWave); }
__device__ __forceinline__ int shfl_idx(int v, int src) { return __shfl(v, src, kWave); }
__device__ __forceinline__ double shfl_idx(double v, int src) { return __shfl(v, src, kWave); }
__device__ __forceinline__ int64_t shfl_idx(int64_t v, int src) {
  return static_cast<int64_t>(__shfl(static_cast<long long>(v), src, kWave));
}
__device__ __forceinline__ float shfl_x(float v, int m) { return __shfl_xor(v, m, kWave); }
__device__ __forceinline__ double shfl_x(double v, int m) { return __shfl_xor(v, m, kWave); }

// The packed vector of a lane that holds no lookup becomes zeros, so that what follows is the same
// multiply-add for every lane (a select on the packed words costs half of one on the converted values,
// and leaves the conversion and the addition to one mixed-precision instruction).
template <typename R> __device__ __forceinline__ void keep_if(R &raw, bool keep) {
  static_assert(sizeof(R) % 4 == 0, "whole registers");
  uint32_t words[sizeof(R) / 4];
  __builtin_memcpy(words, &raw, sizeof(R));
#pragma unroll
  for (size_t i = 0; i < sizeof(R) / 4; ++i) words[i] = keep ? words[i] : 0u;
  __builtin_memcpy(&raw, words, sizeof(R));
}
// <a, b> over the VEC elements a lane holds, as up to four independent partial sums that are added in a
// fixed tree (a single chain of VEC dependent multiply-adds keeps the vector ALU waiting for itself).
template <int VEC, typename A>
__device__ __forceinline__ A lane_dot(const A (&a)[VEC], const A (&b)[VEC]) {
  constexpr int kParts = VEC < 4 ? VEC : 4;
  A part[kParts];
#pragma unroll
  for (int i = 0; i < kParts; ++i) part[i] = a[i] * b[i];
#pragma unroll
  for (int i = kParts; i < VEC; ++i) part[i % kParts] += a[i] * b[i];
  if constexpr (kParts == 4) return (part[0] + part[1]) + (part[2] + part[3]);
  else if constexpr (kParts == 2) return part[0] + part[1];
  else return part[0];
}
// The value as the compiler must take it: a register it knows nothing about.  Used where the instruction
// selection should convert THIS operand once instead of folding its conversion into every use.
__device__ __forceinline__ float opaque(float x) {
  asm volatile("" : "+v"(x));
  return x;
}
__device__ __forceinline__ double opaque(double x) { return x; }

// Sum of `v` over the `chunks` lanes of the caller's lane group; every lane of
// the group gets the result.  CHUNKS > 0: power-of-two group, xor butterfly that
// never leaves the group.  CHUNKS == 0: arbitrary group size, every lane adds the
// group's values in lane order (`group_base` = first lane of the group).
// Lanes exchanged inside a row of 16 by the data-parallel-primitive path of the vector ALU (no LDS
// crossbar, no address arithmetic): 0xB1 = quad_perm [1,0,3,2] (lane ^ 1), 0x4E = quad_perm [2,3,0,1]
// (lane ^ 2), 0x141 = row_half_mirror (lane i of a group of 8 reads lane 7 - i), 0x140 = row_mirror
// (lane i of a row of 16 reads lane 15 - i).
template <int CTRL> __device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int CTRL> __device__ __forceinline__ double dpp_move(double v) {
  const long long bits = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(bits), CTRL, 0xF, 0xF, false);
  const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(bits >> 32), CTRL, 0xF, 0xF, false);
  return __builtin_bit_cast(double, (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}
template <int CHUNKS, typename A>
__device__ __forceinline__ A group_sum(A v, int chunks, int group_base) {
  if constexpr (CHUNKS > 0) {
    // pairs, quads, then -- every lane of a quad (of eight lanes) holding the same sum by then -- the mirrored
    // quad (eight lanes); wider groups finish with lane shuffles
    if constexpr (CHUNKS >= 2) v += dpp_move<0xB1>(v);
    if constexpr (CHUNKS >= 4) v += dpp_move<0x4E>(v);
    if constexpr (CHUNKS >= 8) v += dpp_move<0x141>(v);
    if constexpr (CHUNKS >= 16) v += dpp_move<0x140>(v);
#pragma unroll
    for (int m = 16; m < CHUNKS; m <<= 1) v += shfl_x(v, m);
    return v;
  } else {
    A s = A(0);
    for (int j = 0; j < chunks; ++j) s += shfl_idx(v, group_base + j);
    return s;
  }
}

// Sum over the 64 lanes of a wavefront without a trip through LDS: the rows of 16 lanes as in
// group_sum, then the sum of row 0 into row 1 and of row 2 into row 3 (0x142 = row_bcast:15: lane
// 15 of a row to the next row), then the sum of rows 0 and 1 into rows 2 and 3 (0x143 =
// row_bcast:31).  The total ends up in the lanes 48..63.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_rows(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ double dpp_rows(double v) {
  const long long bits = __builtin_bit_cast(long long, v);
  const int lo = __builtin_amdgcn_update_dpp(0, static_cast<int>(bits), CTRL, ROW_MASK, 0xF, false);
  const int hi = __builtin_amdgcn_update_dpp(0, static_cast<int>(bits >> 32), CTRL, ROW_MASK, 0xF, false);
  return __builtin_bit_cast(double, (static_cast<long long>(hi) << 32) | static_cast<unsigned int>(lo));
}
template <typename A> __device__ __forceinline__ A wave_sum_in_last_row(A v) {
  v = group_sum<16, A>(v, 16, 0);
  v += dpp_rows<0x142, 0xA>(v);  // (rows 1 and 3 take the row before them; the others add zero)
  v += dpp_rows<0x143, 0xC>(v);  // (rows 2 and 3 take row 1)
  return v;
}

// Workgroups are dealt to the 8 XCDs round-robin by blockIdx.  This maps
// blockIdx to a logical work index so that each XCD walks one contiguous
// eighth of the work: consecutive bags / segments (same table, neighbouring
// hot rows) then share one XCD's L2 instead of being replicated in all eight.
// `per_xcd` = ceil(num_work / 8); the grid must hold 8 * per_xcd workgroups
// and indices >= num_work are idle.
__device__ __forceinline__ int64_t xcd_contiguous(int64_t block, int64_t per_xcd) {
  return (block % kNumXcd) * per_xcd + block / kNumXcd;
}

}  // namespace tbe
