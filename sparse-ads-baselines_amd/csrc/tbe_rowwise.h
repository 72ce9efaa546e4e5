// Arithmetic shared by the exact and the approximate row-wise Adagrad kernels.
#pragma once

#include "tbe_common.h"

namespace tbe {

template <typename A> __device__ __forceinline__ A adagrad_multiplier(A state_new, float lr, float eps);
// lr * (1.0 / (sqrt(s) + eps)) with the reference's types: float sqrt and add,
// double reciprocal and product, rounded to float (tbe.cu:453-454).
template <> __device__ __forceinline__ float adagrad_multiplier<float>(float s, float lr, float eps) {
  return static_cast<float>(static_cast<double>(lr) * (1.0 / static_cast<double>(sqrtf(s) + eps)));
}
template <> __device__ __forceinline__ double adagrad_multiplier<double>(double s, float lr, float eps) {
  return static_cast<double>(lr) * (1.0 / (sqrt(s) + static_cast<double>(eps)));
}

template <typename A> __device__ __forceinline__ A approx_multiplier(A state_new, A psw, bool weighted, float lr, float eps);
// (element_weight *) learning_rate * (1.0 / (sqrt(s) + eps)) with the reference's types: float
// sqrt and sum, double reciprocal and product, rounded to float (tbe.cu:453-454, 515-518).
template <> __device__ __forceinline__ float approx_multiplier<float>(float s, float pw, bool weighted, float lr, float eps) {
  const double inv = 1.0 / static_cast<double>(sqrtf(s) + eps);
  return weighted ? static_cast<float>(static_cast<double>(pw * lr) * inv)
                  : static_cast<float>(static_cast<double>(lr) * inv);
}
template <> __device__ __forceinline__ double approx_multiplier<double>(double s, double pw, bool weighted, float lr, float eps) {
  const double inv = 1.0 / (sqrt(s) + static_cast<double>(eps));
  return weighted ? pw * static_cast<double>(lr) * inv : static_cast<double>(lr) * inv;
}

// v of the lane a data-parallel-primitive pattern selects, 0 where the pattern has no source lane
// or the row mask leaves the lane out.
template <int CTRL, int ROW_MASK> __device__ __forceinline__ float dpp_or_zero(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, ROW_MASK == 0xf));
}
template <int CTRL, int ROW_MASK> __device__ __forceinline__ double dpp_or_zero(double v) {
  const int64_t bits = __double_as_longlong(v);
  const uint32_t lo = static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(bits), CTRL, ROW_MASK, 0xf, ROW_MASK == 0xf));
  const uint32_t hi = static_cast<uint32_t>(
      __builtin_amdgcn_update_dpp(0, static_cast<int>(bits >> 32), CTRL, ROW_MASK, 0xf, ROW_MASK == 0xf));
  return __longlong_as_double(static_cast<int64_t>((static_cast<uint64_t>(hi) << 32) | lo));
}

// Inclusive prefix sum over the 64 lanes without a trip through LDS: shifts inside the rows of 16
// lanes, then the last lane of row 0 / 2 added to row 1 / 3 and the last lane of row 1 to rows 2
// and 3 (row_shr:n = 0x110 + n, row_bcast:15 = 0x142, row_bcast:31 = 0x143).
template <typename A> __device__ __forceinline__ A wave_inclusive_sum(A x) {
  x += dpp_or_zero<0x111, 0xf>(x);
  x += dpp_or_zero<0x112, 0xf>(x);
  x += dpp_or_zero<0x114, 0xf>(x);
  x += dpp_or_zero<0x118, 0xf>(x);
  x += dpp_or_zero<0x142, 0xa>(x);
  x += dpp_or_zero<0x143, 0xc>(x);
  return x;
}

// The value a row vector has after it was stored in the weights' type and read again.
template <typename T, int VEC>
__device__ __forceinline__ void round_trip(RowVec<T, VEC> &w, const StochasticRounding &sr, int64_t element) {
  if constexpr (sizeof(T) == 2) w.unpack(pack_rounded<T, VEC>(w, sr, element));
}

// The approximate update rounds the k-th update of a row within a call with its own random words.
__device__ __forceinline__ StochasticRounding rounding_of_update(const StochasticRounding &sr, int k) {
  StochasticRounding out = sr;
  out.seed ^= static_cast<uint64_t>(k) * 0x9E3779B97F4A7C15ull;
  return out;
}

}  // namespace tbe
