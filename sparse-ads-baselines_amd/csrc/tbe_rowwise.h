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
