// Error plumbing, small utility kernels and host-memory allocators of the C ABI.

#include <stdarg.h>
#include <stdio.h>

#include <algorithm>
#include <mutex>
#include <vector>

#include "tbe_common.h"

namespace tbe {

namespace {
thread_local char g_last_error[512] = "";
}

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_last_error, sizeof(g_last_error), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char *what) {
  const hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return TBE_OK;
}

// ------------------------------------------------------------ launch profiling
namespace {
struct TimedLaunch {
  const char *name;
  hipEvent_t start, stop;
  float ms;
};
std::mutex g_profile_mutex;
std::vector<TimedLaunch> g_profile;      // launches recorded since tbe_profile_begin
std::vector<hipEvent_t> g_event_pool;    // events kept for reuse
bool g_profiling = false;

hipEvent_t take_event() {
  if (!g_event_pool.empty()) {
    hipEvent_t e = g_event_pool.back();
    g_event_pool.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  if (hipEventCreate(&e) != hipSuccess) return nullptr;
  return e;
}
}  // namespace

LaunchTimer::LaunchTimer(const char *name, hipStream_t s) : slot(-1), stream(s) {
  if (!g_profiling) return;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  TimedLaunch t{name, take_event(), take_event(), 0.0f};
  if (!t.start || !t.stop) return;
  (void)hipEventRecord(t.start, stream);
  slot = static_cast<int>(g_profile.size());
  g_profile.push_back(t);
}

LaunchTimer::~LaunchTimer() {
  if (slot < 0) return;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  (void)hipEventRecord(g_profile[slot].stop, stream);
}

namespace {

// One thread per bag; same arithmetic as construct_offsets_kernel
// (table_batched_embeddings_cuda.cu:1165-1188).
__global__ __launch_bounds__(kBlockThreads) void construct_offsets_kernel(
    const int32_t *__restrict__ batch_offsets_per_table,
    const int32_t *__restrict__ total_indices_per_table, int T, int B,
    int32_t *__restrict__ output) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i == 0) output[0] = 0;
  if (i >= static_cast<int64_t>(T) * B) return;
  const int t = static_cast<int>(i / B);
  const int b = static_cast<int>(i - static_cast<int64_t>(t) * B);
  const int32_t lower = batch_offsets_per_table[i];
  const int32_t upper = (b != B - 1) ? batch_offsets_per_table[i + 1] : total_indices_per_table[t];
  output[1 + i] = upper - lower;
}

}  // namespace
}  // namespace tbe

extern "C" const char *tbe_last_error(void) { return tbe::g_last_error; }

extern "C" int32_t tbe_abi_version(void) { return 22; }

extern "C" int tbe_profile_begin(void) {
  using namespace tbe;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  for (TimedLaunch &t : g_profile) {
    g_event_pool.push_back(t.start);
    g_event_pool.push_back(t.stop);
  }
  g_profile.clear();
  g_profiling = true;
  return TBE_OK;
}

extern "C" int tbe_profile_end(void) {
  using namespace tbe;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  g_profiling = false;
  for (TimedLaunch &t : g_profile) {
    hipError_t e = hipEventSynchronize(t.stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&t.ms, t.start, t.stop);
    if (e != hipSuccess) return fail(TBE_ERR_HIP, "tbe_profile_end: %s", hipGetErrorString(e));
  }
  return TBE_OK;
}

extern "C" int32_t tbe_profile_count(void) {
  std::lock_guard<std::mutex> lock(tbe::g_profile_mutex);
  return static_cast<int32_t>(tbe::g_profile.size());
}

extern "C" int tbe_profile_get(int32_t i, const char **name, float *milliseconds) {
  using namespace tbe;
  std::lock_guard<std::mutex> lock(g_profile_mutex);
  TBE_REQUIRE(name && milliseconds, "tbe_profile_get: null output pointer");
  TBE_REQUIRE(i >= 0 && i < static_cast<int32_t>(g_profile.size()), "tbe_profile_get: index %d out of range", i);
  *name = g_profile[i].name;
  *milliseconds = g_profile[i].ms;
  return TBE_OK;
}

namespace tbe {
namespace {
__global__ __launch_bounds__(kBlockThreads) void stochastic_round_kernel(const float *__restrict__ values,
                                                                        const uint32_t *__restrict__ words,
                                                                        uint16_t *__restrict__ out, int64_t n) {
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kBlockThreads;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * kBlockThreads + threadIdx.x; i < n; i += stride)
    out[i] = static_cast<uint16_t>(floats_to_half2_stochastic(values[i], 0.0f, words[i], 0u) & 0xffffu);
}
}  // namespace
}  // namespace tbe

extern "C" int tbe_stochastic_round(const float *values, const uint32_t *random_words, uint16_t *out,
                                    int64_t n, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(n >= 0, "tbe_stochastic_round: n must not be negative");
  if (n == 0) return TBE_OK;
  TBE_REQUIRE(values && random_words && out, "tbe_stochastic_round: null pointer argument");
  const dim3 grid(static_cast<unsigned>(std::min<int64_t>(ceil_div(n, kBlockThreads), 256 * 16)));
  hipStream_t s = static_cast<hipStream_t>(stream);
  TBE_LAUNCH("stochastic_round", s, stochastic_round_kernel, grid, dim3(kBlockThreads), values, random_words, out, n);
  return check_launch("tbe_stochastic_round");
}

namespace tbe {
namespace {
// Row-access probe: LANES lanes (16 bytes each) own one row at a time, as in the forward and
// update kernels, and keep kProbeRows independent rows in flight; nothing else happens, so the
// duration is what the memory system takes for the access pattern alone.
constexpr int kProbeRows = 8;
template <int LANES>
__global__ __launch_bounds__(kBlockThreads) void probe_rows_kernel(uint4 *__restrict__ rows,
                                                                  const int32_t *__restrict__ row_ids, int64_t n,
                                                                  float *__restrict__ state, int modify,
                                                                  uint4 *__restrict__ sink) {
  constexpr int kGroups = kBlockThreads / LANES;
  const int sub = threadIdx.x % LANES;
  const int64_t group = static_cast<int64_t>(blockIdx.x) * kGroups + threadIdx.x / LANES;
  const int64_t stride = static_cast<int64_t>(gridDim.x) * kGroups;
  uint4 acc = make_uint4(0, 0, 0, 0);
  for (int64_t i0 = group * kProbeRows; i0 < n; i0 += stride * kProbeRows) {
    int64_t row[kProbeRows];
#pragma unroll
    for (int k = 0; k < kProbeRows; ++k) row[k] = row_ids[min(i0 + k, n - 1)];
    uint4 v[kProbeRows];
    float s[kProbeRows];
#pragma unroll
    for (int k = 0; k < kProbeRows; ++k) {
      v[k] = rows[row[k] * LANES + sub];
      if (state && sub == 0) s[k] = state[row[k]];
    }
#pragma unroll
    for (int k = 0; k < kProbeRows; ++k) {
      if (modify) {
        if (i0 + k < n) {
          v[k].x += 1u;
          rows[row[k] * LANES + sub] = v[k];
          if (state && sub == 0) state[row[k]] = s[k] + 1.0f;
        }
      } else {
        acc.x ^= v[k].x; acc.y ^= v[k].y; acc.z ^= v[k].z; acc.w ^= v[k].w;
        if (state && sub == 0) acc.x ^= __float_as_uint(s[k]);
      }
    }
  }
  // keeps the loads alive; the condition does not hold for the probe's data
  if (!modify && acc.x == 0x9e3779b9u && acc.y == 0x7f4a7c15u) sink[0] = acc;
}
}  // namespace
}  // namespace tbe

extern "C" int tbe_probe_row_access(void *rows, int32_t row_bytes, const int32_t *row_ids, int64_t num_ids,
                                    float *state, int32_t modify, void *sink, void *stream) {
  using namespace tbe;
  const char *name = "tbe_probe_row_access";
  TBE_REQUIRE(rows && row_ids && sink, "%s: null pointer argument", name);
  TBE_REQUIRE(num_ids > 0 && num_ids < INT32_MAX, "%s: num_ids out of range", name);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int lanes = row_bytes / 16;
  const int64_t groups = ceil_div(num_ids, kProbeRows);
  const dim3 grid(static_cast<unsigned>(std::min<int64_t>(ceil_div(groups * lanes, kBlockThreads), 256 * 64)));
#define TBE_PROBE(L)                                                                                          \
  case L:                                                                                                     \
    TBE_LAUNCH("probe_rows", s, probe_rows_kernel<L>, grid, dim3(kBlockThreads), static_cast<uint4 *>(rows), \
               row_ids, num_ids, state, modify, static_cast<uint4 *>(sink));                                  \
    break;
  switch (lanes * (row_bytes % 16 == 0 ? 1 : 0)) {
    TBE_PROBE(4) TBE_PROBE(8) TBE_PROBE(16) TBE_PROBE(32)
    default:
      return fail(TBE_ERR_UNSUPPORTED, "%s: rows of 64, 128, 256 or 512 bytes (got %d)", name, row_bytes);
  }
#undef TBE_PROBE
  return check_launch(name);
}

extern "C" int tbe_construct_offsets(const int32_t *batch_offsets_per_table,
                                     const int32_t *total_indices_per_table, int32_t T,
                                     int32_t B, int32_t *output, void *stream) {
  using namespace tbe;
  TBE_REQUIRE(T > 0 && B > 0, "tbe_construct_offsets: T and B must be positive (got %d, %d)", T, B);
  TBE_REQUIRE(static_cast<int64_t>(T) * B < INT32_MAX, "tbe_construct_offsets: T*B out of range");
  TBE_REQUIRE(batch_offsets_per_table && total_indices_per_table && output,
              "tbe_construct_offsets: null pointer argument");
  const int64_t n = static_cast<int64_t>(T) * B;
  const dim3 grid(static_cast<unsigned>(ceil_div(n, kBlockThreads)));
  hipStream_t s = static_cast<hipStream_t>(stream);
  TBE_LAUNCH("construct_offsets", s, construct_offsets_kernel, grid, dim3(kBlockThreads),
             batch_offsets_per_table, total_indices_per_table, T, B, output);
  return check_launch("tbe_construct_offsets");
}

extern "C" int tbe_host_mapped_alloc(uint64_t bytes, void **host_ptr, void **device_ptr) {
  using namespace tbe;
  TBE_REQUIRE(host_ptr && device_ptr, "tbe_host_mapped_alloc: null output pointer");
  *host_ptr = nullptr;
  *device_ptr = nullptr;
  if (bytes == 0) return TBE_OK;
  void *h = nullptr;
  hipError_t e = hipHostMalloc(&h, bytes, hipHostMallocMapped | hipHostMallocPortable);
  if (e != hipSuccess)
    return fail(TBE_ERR_HIP, "tbe_host_mapped_alloc(%llu): %s", (unsigned long long)bytes,
                hipGetErrorString(e));
  void *d = nullptr;
  e = hipHostGetDevicePointer(&d, h, 0);
  if (e != hipSuccess) {
    (void)hipHostFree(h);
    return fail(TBE_ERR_HIP, "tbe_host_mapped_alloc: hipHostGetDevicePointer: %s",
                hipGetErrorString(e));
  }
  *host_ptr = h;
  *device_ptr = d;
  return TBE_OK;
}

extern "C" int tbe_host_mapped_free(void *host_ptr) {
  using namespace tbe;
  if (!host_ptr) return TBE_OK;
  const hipError_t e = hipHostFree(host_ptr);
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "tbe_host_mapped_free: %s", hipGetErrorString(e));
  return TBE_OK;
}

extern "C" int tbe_managed_alloc(uint64_t bytes, int32_t device, void **ptr) {
  using namespace tbe;
  TBE_REQUIRE(ptr, "tbe_managed_alloc: null output pointer");
  *ptr = nullptr;
  if (bytes == 0) return TBE_OK;
  void *p = nullptr;
  hipError_t e = hipMallocManaged(&p, bytes, hipMemAttachGlobal);
  if (e != hipSuccess)
    return fail(TBE_ERR_HIP, "tbe_managed_alloc(%llu): %s", (unsigned long long)bytes,
                hipGetErrorString(e));
  // Same placement advice as the reference's managed allocator
  // (table_batched_embeddings_cuda.cu:801-804): pages live on the host, the GPU maps them.
  // Advice is best effort: a platform that rejects it still has a valid allocation.
  (void)hipMemAdvise(p, bytes, hipMemAdviseSetPreferredLocation, hipCpuDeviceId);
  (void)hipMemAdvise(p, bytes, hipMemAdviseSetAccessedBy, device);
  (void)hipGetLastError();
  *ptr = p;
  return TBE_OK;
}

extern "C" int tbe_managed_free(void *ptr) {
  using namespace tbe;
  if (!ptr) return TBE_OK;
  const hipError_t e = hipFree(ptr);
  if (e != hipSuccess) return fail(TBE_ERR_HIP, "tbe_managed_free: %s", hipGetErrorString(e));
  return TBE_OK;
}
