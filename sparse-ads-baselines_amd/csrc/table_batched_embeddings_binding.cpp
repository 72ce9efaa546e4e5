// pybind11 module `table_batched_embeddings_cpp`: the reference's extension module
// (table_batched_embeddings.cpp:6-27, 56-70 -- functions taking at::Tensor, bound by name) written
// over the C ABI of libtbe_hip.so.  It is what a maintainer of the reference would put in place
// of table_batched_embeddings.cpp: same function names, same positional arguments, AT_ASSERT-style
// failures as RuntimeError, kernels launched on the current stream of the weights' device, nothing
// synchronised.  Host code only: the kernels are in the library.
//
// All ten functions of the reference's module are bound (forward, backward_sgd,
// backward_approx_adagrad, backward_exact_adagrad, their three mixed-dimension counterparts,
// construct_offsets, new_managed_tensor, new_host_mapped_tensor); the Python module
// table_batched_embeddings.py binds the same entry points plus the plan-ahead and cache ones.
#include <torch/extension.h>

// (PyTorch on ROCm presents the GPU under the device type "cuda": the guard and the stream are
// the ones registered for that type)
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>

#include <algorithm>
#include <map>
#include <memory>
#include <mutex>
#include <iterator>
#include <utility>
#include <vector>

#include "tbe_hip.h"

namespace {

void check(int rc) {
  TORCH_CHECK(rc == TBE_OK, tbe_last_error());
}

int32_t dtype_code(const at::Tensor &t) {
  switch (t.scalar_type()) {
    case at::kFloat: return TBE_DTYPE_F32;
    case at::kHalf: return TBE_DTYPE_F16;
    case at::kDouble: return TBE_DTYPE_F64;
    default: TORCH_CHECK(false, "weights must be float16, float32 or float64");
  }
  return -1;
}

void *stream_of(const at::Tensor &t) {
  return c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(static_cast<c10::DeviceIndex>(t.get_device())).stream();
}

const void *ptr(const c10::optional<at::Tensor> &t) { return t.has_value() ? t->data_ptr() : nullptr; }

struct Shape {
  int32_t T, B, D;
  int64_t n, rows;
};

// table_batched_embeddings_cuda.cu:262-273 (AT_ASSERT on T, B, D) plus the dtype / device /
// contiguity checks that at::Tensor accessors make there.
Shape check_common(const at::Tensor &weights, const at::Tensor &table_offsets, const at::Tensor &indices,
                   const at::Tensor &offsets) {
  TORCH_CHECK(weights.is_cuda(), "weights must be a GPU tensor");
  TORCH_CHECK(weights.dim() == 2 && weights.is_contiguous(), "weights must be a contiguous [rows, D] tensor");
  for (const at::Tensor *t : {&table_offsets, &indices, &offsets}) {
    TORCH_CHECK(t->scalar_type() == at::kInt && t->is_contiguous() && t->dim() == 1,
                "table_offsets, indices and offsets must be contiguous 1-D int32 tensors");
    TORCH_CHECK(t->device() == weights.device(), "all tensors must live on the weights' device");
  }
  Shape s;
  s.T = static_cast<int32_t>(table_offsets.numel());
  TORCH_CHECK(s.T > 0, "T must be positive");
  TORCH_CHECK((offsets.numel() - 1) % s.T == 0 && offsets.numel() > 1, "offsets must have T * B + 1 entries");
  s.B = static_cast<int32_t>((offsets.numel() - 1) / s.T);
  s.D = static_cast<int32_t>(weights.size(1));
  TORCH_CHECK(s.D > 0 && s.D % 4 == 0, "D must be a positive multiple of 4");
  s.n = indices.numel();
  s.rows = weights.size(0);
  return s;
}

at::Tensor check_grad(const at::Tensor &grad_output, const at::Tensor &weights, const Shape &s) {
  TORCH_CHECK(grad_output.scalar_type() == weights.scalar_type(), "grad_output must have the weights' dtype");
  TORCH_CHECK(grad_output.device() == weights.device(), "grad_output must live on the weights' device");
  TORCH_CHECK(grad_output.dim() == 3 && grad_output.size(0) == s.B && grad_output.size(1) == s.T &&
                  grad_output.size(2) == s.D,
              "grad_output must be [B, T, D]");
  return grad_output.contiguous();
}

void check_weights_of_lookups(const c10::optional<at::Tensor> &indice_weights, const at::Tensor &weights,
                              const at::Tensor &indices) {
  if (!indice_weights.has_value()) return;
  TORCH_CHECK(indice_weights->scalar_type() == weights.scalar_type(), "indice_weights must have the weights' dtype");
  TORCH_CHECK(indice_weights->is_contiguous() && indice_weights->numel() == indices.numel(),
              "indice_weights must be contiguous with one entry per index");
  TORCH_CHECK(indice_weights->device() == weights.device(), "indice_weights must live on the weights' device");
}

void check_state(const at::Tensor &optimizer_state, const at::Tensor &weights) {
  const auto want = weights.scalar_type() == at::kDouble ? at::kDouble : at::kFloat;
  TORCH_CHECK(optimizer_state.scalar_type() == want, "optimizer_state must be float32 (float64 for float64 weights)");
  TORCH_CHECK(optimizer_state.is_contiguous() && optimizer_state.numel() == weights.size(0),
              "optimizer_state must be contiguous with one entry per row");
  TORCH_CHECK(optimizer_state.device() == weights.device(), "optimizer_state must live on the weights' device");
}

// One grow-only scratch tensor per (device, stream), so that calls issued on different streams
// of a device may overlap (the reference allocates its sort buffers per call,
// table_batched_embeddings_cuda.cu:1618-1647).  The kMaxWorkspaces most recently used ones are
// kept.  A call holds its tensor (by value: the memory stays until the launches are enqueued,
// whatever happens to the table meanwhile) and the entry's lock until it returns, so two host
// threads that drive one stream cannot interleave their launch sequences on one buffer.
constexpr size_t kMaxWorkspaces = 8;
struct HeldWorkspace {
  at::Tensor tensor;
  std::shared_ptr<std::mutex> busy = std::make_shared<std::mutex>();
  uint64_t last_use = 0;
};
struct Scratch {
  at::Tensor tensor;
  std::shared_ptr<std::mutex> busy;
  std::unique_lock<std::mutex> lock;
  void *data() const { return tensor.data_ptr(); }
  uint64_t bytes() const { return static_cast<uint64_t>(tensor.numel()); }
};
std::mutex g_workspaces_mutex;
std::map<std::pair<int, void *>, HeldWorkspace> g_workspaces;
uint64_t g_workspace_clock = 0;

Scratch workspace(const at::Tensor &like, uint64_t bytes) {
  const std::pair<int, void *> key{static_cast<int>(like.get_device()), stream_of(like)};
  std::shared_ptr<std::mutex> busy;
  {
    std::lock_guard<std::mutex> lock(g_workspaces_mutex);
    HeldWorkspace &held = g_workspaces[key];
    held.last_use = ++g_workspace_clock;
    busy = held.busy;
    while (g_workspaces.size() > kMaxWorkspaces) {
      auto oldest = g_workspaces.begin();
      for (auto it = g_workspaces.begin(); it != g_workspaces.end(); ++it)
        if (it->second.last_use < oldest->second.last_use) oldest = it;
      g_workspaces.erase(oldest);
    }
  }
  std::unique_lock<std::mutex> in_use(*busy);
  std::lock_guard<std::mutex> lock(g_workspaces_mutex);
  HeldWorkspace &held = g_workspaces[key];  // (back again if the eviction above or a release took it)
  held.busy = busy;
  if (!held.tensor.defined() || static_cast<uint64_t>(held.tensor.numel()) < bytes)
    held.tensor = at::empty({static_cast<int64_t>(bytes + bytes / 4 + 256)}, like.options().dtype(at::kByte));
  return Scratch{held.tensor, busy, std::move(in_use)};
}

// Sizes the current stream's scratch tensor ahead of time (before a graph capture on that stream).
void reserve_workspace(at::Tensor like, int64_t bytes) {
  TORCH_CHECK(like.is_cuda() && bytes >= 0, "reserve_workspace takes a GPU tensor (for its device) and a size");
  c10::DeviceGuard guard(like.device());
  (void)workspace(like, static_cast<uint64_t>(bytes));
}

// Drops every scratch tensor; work already enqueued keeps running on them.
void release_workspaces() {
  std::lock_guard<std::mutex> lock(g_workspaces_mutex);
  g_workspaces.clear();
}

// Small int32 tensors whose values the host needs (table_offsets for the largest table's row
// count, which decides how many key bits the backward sorts; dim_offsets for the vector width of
// fp16 rows) are copied to the host once per tensor and kept while that tensor lives and is not
// written to: an entry holds a weak reference to the tensor, which also keeps its address from
// being handed to another tensor, and the version counter it had.
std::vector<int32_t> host_values(const at::Tensor &t) {
  struct Known {
    c10::weak_intrusive_ptr<c10::TensorImpl> tensor;
    uint32_t version;
    std::vector<int32_t> values;
  };
  static std::mutex mutex;
  static std::map<const void *, Known> known;
  const void *address = t.unsafeGetTensorImpl();
  {
    std::lock_guard<std::mutex> lock(mutex);
    const auto it = known.find(address);
    if (it != known.end()) {
      if (!it->second.tensor.expired() && it->second.version == t._version()) return it->second.values;
      known.erase(it);
    }
  }
  const at::Tensor host = t.cpu().contiguous();
  std::vector<int32_t> values(host.data_ptr<int32_t>(), host.data_ptr<int32_t>() + host.numel());
  std::lock_guard<std::mutex> lock(mutex);
  for (auto it = known.begin(); it != known.end();) it = it->second.tensor.expired() ? known.erase(it) : std::next(it);
  known.emplace(address, Known{c10::weak_intrusive_ptr<c10::TensorImpl>(t.getIntrusivePtr()), t._version(), values});
  return values;
}

// starts: first row of every table; uniform tables have T entries and end at total_rows, the
// mixed-dimension modules pass T + 1 entries (total_rows < 0: the last entry is the end).
int64_t max_table_rows(const at::Tensor &starts_tensor, int64_t total_rows) {
  const std::vector<int32_t> starts = host_values(starts_tensor);
  const int64_t tables = total_rows < 0 ? static_cast<int64_t>(starts.size()) - 1 : static_cast<int64_t>(starts.size());
  int64_t largest = 0;
  for (int64_t t = 0; t < tables; ++t) {
    const int64_t end = t + 1 < static_cast<int64_t>(starts.size()) ? starts[t + 1] : total_rows;
    largest = std::max<int64_t>(largest, end - starts[t]);
  }
  return largest;
}

// fp16 rows move 16 bytes at a time when every table's D allows it, else 8 bytes.
int32_t fp16_vector_width(const at::Tensor &dim_offsets) {
  const std::vector<int32_t> offsets = host_values(dim_offsets);
  int32_t width = 8;
  for (size_t t = 0; t + 1 < offsets.size(); ++t) {
    const int32_t d = offsets[t + 1] - offsets[t];
    TORCH_CHECK(d > 0 && d % 4 == 0, "every D_t must be a positive multiple of 4");
    if (d % 8 != 0) width = 4;
  }
  return width;
}

uint64_t workspace_bytes(const Shape &s, int32_t dtype) {
  tbe_workspace_layout_t layout;
  check(tbe_backward_workspace_layout(s.n, s.D, dtype, s.T, &layout));
  return layout.total_bytes;
}

// batched_embedding_forward_cuda (table_batched_embeddings_cuda.cu:253-316).  L_max, BT_block_size and
// shmem are the reference's launch knobs: accepted, not used.
at::Tensor forward(at::Tensor weights, at::Tensor table_offsets, at::Tensor indices, at::Tensor offsets,
                   c10::optional<at::Tensor> indice_weights, int64_t L_max, int64_t BT_block_size, bool shmem) {
  (void)L_max;
  (void)shmem;
  const Shape s = check_common(weights, table_offsets, indices, offsets);
  TORCH_CHECK(BT_block_size != 0, "BT_block_size must be non-zero");
  check_weights_of_lookups(indice_weights, weights, indices);
  c10::DeviceGuard guard(weights.device());
  at::Tensor output = at::empty({s.B, s.T, s.D}, weights.options());
  check(tbe_forward(weights.data_ptr(), dtype_code(weights), s.D, table_offsets.data_ptr<int32_t>(), s.T,
                    indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B, ptr(indice_weights),
                    output.data_ptr(), stream_of(weights)));
  return output;
}

// batched_embedding_backward_sgd_cuda (table_batched_embeddings_cuda.cu:383-435), exact.
void backward_sgd(at::Tensor grad_output, at::Tensor weights, at::Tensor table_offsets, at::Tensor indices,
                  at::Tensor offsets, double learning_rate, int64_t L_max, int64_t BT_block_size, bool shmem) {
  (void)L_max;
  (void)shmem;
  const Shape s = check_common(weights, table_offsets, indices, offsets);
  TORCH_CHECK(BT_block_size > 0, "BT_block_size must be positive");
  grad_output = check_grad(grad_output, weights, s);
  const int32_t dtype = dtype_code(weights);
  c10::DeviceGuard guard(weights.device());
  Scratch ws = workspace(weights, workspace_bytes(s, dtype));
  check(tbe_backward_sgd(grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows,
                         max_table_rows(table_offsets, s.rows), s.D, table_offsets.data_ptr<int32_t>(), s.T,
                         indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
                         static_cast<float>(learning_rate), ws.data(), ws.bytes(),
                         stream_of(weights)));
}

// The (seed, offset) of this call's random stream: four values of the device's default generator,
// as the reference takes them (table_batched_embeddings_cuda.cu:1683-1690).
std::pair<uint64_t, uint64_t> rounding_stream(const at::Tensor &weights) {
  py::gil_scoped_acquire gil;
  py::object torch_cuda = py::module::import("torch").attr("cuda");
  py::object gen = torch_cuda.attr("default_generators")[py::int_(weights.get_device())];
  const uint64_t seed = gen.attr("initial_seed")().cast<uint64_t>();
  const uint64_t offset = gen.attr("get_offset")().cast<uint64_t>();
  gen.attr("set_offset")(offset + 4);
  return {seed, offset};
}

// batched_embedding_backward_adagrad_exact_cuda (table_batched_embeddings_cuda.cu:1589-1706); the
// weighted case, which the reference asserts out (:1678-1679), is served.
c10::optional<at::Tensor> backward_exact_adagrad(at::Tensor grad_output, at::Tensor weights, at::Tensor table_offsets,
                                                 at::Tensor indices, at::Tensor offsets,
                                                 c10::optional<at::Tensor> indice_weights, at::Tensor optimizer_state,
                                                 double learning_rate, double eps, bool stochastic_rounding,
                                                 int64_t BT_block_size) {
  const Shape s = check_common(weights, table_offsets, indices, offsets);
  TORCH_CHECK(BT_block_size > 0, "BT_block_size must be positive");
  grad_output = check_grad(grad_output, weights, s);
  check_state(optimizer_state, weights);
  check_weights_of_lookups(indice_weights, weights, indices);
  const int32_t dtype = dtype_code(weights);
  c10::DeviceGuard guard(weights.device());
  c10::optional<at::Tensor> grad_indice_weights;
  if (indice_weights.has_value()) grad_indice_weights = at::empty_like(*indice_weights);
  Scratch ws = workspace(weights, workspace_bytes(s, dtype));
  void *grad_psw = grad_indice_weights.has_value() ? grad_indice_weights->data_ptr() : nullptr;
  if (stochastic_rounding && weights.scalar_type() == at::kHalf) {
    const auto stream = rounding_stream(weights);
    check(tbe_backward_exact_adagrad_stochastic(
        grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows, max_table_rows(table_offsets, s.rows), s.D,
        table_offsets.data_ptr<int32_t>(), s.T, indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
        ptr(indice_weights), optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
        grad_psw, stream.first, stream.second, ws.data(), ws.bytes(), stream_of(weights)));
  } else {
    check(tbe_backward_exact_adagrad(
        grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows, max_table_rows(table_offsets, s.rows), s.D,
        table_offsets.data_ptr<int32_t>(), s.T, indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
        ptr(indice_weights), optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
        grad_psw, ws.data(), ws.bytes(), stream_of(weights)));
  }
  return grad_indice_weights;
}

// batched_embedding_backward_adagrad_approx_cuda (table_batched_embeddings_cuda.cu:706-793).
c10::optional<at::Tensor> backward_approx_adagrad(at::Tensor grad_output, at::Tensor weights,
                                                  at::Tensor table_offsets, at::Tensor indices, at::Tensor offsets,
                                                  c10::optional<at::Tensor> indice_weights,
                                                  at::Tensor optimizer_state, double learning_rate, double eps,
                                                  int64_t L_max, bool stochastic_rounding, int64_t BT_block_size) {
  (void)L_max;
  const Shape s = check_common(weights, table_offsets, indices, offsets);
  TORCH_CHECK(BT_block_size > 0, "BT_block_size must be positive");
  grad_output = check_grad(grad_output, weights, s);
  check_state(optimizer_state, weights);
  check_weights_of_lookups(indice_weights, weights, indices);
  const int32_t dtype = dtype_code(weights);
  c10::DeviceGuard guard(weights.device());
  c10::optional<at::Tensor> grad_indice_weights;
  if (indice_weights.has_value()) grad_indice_weights = at::empty_like(*indice_weights);
  Scratch ws = workspace(weights, workspace_bytes(s, dtype));
  const bool rounds = stochastic_rounding && weights.scalar_type() == at::kHalf;
  std::pair<uint64_t, uint64_t> stream{0, 0};
  if (rounds) stream = rounding_stream(weights);
  check(tbe_backward_approx_adagrad(
      grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows, max_table_rows(table_offsets, s.rows), s.D,
      table_offsets.data_ptr<int32_t>(), s.T, indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
      ptr(indice_weights), optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
      grad_indice_weights.has_value() ? grad_indice_weights->data_ptr() : nullptr, rounds ? 1 : 0, stream.first,
      stream.second, ws.data(), ws.bytes(), stream_of(weights)));
  return grad_indice_weights;
}

// construct_offsets (table_batched_embeddings_cuda.cu:1190-1213).
at::Tensor construct_offsets(at::Tensor batch_offsets_per_table, at::Tensor total_indices_per_table) {
  TORCH_CHECK(batch_offsets_per_table.is_cuda() && batch_offsets_per_table.dim() == 2 &&
                  batch_offsets_per_table.scalar_type() == at::kInt && batch_offsets_per_table.is_contiguous(),
              "batch_offsets_per_table must be a contiguous int32 [T, B] GPU tensor");
  const int32_t T = static_cast<int32_t>(batch_offsets_per_table.size(0));
  const int32_t B = static_cast<int32_t>(batch_offsets_per_table.size(1));
  TORCH_CHECK(total_indices_per_table.scalar_type() == at::kInt && total_indices_per_table.is_contiguous() &&
                  total_indices_per_table.numel() == T &&
                  total_indices_per_table.device() == batch_offsets_per_table.device(),
              "total_indices_per_table must be a contiguous int32 [T] tensor on the same device");
  c10::DeviceGuard guard(batch_offsets_per_table.device());
  at::Tensor output = at::empty({1 + static_cast<int64_t>(T) * B}, batch_offsets_per_table.options());
  check(tbe_construct_offsets(batch_offsets_per_table.data_ptr<int32_t>(), total_indices_per_table.data_ptr<int32_t>(),
                              T, B, output.data_ptr<int32_t>(), stream_of(batch_offsets_per_table)));
  return output;
}

struct MixedShape {
  int32_t T, B;
  int64_t n;
};

// table_batched_embeddings_cuda.cu:945-962: weights is the flat 1-D buffer of all tables,
// table_offsets int64 [T+1] element offsets, dim_offsets int32 [T+1] column offsets.
MixedShape check_mixed(const at::Tensor &weights, const at::Tensor &table_offsets, const at::Tensor &dim_offsets,
                       const at::Tensor &indices, const at::Tensor &offsets) {
  TORCH_CHECK(weights.is_cuda(), "weights must be a GPU tensor");
  TORCH_CHECK(weights.dim() == 1 && weights.is_contiguous(), "weights must be a contiguous 1-D tensor");
  TORCH_CHECK(table_offsets.scalar_type() == at::kLong, "table_offsets must be int64");
  for (const at::Tensor *t : {&dim_offsets, &indices, &offsets})
    TORCH_CHECK(t->scalar_type() == at::kInt, "dim_offsets, indices and offsets must be int32");
  for (const at::Tensor *t : {&table_offsets, &dim_offsets, &indices, &offsets}) {
    TORCH_CHECK(t->device() == weights.device(), "all tensors must live on the weights' device");
    TORCH_CHECK(t->dim() == 1 && t->is_contiguous(), "offsets and indices must be contiguous 1-D tensors");
  }
  MixedShape s;
  s.T = static_cast<int32_t>(table_offsets.numel() - 1);
  TORCH_CHECK(s.T > 0, "T must be positive");
  TORCH_CHECK(dim_offsets.numel() == s.T + 1, "dim_offsets must hold T+1 entries");
  s.B = static_cast<int32_t>((offsets.numel() - 1) / s.T);
  TORCH_CHECK(s.B > 0 && offsets.numel() == static_cast<int64_t>(s.T) * s.B + 1, "offsets must hold T*B+1 entries");
  s.n = indices.numel();
  return s;
}

// batched_embedding_forward_mixed_D_cuda (table_batched_embeddings_cuda.cu:945-1004).
at::Tensor forward_mixed_D(at::Tensor weights, at::Tensor table_offsets, at::Tensor dim_offsets, int64_t total_D,
                           at::Tensor indices, at::Tensor offsets, c10::optional<at::Tensor> indice_weights,
                           int64_t L_max, int64_t BT_block_size, bool shmem) {
  (void)L_max;
  (void)shmem;
  const MixedShape s = check_mixed(weights, table_offsets, dim_offsets, indices, offsets);
  TORCH_CHECK(BT_block_size != 0, "BT_block_size must be non-zero");
  check_weights_of_lookups(indice_weights, weights, indices);
  c10::DeviceGuard guard(weights.device());
  at::Tensor output = at::empty({s.B, total_D}, weights.options());
  check(tbe_forward_mixed(weights.data_ptr(), dtype_code(weights), fp16_vector_width(dim_offsets),
                          table_offsets.data_ptr<int64_t>(), dim_offsets.data_ptr<int32_t>(),
                          static_cast<int32_t>(total_D), s.T, indices.data_ptr<int32_t>(), s.n,
                          offsets.data_ptr<int32_t>(), s.B, ptr(indice_weights), output.data_ptr(),
                          stream_of(weights)));
  return output;
}

c10::optional<at::Tensor> backward_mixed(int32_t optimizer, at::Tensor grad_output, const at::Tensor &weights,
                                         const at::Tensor &table_offsets, const at::Tensor &table_dim_offsets,
                                         const at::Tensor &dim_offsets, int64_t total_D, const at::Tensor &indices,
                                         const at::Tensor &offsets, const c10::optional<at::Tensor> &indice_weights,
                                         const at::Tensor &optimizer_state, double learning_rate, double eps,
                                         bool stochastic_rounding, int64_t BT_block_size) {
  const MixedShape s = check_mixed(weights, table_offsets, dim_offsets, indices, offsets);
  TORCH_CHECK(BT_block_size > 0, "BT_block_size must be positive");
  TORCH_CHECK(table_dim_offsets.scalar_type() == at::kInt && table_dim_offsets.numel() == s.T + 1 &&
                  table_dim_offsets.is_contiguous() && table_dim_offsets.device() == weights.device(),
              "table_dim_offsets must be a contiguous int32 tensor with T+1 entries on the weights' device");
  TORCH_CHECK(grad_output.scalar_type() == weights.scalar_type() && grad_output.dim() == 2 &&
                  grad_output.size(0) == s.B && grad_output.size(1) == total_D &&
                  grad_output.device() == weights.device(),
              "grad_output must be [B, total_D] of the weights' dtype");
  grad_output = grad_output.contiguous();
  const auto want = weights.scalar_type() == at::kDouble ? at::kDouble : at::kFloat;
  TORCH_CHECK(optimizer_state.scalar_type() == want && optimizer_state.is_contiguous() &&
                  optimizer_state.device() == weights.device(),
              "optimizer_state must be contiguous float32 (float64 for float64 weights)");
  check_weights_of_lookups(indice_weights, weights, indices);
  const int32_t dtype = dtype_code(weights);
  c10::DeviceGuard guard(weights.device());
  c10::optional<at::Tensor> grad_indice_weights;
  if (indice_weights.has_value()) grad_indice_weights = at::empty_like(*indice_weights);
  tbe_workspace_layout_t layout;
  check(tbe_backward_mixed_workspace_layout(s.n, dtype, s.T, &layout));
  Scratch ws = workspace(weights, layout.total_bytes);
  const bool rounds = stochastic_rounding && weights.scalar_type() == at::kHalf;
  std::pair<uint64_t, uint64_t> stream{0, 0};
  if (rounds) stream = rounding_stream(weights);
  check(tbe_backward_mixed(optimizer, grad_output.data_ptr(), weights.data_ptr(), dtype, fp16_vector_width(dim_offsets),
                           optimizer_state.numel(), max_table_rows(table_dim_offsets, -1),
                           table_offsets.data_ptr<int64_t>(), table_dim_offsets.data_ptr<int32_t>(),
                           dim_offsets.data_ptr<int32_t>(), static_cast<int32_t>(total_D), s.T,
                           indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B, ptr(indice_weights),
                           optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
                           grad_indice_weights.has_value() ? grad_indice_weights->data_ptr() : nullptr, rounds ? 1 : 0,
                           stream.first, stream.second, ws.data(), ws.bytes(),
                           stream_of(weights)));
  return grad_indice_weights;
}

// batched_embedding_backward_adagrad_exact_mixed_D_cuda (table_batched_embeddings_cuda.cu:1350-1469).
c10::optional<at::Tensor> backward_exact_adagrad_mixed_D(at::Tensor grad_output, at::Tensor weights,
                                                         at::Tensor table_offsets, at::Tensor table_dim_offsets,
                                                         at::Tensor dim_offsets, int64_t total_D, at::Tensor indices,
                                                         at::Tensor offsets, c10::optional<at::Tensor> indice_weights,
                                                         at::Tensor optimizer_state, double learning_rate, double eps,
                                                         bool stochastic_rounding, int64_t BT_block_size) {
  return backward_mixed(TBE_OPT_ROWWISE_ADAGRAD, grad_output, weights, table_offsets, table_dim_offsets, dim_offsets,
                        total_D, indices, offsets, indice_weights, optimizer_state, learning_rate, eps,
                        stochastic_rounding, BT_block_size);
}

// batched_embedding_backward_adagrad_approx_mixed_D_cuda (table_batched_embeddings_cuda.cu:1076-1163).
c10::optional<at::Tensor> backward_approx_adagrad_mixed_D(at::Tensor grad_output, at::Tensor weights,
                                                          at::Tensor table_offsets, at::Tensor table_dim_offsets,
                                                          at::Tensor dim_offsets, int64_t total_D, at::Tensor indices,
                                                          at::Tensor offsets, c10::optional<at::Tensor> indice_weights,
                                                          at::Tensor optimizer_state, double learning_rate, double eps,
                                                          int64_t L_max, bool stochastic_rounding,
                                                          int64_t BT_block_size) {
  (void)L_max;
  return backward_mixed(TBE_OPT_APPROX_ROWWISE_ADAGRAD, grad_output, weights, table_offsets, table_dim_offsets,
                        dim_offsets, total_D, indices, offsets, indice_weights, optimizer_state, learning_rate, eps,
                        stochastic_rounding, BT_block_size);
}

int64_t bytes_of(const at::Tensor &self, const std::vector<int64_t> &sizes) {
  TORCH_CHECK(self.is_cuda() && self.is_floating_point(), "the prototype must be a floating GPU tensor");
  int64_t bytes = static_cast<int64_t>(self.element_size());
  for (const int64_t size : sizes) {
    TORCH_CHECK(size >= 0, "sizes must not be negative");
    bytes *= size;
  }
  return bytes;
}

// new_managed_tensor (table_batched_embeddings_cuda.cu:864-871): managed memory preferring the
// host, tagged with the prototype's device and dtype; released with the tensor's storage, as by
// the reference's CUDAManagedDeleter (:795-812).
at::Tensor new_managed_tensor(at::Tensor self, std::vector<int64_t> sizes) {
  const int64_t bytes = bytes_of(self, sizes);
  c10::DeviceGuard guard(self.device());
  void *memory = nullptr;
  check(tbe_managed_alloc(static_cast<uint64_t>(std::max<int64_t>(bytes, 1)), self.get_device(), &memory));
  return at::from_blob(memory, sizes, [](void *p) { tbe_managed_free(p); }, self.options(), self.device());
}

// new_host_mapped_tensor (table_batched_embeddings_cuda.cu:873-880): pinned host memory mapped
// into the device's address space; released with the tensor's storage (CUDAHostMappedDeleter, :820-835).
at::Tensor new_host_mapped_tensor(at::Tensor self, std::vector<int64_t> sizes) {
  const int64_t bytes = bytes_of(self, sizes);
  c10::DeviceGuard guard(self.device());
  void *host = nullptr, *device = nullptr;
  check(tbe_host_mapped_alloc(static_cast<uint64_t>(std::max<int64_t>(bytes, 1)), &host, &device));
  return at::from_blob(device, sizes, [host](void *) { tbe_host_mapped_free(host); }, self.options(), self.device());
}

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("forward", &forward, "forward");
  m.def("backward_sgd", &backward_sgd, "backward_sgd");
  m.def("backward_exact_adagrad", &backward_exact_adagrad, "backward_exact_adagrad");
  m.def("backward_approx_adagrad", &backward_approx_adagrad, "backward_approx_adagrad");
  m.def("construct_offsets", &construct_offsets, "construct_offsets");
  m.def("forward_mixed_D", &forward_mixed_D, "forward_mixed_D");
  m.def("backward_exact_adagrad_mixed_D", &backward_exact_adagrad_mixed_D, "backward_exact_adagrad_mixed_D");
  m.def("backward_approx_adagrad_mixed_D", &backward_approx_adagrad_mixed_D, "backward_approx_adagrad_mixed_D");
  m.def("new_managed_tensor", &new_managed_tensor, "new_managed_tensor");
  m.def("new_host_mapped_tensor", &new_host_mapped_tensor, "new_host_mapped_tensor");
  m.def("abi_version", []() { return tbe_abi_version(); }, "version of the C ABI the library exports");
  m.def("reserve_workspace", &reserve_workspace, "sizes the current stream's scratch tensor ahead of time");
  m.def("release_workspaces", &release_workspaces, "drops the scratch tensors the module holds");
}
