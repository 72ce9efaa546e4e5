// pybind11 module `table_batched_embeddings_cpp`: the reference's extension module
// (table_batched_embeddings.cpp:6-27, 56-70 -- functions taking at::Tensor, bound by name) written
// over the C ABI of libtbe_hip.so.  It is what a maintainer of the reference would put in place
// of table_batched_embeddings.cpp: same function names, same positional arguments, AT_ASSERT-style
// failures as RuntimeError, kernels launched on the current stream of the weights' device, nothing
// synchronised.  Host code only: the kernels are in the library.
//
// The uniform-table functions of the hot path are bound here (forward, backward_sgd,
// backward_exact_adagrad, backward_approx_adagrad, construct_offsets); the Python module
// table_batched_embeddings.py binds the same entry points plus the mixed-dimension, host-memory and
// plan-ahead ones.
#include <torch/extension.h>

// (PyTorch on ROCm presents the GPU under the device type "cuda": the guard and the stream are
// the ones registered for that type)
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>

#include <algorithm>
#include <map>
#include <mutex>
#include <iterator>

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

// One grow-only scratch tensor per device (the reference allocates its sort buffers per call,
// table_batched_embeddings_cuda.cu:1618-1647).
at::Tensor &workspace(const at::Tensor &like, uint64_t bytes) {
  static std::mutex mutex;
  static std::map<int, at::Tensor> held;
  std::lock_guard<std::mutex> lock(mutex);
  at::Tensor &ws = held[like.get_device()];
  if (!ws.defined() || static_cast<uint64_t>(ws.numel()) < bytes)
    ws = at::empty({static_cast<int64_t>(bytes + bytes / 4 + 256)}, like.options().dtype(at::kByte));
  return ws;
}

// The largest table's row count decides how many key bits the backward sorts.  It is derived
// from table_offsets once per tensor (one device-to-host copy) and kept while that tensor lives
// and is not written to: an entry holds a weak reference to the tensor, which also keeps its
// address from being handed to another tensor, and the version counter it had.
int64_t max_table_rows(const at::Tensor &table_offsets, int64_t total_rows) {
  struct Known {
    c10::weak_intrusive_ptr<c10::TensorImpl> tensor;
    uint32_t version;
    int64_t total_rows;
    int64_t largest;
  };
  static std::mutex mutex;
  static std::map<const void *, Known> known;
  const void *address = table_offsets.unsafeGetTensorImpl();
  {
    std::lock_guard<std::mutex> lock(mutex);
    const auto it = known.find(address);
    if (it != known.end()) {
      if (!it->second.tensor.expired() && it->second.version == table_offsets._version() &&
          it->second.total_rows == total_rows)
        return it->second.largest;
      known.erase(it);
    }
  }
  const at::Tensor host = table_offsets.cpu();
  const int32_t *starts = host.data_ptr<int32_t>();
  int64_t largest = 0;
  for (int64_t t = 0; t < host.numel(); ++t) {
    const int64_t end = t + 1 < host.numel() ? starts[t + 1] : total_rows;
    largest = std::max<int64_t>(largest, end - starts[t]);
  }
  std::lock_guard<std::mutex> lock(mutex);
  for (auto it = known.begin(); it != known.end();) it = it->second.tensor.expired() ? known.erase(it) : std::next(it);
  known.emplace(address, Known{c10::weak_intrusive_ptr<c10::TensorImpl>(table_offsets.getIntrusivePtr()),
                               table_offsets._version(), total_rows, largest});
  return largest;
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
  at::Tensor &ws = workspace(weights, workspace_bytes(s, dtype));
  check(tbe_backward_sgd(grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows,
                         max_table_rows(table_offsets, s.rows), s.D, table_offsets.data_ptr<int32_t>(), s.T,
                         indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
                         static_cast<float>(learning_rate), ws.data_ptr(), static_cast<uint64_t>(ws.numel()),
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
  at::Tensor &ws = workspace(weights, workspace_bytes(s, dtype));
  void *grad_psw = grad_indice_weights.has_value() ? grad_indice_weights->data_ptr() : nullptr;
  if (stochastic_rounding && weights.scalar_type() == at::kHalf) {
    const auto stream = rounding_stream(weights);
    check(tbe_backward_exact_adagrad_stochastic(
        grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows, max_table_rows(table_offsets, s.rows), s.D,
        table_offsets.data_ptr<int32_t>(), s.T, indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
        ptr(indice_weights), optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
        grad_psw, stream.first, stream.second, ws.data_ptr(), static_cast<uint64_t>(ws.numel()), stream_of(weights)));
  } else {
    check(tbe_backward_exact_adagrad(
        grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows, max_table_rows(table_offsets, s.rows), s.D,
        table_offsets.data_ptr<int32_t>(), s.T, indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
        ptr(indice_weights), optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
        grad_psw, ws.data_ptr(), static_cast<uint64_t>(ws.numel()), stream_of(weights)));
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
  at::Tensor &ws = workspace(weights, workspace_bytes(s, dtype));
  const bool rounds = stochastic_rounding && weights.scalar_type() == at::kHalf;
  std::pair<uint64_t, uint64_t> stream{0, 0};
  if (rounds) stream = rounding_stream(weights);
  check(tbe_backward_approx_adagrad(
      grad_output.data_ptr(), weights.data_ptr(), dtype, s.rows, max_table_rows(table_offsets, s.rows), s.D,
      table_offsets.data_ptr<int32_t>(), s.T, indices.data_ptr<int32_t>(), s.n, offsets.data_ptr<int32_t>(), s.B,
      ptr(indice_weights), optimizer_state.data_ptr(), static_cast<float>(learning_rate), static_cast<float>(eps),
      grad_indice_weights.has_value() ? grad_indice_weights->data_ptr() : nullptr, rounds ? 1 : 0, stream.first,
      stream.second, ws.data_ptr(), static_cast<uint64_t>(ws.numel()), stream_of(weights)));
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

}  // namespace

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("forward", &forward, "forward");
  m.def("backward_sgd", &backward_sgd, "backward_sgd");
  m.def("backward_exact_adagrad", &backward_exact_adagrad, "backward_exact_adagrad");
  m.def("backward_approx_adagrad", &backward_approx_adagrad, "backward_approx_adagrad");
  m.def("construct_offsets", &construct_offsets, "construct_offsets");
  m.def("abi_version", []() { return tbe_abi_version(); }, "version of the C ABI the library exports");
}
