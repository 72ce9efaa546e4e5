"""Drop-in for the single-GPU functions of the reference's older `sparse_embedding_cuda`
extension (sparse_embedding_cuda.cpp:568-601): tables interleaved in one [E][T][D] array, bags
numbered bag-major, dense [B][T][L] indices or flat indices with [B][T+1] offsets.  The calls go
to tbe_forward_interleaved / tbe_backward_sgd_interleaved, which read that layout in place (row
idx*T + t of the [E*T][D] view): no index array is rewritten, and apart from the output nothing
is allocated per call.  The multi-GPU collectives of that module are not served."""
import ctypes

import torch

import table_batched_embeddings as _tbe
import tbe_native as _native

_require = _tbe._require
_ptr = _tbe._ptr

_dense_offsets_cache = {}  # (B*T, L, device) -> int32 [B*T+1] = arange * L


def _check(weights, indices):
    _require(weights.is_cuda and weights.dim() == 3 and weights.is_contiguous(),
             "weights must be a contiguous [E, T, D] GPU tensor")
    _require(weights.dtype in _tbe._DTYPE_CODES, "weights must be float16, float32 or float64")
    _require(indices.dtype == torch.int32 and indices.is_cuda and indices.device == weights.device,
             "indices must be an int32 tensor on the weights' device")
    E, T, D = weights.shape
    _require(E * T < 2 ** 31, "E * T must fit a 32-bit row number")
    _require(D % 4 == 0, "D must be a multiple of 4")
    return E, T, D


def _dense_offsets(B, T, L, device):
    """Bag bounds of dense [B][T][L] indices, offsets[i] = i*L; kept per shape (a tensor the kernels
    only read), so that a call allocates nothing for it."""
    key = (B * T, L, device)
    hit = _dense_offsets_cache.get(key)
    if hit is None:
        if len(_dense_offsets_cache) >= 16:
            _dense_offsets_cache.clear()
        hit = _dense_offsets_cache[key] = torch.arange(0, B * T * L + 1, L, dtype=torch.int32, device=device)
    return hit


def _check_offsets(offsets, weights, T):
    _require(offsets.dtype == torch.int32 and offsets.dim() == 2 and offsets.size(1) == T + 1,
             "offsets must be an int32 [B, T+1] tensor")
    _require(offsets.is_cuda and offsets.device == weights.device and offsets.is_contiguous(),
             "offsets must be contiguous on the weights' device")
    return offsets.size(0)


def _forward(weights, indices, offsets, stride, E, T, D, B):
    indices = indices.contiguous()
    out = torch.empty((B, T, D), dtype=weights.dtype, device=weights.device)
    with torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_forward_interleaved(
            _ptr(weights), _tbe._DTYPE_CODES[weights.dtype], E, T, D, _ptr(indices), indices.numel(), _ptr(offsets),
            stride, B, _ptr(out), _tbe._stream(weights.device)))
    return out


def _backward(grad_output, weights, indices, offsets, stride, E, T, D, B, lr):
    _require(grad_output.dtype == weights.dtype and grad_output.device == weights.device and
             tuple(grad_output.shape) == (B, T, D), "grad_output must be [B, T, D] of the weights' dtype")
    grad_output = grad_output.contiguous()
    indices = indices.contiguous()
    code = _tbe._DTYPE_CODES[weights.dtype]
    layout = _native.backward_interleaved_workspace_layout(indices.numel(), D, code, T, B)
    with _tbe._workspace(weights.device, layout.total_bytes) as (ws, stream), torch.cuda.device(weights.device):
        _native.check(_native.load().tbe_backward_sgd_interleaved(
            _ptr(grad_output), _ptr(weights), code, E, T, D, _ptr(indices), indices.numel(), _ptr(offsets), stride, B,
            float(lr), _ptr(ws), ws.numel(), stream))


def forward_fast_single(weights, indices):
    """sparse_embedding_cuda_forward_fast_single (sparse_embedding_cuda.cpp:265-274):
    weights [E][T][D], indices int32 [B][T][L] -> [B][T][D]."""
    E, T, D = _check(weights, indices)
    _require(indices.dim() == 3 and indices.size(1) == T, "indices must be [B, T, L]")
    B, _, L = indices.shape
    return _forward(weights, indices, _dense_offsets(B, T, L, weights.device), T, E, T, D, B)


forward_single = forward_fast_single  # same contract, different launch geometry in the reference (:255-263)


def forward_offsets(weights, indices, offsets):
    """sparse_embedding_cuda_forward_offsets (sparse_embedding_cuda.cpp:276-288): flat indices,
    offsets int32 [B][T+1] -> [B][T][D]."""
    E, T, D = _check(weights, indices)
    B = _check_offsets(offsets, weights, T)
    return _forward(weights, indices, offsets, T + 1, E, T, D, B)


def backward_update_fast_single(grad_output, weights, indices, lr):
    """sparse_embedding_cuda_backward_update_fast_single (sparse_embedding_cuda.cpp:306-314), made
    exact: every distinct row receives -lr * (sum of its gradients) once (the reference's
    `weights[ind][t][d] -= lr * g` races on repeats, sparse_embedding_cuda_kernel.cu:493-497)."""
    E, T, D = _check(weights, indices)
    _require(indices.dim() == 3 and indices.size(1) == T, "indices must be [B, T, L]")
    B, _, L = indices.shape
    _backward(grad_output, weights, indices, _dense_offsets(B, T, L, weights.device), T, E, T, D, B, lr)


backward_update_single = backward_update_fast_single


def backward_update_offsets(grad_output, weights, indices, offsets, lr):
    """sparse_embedding_cuda_backward_update_offsets (sparse_embedding_cuda.cpp:316-322), exact."""
    E, T, D = _check(weights, indices)
    B = _check_offsets(offsets, weights, T)
    _backward(grad_output, weights, indices, offsets, T + 1, E, T, D, B, lr)


def _needs_more_gpus(*args, **kwargs):
    raise NotImplementedError("the collective entry points need more than one GPU and are not served")


forward = forward_all2all = forward_all2all_nccl = forward_reducescatter = forward_allgather = _needs_more_gpus
