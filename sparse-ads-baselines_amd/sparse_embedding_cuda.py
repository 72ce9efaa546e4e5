"""Drop-in for the single-GPU functions of the reference's older `sparse_embedding_cuda`
extension (sparse_embedding_cuda.cpp:568-601): tables interleaved in one [E][T][D] array, bags
numbered bag-major.  Each call rewrites the indices into row numbers of the [E*T][D] view
(tbe_interleaved_rows) and runs the table-batched kernels on that single virtual table.
The multi-GPU collectives of that module are not served."""
import ctypes

import torch

import table_batched_embeddings as _tbe
import tbe_native as _native

_require = _tbe._require
_ptr = _tbe._ptr


def _check(weights, indices):
    _require(weights.is_cuda and weights.dim() == 3 and weights.is_contiguous(),
             "weights must be a contiguous [E, T, D] GPU tensor")
    _require(indices.dtype == torch.int32 and indices.is_cuda and indices.device == weights.device,
             "indices must be an int32 tensor on the weights' device")
    E, T, D = weights.shape
    _require(E * T < 2 ** 31, "E * T must fit a 32-bit row number")
    return E, T, D


def _rows(indices, flat_offsets, T, B):
    indices = indices.contiguous().view(-1)
    rows = torch.empty_like(indices)
    with torch.cuda.device(indices.device):
        _native.check(_native.load().tbe_interleaved_rows(
            _ptr(indices), indices.numel(), _ptr(flat_offsets), T, B, _ptr(rows), _tbe._stream(indices.device)))
    return rows


def _dense_offsets(B, T, L, device):
    return torch.arange(0, B * T * L + 1, L, dtype=torch.int32, device=device)


def _flatten_offsets(offsets):
    """[B][T+1] with offsets[b][T] == offsets[b+1][0] -> [B*T+1]."""
    _require(offsets.dtype == torch.int32 and offsets.dim() == 2, "offsets must be an int32 [B, T+1] tensor")
    return torch.cat([offsets[:, :-1].reshape(-1), offsets[-1, -1:]]).contiguous()


def _zero(device):
    return torch.zeros(1, dtype=torch.int32, device=device)


def forward_fast_single(weights, indices):
    """sparse_embedding_cuda_forward_fast_single (sparse_embedding_cuda.cpp:265-274):
    weights [E][T][D], indices int32 [B][T][L] -> [B][T][D]."""
    E, T, D = _check(weights, indices)
    _require(indices.dim() == 3 and indices.size(1) == T, "indices must be [B, T, L]")
    B, _, L = indices.shape
    offsets = _dense_offsets(B, T, L, weights.device)
    out = _tbe.forward(weights.view(E * T, D), _zero(weights.device), _rows(indices, offsets, T, B), offsets, None,
                       200, 1, False)
    return out.view(B, T, D)


forward_single = forward_fast_single  # same contract, different launch geometry in the reference (:255-263)


def forward_offsets(weights, indices, offsets):
    """sparse_embedding_cuda_forward_offsets (sparse_embedding_cuda.cpp:276-288): flat indices,
    offsets int32 [B][T+1] -> [B][T][D]."""
    E, T, D = _check(weights, indices)
    _require(offsets.size(1) == T + 1, "offsets must be [B, T+1]")
    B = offsets.size(0)
    flat = _flatten_offsets(offsets)
    out = _tbe.forward(weights.view(E * T, D), _zero(weights.device), _rows(indices, flat, T, B), flat, None, 200, 1,
                       False)
    return out.view(B, T, D)


def backward_update_fast_single(grad_output, weights, indices, lr):
    """sparse_embedding_cuda_backward_update_fast_single (sparse_embedding_cuda.cpp:306-314), made
    exact: every distinct row receives -lr * (sum of its gradients) once (the reference's
    `weights[ind][t][d] -= lr * g` races on repeats, sparse_embedding_cuda_kernel.cu:493-497)."""
    E, T, D = _check(weights, indices)
    B, _, L = indices.shape
    offsets = _dense_offsets(B, T, L, weights.device)
    _tbe.backward_sgd(grad_output.contiguous().view(B * T, 1, D), weights.view(E * T, D), _zero(weights.device),
                      _rows(indices, offsets, T, B), offsets, lr, 200, 1, False)


backward_update_single = backward_update_fast_single


def backward_update_offsets(grad_output, weights, indices, offsets, lr):
    """sparse_embedding_cuda_backward_update_offsets (sparse_embedding_cuda.cpp:316-322), exact."""
    E, T, D = _check(weights, indices)
    B = offsets.size(0)
    flat = _flatten_offsets(offsets)
    _tbe.backward_sgd(grad_output.contiguous().view(B * T, 1, D), weights.view(E * T, D), _zero(weights.device),
                      _rows(indices, flat, T, B), flat, lr, 200, 1, False)


def _needs_more_gpus(*args, **kwargs):
    raise NotImplementedError("the collective entry points need more than one GPU and are not served")


forward = forward_all2all = forward_all2all_nccl = forward_reducescatter = forward_allgather = _needs_more_gpus
