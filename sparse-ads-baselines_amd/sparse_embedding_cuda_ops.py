"""Drop-in for the single-GPU part of the reference's sparse_embedding_cuda_ops.py (:24-75):
`UniformShardedEmbeddingBags` with weights [E][T][D], dense [B][T][L] indices or flat indices
plus [B][T+1] offsets, and a fused SGD update with the reference's fixed learning rate.
The collective Functions and FastZeroFusedSGD of that file are not served."""
import enum
import logging

import torch
from torch import nn

import sparse_embedding_cuda
import table_batched_embeddings


class LookupFunction(torch.autograd.Function):
    """Mirror of LookupFunction (sparse_embedding_cuda_ops.py:24-45)."""

    @staticmethod
    def forward(ctx, weights, indices, offsets=None):
        ctx.save_for_backward(weights, indices, offsets)
        if offsets is None:
            return sparse_embedding_cuda.forward_fast_single(weights, indices)
        return sparse_embedding_cuda.forward_offsets(weights, indices, offsets)

    @staticmethod
    def backward(ctx, grad_output):
        weights, indices, offsets = ctx.saved_tensors
        LR = 0.05  # the reference hard-codes it (sparse_embedding_cuda_ops.py:36-37)
        if offsets is None:
            sparse_embedding_cuda.backward_update_fast_single(grad_output, weights, indices, LR)
        else:
            sparse_embedding_cuda.backward_update_offsets(grad_output, weights, indices, offsets, LR)
        empty_grad = torch.sparse_coo_tensor(
            torch.empty((3, 0), dtype=torch.int64, device=weights.device),
            torch.empty((0,), dtype=weights.dtype, device=weights.device), size=tuple(weights.shape))
        return (empty_grad, None, None)


class EmbeddingLocation(enum.Enum):
    DEVICE = 0
    MANAGED = 1
    HOST_MAPPED = 2


class UniformShardedEmbeddingBags(nn.Module):
    """Mirror of UniformShardedEmbeddingBags (sparse_embedding_cuda_ops.py:54-75)."""

    def __init__(self, num_tables, num_embeddings, embedding_dim, managed=EmbeddingLocation.DEVICE, fp16=False):
        super(UniformShardedEmbeddingBags, self).__init__()
        dtype = torch.float16 if fp16 else torch.float32
        device = torch.device("cuda", torch.cuda.current_device())
        shape = (num_embeddings, num_tables, embedding_dim)
        if managed == EmbeddingLocation.DEVICE:
            logging.info("Allocating device embedding bag")
            embedding_data = torch.randn(*shape, device=device, dtype=dtype)
        else:
            logging.info("Allocating managed embedding bag")
            embedding_data = table_batched_embeddings.new_managed_tensor(torch.empty(1, device=device, dtype=dtype),
                                                                         shape)
            embedding_data.normal_()
        self.embedding_weights = nn.Parameter(embedding_data)

    def forward(self, sharded_sparse_features, sharded_offsets=None):
        return LookupFunction.apply(self.embedding_weights, sharded_sparse_features, sharded_offsets)
