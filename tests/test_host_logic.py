"""CPU-side checks of the Python host layer that mirrors table_batched_embeddings_ops.py
and the extension module's surface (table_batched_embeddings.cpp:56-70)."""
import inspect

import pytest
import torch

import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops


def test_enums_keep_reference_values():
    # table_batched_embeddings_ops.py:124-132
    assert [(e.name, e.value) for e in ops.Optimizer] == [("SGD", 1), ("APPROX_ROWWISE_ADAGRAD", 2),
                                                          ("EXACT_ROWWISE_ADAGRAD", 3)]
    # DEVICE / HOST_MAPPED as in the reference; HOST_CACHED is this library's extension
    assert [(e.name, e.value) for e in ops.EmbeddingLocation] == [("DEVICE", 0), ("HOST_MAPPED", 1),
                                                                   ("HOST_CACHED", 2)]


def test_extension_module_exports_the_ten_reference_functions():
    for name in ("forward", "backward_sgd", "backward_approx_adagrad", "backward_exact_adagrad",
                 "backward_approx_adagrad_mixed_D", "backward_exact_adagrad_mixed_D", "forward_mixed_D",
                 "construct_offsets", "new_managed_tensor", "new_host_mapped_tensor"):
        assert callable(getattr(ext, name))


def test_positional_signatures_match_the_pybind_declarations():
    # table_batched_embeddings.cpp:6-27
    assert list(inspect.signature(ext.forward).parameters) == [
        "weights", "table_offsets", "indices", "offsets", "indice_weights", "L_max", "BT_block_size", "shmem"]
    assert list(inspect.signature(ext.backward_sgd).parameters) == [
        "grad_output", "weights", "table_offsets", "indices", "offsets", "learning_rate", "L_max", "BT_block_size",
        "shmem"]
    assert list(inspect.signature(ext.backward_exact_adagrad).parameters) == [
        "grad_output", "weights", "table_offsets", "indices", "offsets", "indice_weights", "optimizer_state",
        "learning_rate", "eps", "stochastic_rounding", "BT_block_size"]
    assert list(inspect.signature(ext.backward_approx_adagrad).parameters) == [
        "grad_output", "weights", "table_offsets", "indices", "offsets", "indice_weights", "optimizer_state",
        "learning_rate", "eps", "L_max", "stochastic_rounding", "BT_block_size"]


def test_module_constructor_signature_matches_reference():
    # table_batched_embeddings_ops.py:136-147
    params = inspect.signature(ops.TableBatchedEmbeddingBags.__init__).parameters
    # the reference's nine arguments in order, then the cache extension
    assert list(params)[1:] == ["num_tables", "num_embeddings", "embedding_dim", "optimizer", "learning_rate", "eps",
                                "stochastic_rounding", "fp16", "managed", "cache_slots", "cache_policy",
                                "cache_stage_slots"]
    assert params["optimizer"].default is ops.Optimizer.SGD
    assert params["learning_rate"].default == 0.01
    assert params["managed"].default is ops.EmbeddingLocation.DEVICE
    fwd = inspect.signature(ops.TableBatchedEmbeddingBags.forward).parameters
    assert list(fwd)[1:] == ["sharded_sparse_features", "sharded_offsets", "per_sample_weights"]


def test_cpu_tensors_are_rejected_not_silently_computed():
    w = torch.zeros(8, 4)
    i32 = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(RuntimeError, match="GPU tensor"):
        ext.forward(w, i32[:1], i32, i32, None, 200, 1, False)


def test_mixed_d_signatures_match_the_pybind_declarations():
    # table_batched_embeddings.cpp:32-50
    assert list(inspect.signature(ext.forward_mixed_D).parameters) == [
        "weights", "table_offsets", "dim_offsets", "total_D", "indices", "offsets", "indice_weights", "L_max",
        "BT_block_size", "shmem"]
    assert list(inspect.signature(ext.backward_exact_adagrad_mixed_D).parameters) == [
        "grad_output", "weights", "table_offsets", "table_dim_offsets", "dim_offsets", "total_D", "indices",
        "offsets", "indice_weights", "optimizer_state", "learning_rate", "eps", "stochastic_rounding",
        "BT_block_size"]
    assert list(inspect.signature(ext.backward_approx_adagrad_mixed_D).parameters) == [
        "grad_output", "weights", "table_offsets", "table_dim_offsets", "dim_offsets", "total_D", "indices",
        "offsets", "indice_weights", "optimizer_state", "learning_rate", "eps", "L_max", "stochastic_rounding",
        "BT_block_size"]
    params = inspect.signature(ops.MixedDimTableBatchedEmbeddingBags.__init__).parameters
    assert list(params)[1:] == ["embeddings", "optimizer", "learning_rate", "eps", "stochastic_rounding", "fp16",
                                "managed"]
    for helper in ("split_embedding_weights", "split_optimizer_state", "split_output"):
        assert callable(getattr(ops.MixedDimTableBatchedEmbeddingBags, helper))


def test_bench_refuses_more_than_one_gpu():
    import os
    import subprocess
    import sys
    from conftest import ROOT
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True,
                         text=True, timeout=120)
    assert out.returncode != 0 and "one GPU" in out.stderr and out.stdout.strip() == ""
