"""CPU-side checks of the C-ABI library: it loads, exports every symbol that
include/tbe_hip.h declares, and rejects bad arguments before touching a device."""
import ctypes
import os
import re

import pytest

from conftest import ROOT

import tbe_native

HEADER = os.path.join(ROOT, "include", "tbe_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    return sorted(set(re.findall(r"TBE_API[^;(]*?\b(tbe_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("tbe_forward", "tbe_backward_sgd", "tbe_backward_exact_adagrad", "tbe_linearize", "tbe_sort_pairs",
                 "tbe_find_segments", "tbe_construct_offsets", "tbe_host_mapped_alloc", "tbe_managed_alloc",
                 "tbe_backward_workspace_layout", "tbe_last_error"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = tbe_native.load()
    for name in declared_symbols():
        assert hasattr(lib, name), "libtbe_hip.so does not export %s" % name


def test_python_binding_covers_every_declared_symbol():
    assert sorted(tbe_native.SIGNATURES) == declared_symbols()


def test_abi_version_matches_binding():
    assert tbe_native.load().tbe_abi_version() == tbe_native.ABI_VERSION


def test_workspace_layout_is_ordered_and_sized():
    lay = tbe_native.backward_workspace_layout(5242880, 128, tbe_native.DTYPE_F32, 64)
    offs = [lay.keys, lay.grad_rows, lay.keys_sorted, lay.positions_sorted, lay.segment_starts, lay.num_unique,
            lay.sort_scratch, lay.segment_scratch, lay.segment_ids, lay.long_segments, lay.chunk_segments,
            lay.partial_sums]
    assert offs == sorted(offs) and len(set(offs)) == len(offs)
    assert all(o % 256 == 0 for o in offs)
    assert lay.grad_rows - lay.keys == 256  # 64 tables are sorted apart: no linearized keys are kept
    many = tbe_native.backward_workspace_layout(5242880, 128, tbe_native.DTYPE_F32, 4096)
    assert many.grad_rows - many.keys >= 5242880 * 4  # more tables than are sorted apart: keys sorted in one piece
    assert lay.total_bytes >= lay.partial_sums + lay.max_partial_rows * 128 * 4
    assert lay.partial_sums - lay.chunk_segments >= lay.max_chunks * 32
    assert lay.total_bytes < 512 << 20
    half = tbe_native.backward_workspace_layout(1000, 64, tbe_native.DTYPE_F16, 3)
    dbl = tbe_native.backward_workspace_layout(1000, 64, tbe_native.DTYPE_F64, 3)
    assert dbl.total_bytes > half.total_bytes  # fp64 partial sums are 8 bytes wide


def _null():
    return ctypes.c_void_p(0)


def _fake():
    return ctypes.c_void_p(4096)  # never dereferenced: validation fails first


@pytest.mark.parametrize("D,T,B,needle", [(6, 1, 1, "multiple of 4"), (0, 1, 1, "D must be positive"),
                                          (4, 0, 1, "T must be positive"), (4, 1, 0, "B must be positive")])
def test_forward_rejects_bad_shapes_like_the_reference_asserts(D, T, B, needle):
    # table_batched_embeddings_cuda.cu:262-273: AT_ASSERT(T > 0), (D > 0), (B > 0), (D % 4 == 0)
    lib = tbe_native.load()
    rc = lib.tbe_forward(_fake(), 0, D, _fake(), T, _fake(), 4, _fake(), B, _null(), _fake(), _null())
    assert rc == 1
    assert needle in lib.tbe_last_error().decode()
    with pytest.raises(RuntimeError, match=needle):
        tbe_native.check(rc)


def test_null_pointers_and_bad_dtype_are_rejected():
    lib = tbe_native.load()
    assert lib.tbe_forward(_null(), 0, 4, _fake(), 1, _fake(), 4, _fake(), 1, _null(), _fake(), _null()) == 1
    assert lib.tbe_forward(_fake(), 7, 4, _fake(), 1, _fake(), 4, _fake(), 1, _null(), _fake(), _null()) == 1
    assert "dtype" in lib.tbe_last_error().decode()


def test_backward_rejects_small_workspace_and_mismatched_weighting():
    lib = tbe_native.load()
    rc = lib.tbe_backward_sgd(_fake(), _fake(), 0, 100, 0, 4, _fake(), 1, _fake(), 10, _fake(), 1, 0.1, _fake(), 16,
                              _null())
    assert rc == 2 and "workspace" in lib.tbe_last_error().decode()
    rc = lib.tbe_backward_exact_adagrad(_fake(), _fake(), 0, 100, 0, 4, _fake(), 1, _fake(), 10, _fake(), 1, _fake(),
                                        _fake(), 0.1, 0.1, _null(), _fake(), 1 << 30, _null())
    assert rc == 1 and "per_sample_weights" in lib.tbe_last_error().decode()
    rc = lib.tbe_backward_exact_adagrad(_fake(), _fake(), 0, 100, 0, 4, _fake(), 1, _fake(), 10, _fake(), 1, _null(),
                                        _null(), 0.1, 0.1, _null(), _fake(), 1 << 30, _null())
    assert rc == 1 and "optimizer_state" in lib.tbe_last_error().decode()


def test_sort_and_segment_workspace_queries():
    lib = tbe_native.load()
    assert lib.tbe_sort_workspace_bytes(0) > 0
    small, big = lib.tbe_sort_workspace_bytes(1000), lib.tbe_sort_workspace_bytes(5242880)
    assert big > small >= 2 * 1000 * 4
    assert lib.tbe_segments_workspace_bytes(5242880) >= 5242880 // 2048 * 4
    # a workspace sized for a maximum serves every smaller batch, also across the switch of tile sizes
    sizes = [lib.tbe_sort_workspace_bytes(n) for n in (1, 1000, 262144, 524287, 524288, 524289, 600000, 700000,
                                                       1 << 20, 5242880)]
    assert sizes == sorted(sizes)
    layouts = [tbe_native.backward_workspace_layout(n, 128, tbe_native.DTYPE_F32, 64).total_bytes
               for n in (1000, 524288, 524289, 600000, 1 << 20)]
    assert layouts == sorted(layouts)
    assert lib.tbe_sort_pairs(_fake(), _null(), _fake(), _fake(), 10, 40, _fake(), 1 << 20, _null()) == 1
    assert lib.tbe_sort_pairs(_fake(), _null(), _fake(), _fake(), 10, 8, _fake(), 8, _null()) == 2


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(tbe_native, "_lib", None)
    monkeypatch.setattr(tbe_native, "LIB_PATH", str(tmp_path / "absent.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        tbe_native.load()
