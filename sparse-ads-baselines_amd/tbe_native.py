"""ctypes binding of libtbe_hip.so, the C-ABI library declared in include/tbe_hip.h.

The library is the only compute path: if it is missing or fails to load, every
operator raises.  There is no CPU or eager fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# TBE_HIP_LIBRARY names another build of the library (same ABI version, checked on load).
LIB_PATH = os.environ.get("TBE_HIP_LIBRARY") or os.path.join(_HERE, "libtbe_hip.so")

DTYPE_F32, DTYPE_F16, DTYPE_F64 = 0, 1, 2
ABI_VERSION = 22

_c_i32p = ctypes.c_void_p
_vp = ctypes.c_void_p
_i32 = ctypes.c_int32
_i64 = ctypes.c_int64
_u64 = ctypes.c_uint64
_f32 = ctypes.c_float


class WorkspaceLayout(ctypes.Structure):
    """Mirror of tbe_workspace_layout_t."""

    _fields_ = [
        ("total_bytes", _u64),
        ("keys", _u64),
        ("grad_rows", _u64),
        ("keys_sorted", _u64),
        ("positions_sorted", _u64),
        ("segment_starts", _u64),
        ("num_unique", _u64),
        ("sort_scratch", _u64),
        ("segment_scratch", _u64),
        ("segment_ids", _u64),
        ("long_segments", _u64),
        ("chunk_segments", _u64),
        ("partial_sums", _u64),
        ("max_long_segments", _i64),
        ("max_chunks", _i64),
        ("max_partial_rows", _i64),
    ]


class Cache(ctypes.Structure):
    """Mirror of tbe_cache_t."""

    _fields_ = [
        ("tags", _vp),
        ("last_used", _vp),
        ("use_count", _vp),
        ("rows", _vp),
        ("backing_rows", _vp),
        ("num_sets", _i64),
        ("policy", _i32),
        ("stage_slots", _i64),
        ("stage_of_row", _vp),
        ("stage_keys", _vp),
        ("total_rows", _i64),
        ("mixed_table_offsets", _vp),
        ("mixed_table_rows", _vp),
        ("mixed_dim_offsets", _vp),
        ("mixed_T", _i32),
    ]


class CacheWorkspaceLayout(ctypes.Structure):
    """Mirror of tbe_cache_workspace_layout_t."""

    _fields_ = [(name, _u64) for name in (
        "total_bytes", "unique_slots", "lookup_slots", "evicted_keys", "miss_sets", "miss_list",
        "set_counts", "set_fill", "set_starts", "stats", "fetch_source", "landing", "write_out")]


CACHE_WAYS = 64
STATIC_SCRATCH_BYTES = 32 << 20  # TBE_STATIC_SCRATCH_BYTES
CACHE_LRU, CACHE_LFU = 0, 1
OPT_SGD, OPT_ROWWISE_ADAGRAD, OPT_APPROX_ROWWISE_ADAGRAD = 0, 1, 2
_cache_p = ctypes.POINTER(Cache)

# name -> (restype, argtypes); exactly the declarations of include/tbe_hip.h
SIGNATURES = {
    "tbe_last_error": (ctypes.c_char_p, []),
    "tbe_abi_version": (_i32, []),
    "tbe_profile_begin": (ctypes.c_int, []),
    "tbe_profile_end": (ctypes.c_int, []),
    "tbe_profile_count": (_i32, []),
    "tbe_profile_get": (ctypes.c_int, [_i32, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(_f32)]),
    "tbe_probe_row_access": (ctypes.c_int, [_vp, _i32, _c_i32p, _i64, _vp, _i32, _vp, _vp]),
    "tbe_forward": (ctypes.c_int, [_vp, _i32, _i32, _c_i32p, _i32, _c_i32p, _i64, _c_i32p, _i32, _vp, _vp, _vp]),
    "tbe_backward_workspace_layout": (ctypes.c_int, [_i64, _i32, _i32, _i32, ctypes.POINTER(WorkspaceLayout)]),
    "tbe_backward_mixed_workspace_layout": (ctypes.c_int, [_i64, _i32, _i32, ctypes.POINTER(WorkspaceLayout)]),
    "tbe_backward_sgd": (ctypes.c_int, [_vp, _vp, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p, _i64, _c_i32p,
                                        _i32, _f32, _vp, _u64, _vp]),
    "tbe_backward_sgd_static": (ctypes.c_int, [_vp, _vp, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p, _i64,
                                               _c_i32p, _i32, _f32, _vp]),
    "tbe_backward_exact_adagrad": (ctypes.c_int, [_vp, _vp, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p, _i64,
                                                  _c_i32p, _i32, _vp, _vp, _f32, _f32, _vp, _vp, _u64, _vp]),
    "tbe_plan_batch": (ctypes.c_int, [_c_i32p, _i32, _c_i32p, _i64, _c_i32p, _i32, _i64, _i64, _i32, _i32, _vp, _u64, _vp]),
    "tbe_backward_planned": (ctypes.c_int, [_i32, _vp, _vp, _i32, _i64, _i32, _i32, _i32, _i64, _vp, _vp, _f32, _f32,
                                            _vp, _i32, _u64, _u64, _vp, _u64, _vp]),
    "tbe_linearize": (ctypes.c_int, [_c_i32p, _i32, _c_i32p, _i64, _c_i32p, _i32, _c_i32p, _c_i32p, _vp]),
    "tbe_forward_interleaved": (ctypes.c_int, [_vp, _i32, _i64, _i32, _i32, _c_i32p, _i64, _c_i32p, _i32, _i32, _vp,
                                               _vp]),
    "tbe_backward_interleaved_workspace_layout": (ctypes.c_int, [_i64, _i32, _i32, _i32, _i32,
                                                                 ctypes.POINTER(WorkspaceLayout)]),
    "tbe_backward_sgd_interleaved": (ctypes.c_int, [_vp, _vp, _i32, _i64, _i32, _i32, _c_i32p, _i64, _c_i32p, _i32,
                                                    _i32, _f32, _vp, _u64, _vp]),
    "tbe_sort_workspace_bytes": (_u64, [_i64]),
    "tbe_sort_pairs": (ctypes.c_int, [_c_i32p, _c_i32p, _c_i32p, _c_i32p, _i64, _i32, _vp, _u64, _vp]),
    "tbe_segments_workspace_bytes": (_u64, [_i64]),
    "tbe_find_segments": (ctypes.c_int, [_c_i32p, _i64, _c_i32p, _c_i32p, _vp, _u64, _vp]),
    "tbe_construct_offsets": (ctypes.c_int, [_c_i32p, _c_i32p, _i32, _i32, _c_i32p, _vp]),
    "tbe_stochastic_round": (ctypes.c_int, [_vp, _vp, _vp, _i64, _vp]),
    "tbe_forward_mixed": (ctypes.c_int, [_vp, _i32, _i32, _vp, _c_i32p, _i32, _i32, _c_i32p, _i64, _c_i32p, _i32, _vp,
                                         _vp, _vp]),
    "tbe_backward_mixed": (ctypes.c_int, [_i32, _vp, _vp, _i32, _i32, _i64, _i64, _vp, _c_i32p, _c_i32p, _i32, _i32,
                                          _c_i32p, _i64, _c_i32p, _i32, _vp, _vp, _f32, _f32, _vp, _i32, _u64, _u64,
                                          _vp, _u64, _vp]),
    "tbe_backward_exact_adagrad_stochastic": (ctypes.c_int, [_vp, _vp, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p,
                                                             _i64, _c_i32p, _i32, _vp, _vp, _f32, _f32, _vp, _u64,
                                                             _u64, _vp, _u64, _vp]),
    "tbe_backward_approx_adagrad": (ctypes.c_int, [_vp, _vp, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p, _i64,
                                                   _c_i32p, _i32, _vp, _vp, _f32, _f32, _vp, _i32, _u64, _u64, _vp,
                                                   _u64, _vp]),
    "tbe_cache_workspace_layout": (ctypes.c_int, [_i64, _i64, _i64, ctypes.POINTER(CacheWorkspaceLayout)]),
    "tbe_cache_init": (ctypes.c_int, [_cache_p, _vp]),
    "tbe_cache_prepare": (ctypes.c_int, [_cache_p, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p, _i64, _c_i32p, _i32,
                                         _i32, _i32, _vp, _u64, _vp, _u64, _vp, _vp]),
    "tbe_cache_plan": (ctypes.c_int, [_cache_p, _i32, _i64, _i64, _i32, _c_i32p, _i32, _c_i32p, _i64, _c_i32p, _i32,
                                      _i32, _i32, _vp, _u64, _vp, _u64, _vp, _vp]),
    "tbe_cache_commit": (ctypes.c_int, [_cache_p, _i32, _i32, _i32, _i64, _i32, _vp, _u64, _vp, _u64, _vp]),
    "tbe_forward_cached": (ctypes.c_int, [_cache_p, _i32, _i32, _c_i32p, _i32, _c_i32p, _i64, _c_i32p, _i32, _vp,
                                          _c_i32p, _vp, _vp]),
    "tbe_backward_cached": (ctypes.c_int, [_i32, _vp, _cache_p, _i32, _i64, _i32, _i32, _i32, _i64, _vp, _vp, _f32,
                                           _f32, _vp, _i32, _u64, _u64, _vp, _u64, _c_i32p, _vp]),
    "tbe_backward_approx_cached": (ctypes.c_int, [_vp, _cache_p, _i32, _i64, _i32, _i32, _i32, _i64, _c_i32p, _vp, _vp,
                                                  _f32, _f32, _vp, _i32, _u64, _u64, _vp, _u64, _c_i32p, _vp]),
    "tbe_cache_flush": (ctypes.c_int, [_cache_p, _i32, _i32, ctypes.c_uint32, _i32, _vp]),
    "tbe_forward_mixed_cached": (ctypes.c_int, [_cache_p, _i32, _i32, _i32, _i32, _c_i32p, _i64, _c_i32p, _i32, _vp,
                                                _c_i32p, _vp, _vp]),
    "tbe_backward_mixed_cached": (ctypes.c_int, [_i32, _vp, _cache_p, _i32, _i32, _i32, _i32, _i32, _i64, _c_i32p, _vp,
                                                 _vp, _f32, _f32, _vp, _i32, _u64, _u64, _vp, _u64, _c_i32p, _vp]),
    "tbe_host_mapped_alloc": (ctypes.c_int, [_u64, ctypes.POINTER(_vp), ctypes.POINTER(_vp)]),
    "tbe_host_mapped_free": (ctypes.c_int, [_vp]),
    "tbe_managed_alloc": (ctypes.c_int, [_u64, _i32, ctypes.POINTER(_vp)]),
    "tbe_managed_free": (ctypes.c_int, [_vp]),
}

_lib = None


def load():
    """Loads the library once and attaches the prototypes.  Raises if it is absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "%s is missing: build it with `python %s` (needs hipcc); there is no fallback path"
            % (LIB_PATH, os.path.join(_HERE, "build.py"))
        )
    # The library needs libamdhip64.so.7 by soname.  PyTorch ships its own copy of that
    # runtime; importing torch first makes the loader reuse it, so the kernels launched here
    # and torch's allocator and streams share one HIP runtime.  Loaded the other way round,
    # the process would hold two runtimes and torch's streams would be foreign to this one.
    import torch  # noqa: F401

    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code):
    """Turns a non-zero return code into RuntimeError, the exception AT_ASSERT /
    AT_CUDA_CHECK surface as in the reference (table_batched_embeddings_cuda.cu:262-273, 314)."""
    if code != 0:
        msg = load().tbe_last_error()
        raise RuntimeError(msg.decode("utf-8", "replace") if msg else "tbe error %d" % code)


def backward_workspace_layout(num_indices, D, dtype_code, T):
    layout = WorkspaceLayout()
    check(load().tbe_backward_workspace_layout(num_indices, D, dtype_code, T, ctypes.byref(layout)))
    return layout


def backward_mixed_workspace_layout(num_indices, dtype_code, T):
    layout = WorkspaceLayout()
    check(load().tbe_backward_mixed_workspace_layout(num_indices, dtype_code, T, ctypes.byref(layout)))
    return layout


def backward_interleaved_workspace_layout(num_indices, D, dtype_code, T, B):
    layout = WorkspaceLayout()
    check(load().tbe_backward_interleaved_workspace_layout(num_indices, D, dtype_code, T, B, ctypes.byref(layout)))
    return layout


def cache_workspace_layout(num_indices, num_sets, stage_slots=0):
    layout = CacheWorkspaceLayout()
    check(load().tbe_cache_workspace_layout(num_indices, num_sets, stage_slots, ctypes.byref(layout)))
    return layout


class profile:
    """Context manager: times every kernel launched by the library inside the block.

    After the block, `.launches` is a list of (kernel name, milliseconds) in launch order."""

    def __enter__(self):
        check(load().tbe_profile_begin())
        self.launches = []
        return self

    def __exit__(self, *exc):
        lib = load()
        check(lib.tbe_profile_end())
        name, ms = ctypes.c_char_p(), _f32()
        for i in range(lib.tbe_profile_count()):
            check(lib.tbe_profile_get(i, ctypes.byref(name), ctypes.byref(ms)))
            self.launches.append((name.value.decode(), ms.value))
        return False
