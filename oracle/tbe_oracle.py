"""numpy-facing wrapper of the C oracle (oracle/tbe_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py as the checker.  The shipped package never imports it.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtbe_oracle.so")
_lib = None

F32, F16, F64 = 0, 1, 2
_CODES = {np.dtype(np.float32): F32, np.dtype(np.float16): F16, np.dtype(np.float64): F64}


def build():
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "libtbe_oracle.so"], check=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_half_to_float.restype = ctypes.c_float
        _lib.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        _lib.oracle_float_to_half.restype = ctypes.c_uint16
        _lib.oracle_float_to_half.argtypes = [ctypes.c_float]
        _lib.oracle_segments.restype = ctypes.c_int64
    return _lib


def _p(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else ctypes.c_void_p(0)


def _i32(a):
    a = np.ascontiguousarray(a, dtype=np.int32)
    return a


def forward(weights, table_offsets, indices, offsets, per_sample_weights=None):
    """-> output [B, T, D] in the weights' dtype."""
    weights = np.ascontiguousarray(weights)
    code = _CODES[weights.dtype]
    table_offsets, indices, offsets = _i32(table_offsets), _i32(indices), _i32(offsets)
    T = table_offsets.size
    B = (offsets.size - 1) // T
    D = weights.shape[1]
    psw = None if per_sample_weights is None else np.ascontiguousarray(per_sample_weights, dtype=weights.dtype)
    out = np.empty((B, T, D), dtype=weights.dtype)
    lib().oracle_forward(_p(weights), code, ctypes.c_int32(D), _p(table_offsets), ctypes.c_int32(T), _p(indices),
                         _p(offsets), ctypes.c_int32(B), _p(psw), _p(out))
    return out


def linearize(table_offsets, indices, offsets):
    """-> keys, info_b_t, info_indices_idx (all int32 [N])."""
    table_offsets, indices, offsets = _i32(table_offsets), _i32(indices), _i32(offsets)
    T = table_offsets.size
    B = (offsets.size - 1) // T
    n = indices.size
    keys, b_t, idx = (np.empty(n, np.int32) for _ in range(3))
    lib().oracle_linearize(_p(table_offsets), ctypes.c_int32(T), _p(indices), _p(offsets), ctypes.c_int32(B),
                           _p(keys), _p(b_t), _p(idx))
    return keys, b_t, idx


def sort_pairs(keys, values, end_bit):
    keys = _i32(keys)
    values = None if values is None else _i32(values)
    ko, vo = np.empty(keys.size, np.int32), np.empty(keys.size, np.int32)
    lib().oracle_sort_pairs(_p(keys), _p(values), _p(ko), _p(vo), ctypes.c_int64(keys.size), ctypes.c_int32(end_bit))
    return ko, vo


def segments(keys_sorted):
    keys_sorted = _i32(keys_sorted)
    starts = np.empty(keys_sorted.size + 1, np.int32)
    U = lib().oracle_segments(_p(keys_sorted), ctypes.c_int64(keys_sorted.size), _p(starts))
    return starts[: U + 1].copy()


def backward(optimizer, grad_output, weights, table_offsets, indices, offsets, lr, eps=0.0,
             optimizer_state=None, per_sample_weights=None, stochastic_rounding=None):
    """In-place update of `weights` (and `optimizer_state`); optimizer 'sgd' or 'adagrad'.

    stochastic_rounding: None or (seed, offset) for fp16 weights.
    Returns dict(keys_sorted, positions_sorted, segment_starts, grad_psw)."""
    assert weights.flags["C_CONTIGUOUS"] and weights.dtype in _CODES
    code = _CODES[weights.dtype]
    grad_output = np.ascontiguousarray(grad_output, dtype=weights.dtype)
    table_offsets, indices, offsets = _i32(table_offsets), _i32(indices), _i32(offsets)
    T = table_offsets.size
    B = (offsets.size - 1) // T
    D = weights.shape[1]
    n = indices.size
    assert grad_output.shape == (B, T, D)
    psw = gpsw = None
    if per_sample_weights is not None:
        psw = np.ascontiguousarray(per_sample_weights, dtype=weights.dtype)
        gpsw = np.zeros(n, dtype=weights.dtype)
    opt = {"sgd": 0, "adagrad": 1}[optimizer]
    if opt == 1:
        want = np.float64 if weights.dtype == np.float64 else np.float32
        assert optimizer_state is not None and optimizer_state.dtype == want
        assert optimizer_state.flags["C_CONTIGUOUS"]
    ks, ps, ss = np.empty(n, np.int32), np.empty(n, np.int32), np.empty(n + 1, np.int32)
    U = ctypes.c_int64(0)
    lib().oracle_backward(ctypes.c_int(opt), _p(grad_output), _p(weights), ctypes.c_int(code),
                          ctypes.c_int64(weights.shape[0]), ctypes.c_int32(D), _p(table_offsets), ctypes.c_int32(T),
                          _p(indices), ctypes.c_int64(n), _p(offsets), ctypes.c_int32(B), _p(psw),
                          _p(optimizer_state), ctypes.c_float(lr), ctypes.c_float(eps), _p(gpsw), _p(ks), _p(ps),
                          _p(ss), ctypes.byref(U), ctypes.c_int32(0 if stochastic_rounding is None else 1),
                          ctypes.c_uint64(0 if stochastic_rounding is None else stochastic_rounding[0]),
                          ctypes.c_uint64(0 if stochastic_rounding is None else stochastic_rounding[1]))
    return {"keys_sorted": ks, "positions_sorted": ps, "segment_starts": ss[: U.value + 1].copy(), "grad_psw": gpsw}


def backward_approx(grad_output, weights, table_offsets, indices, offsets, lr, eps, optimizer_state,
                    per_sample_weights=None, stochastic_rounding=None):
    """Approximate row-wise Adagrad, one lookup at a time in position order (oracle_backward_approx):
    in place on `weights` [rows, D] and `optimizer_state`; returns grad_psw or None."""
    assert weights.flags["C_CONTIGUOUS"] and weights.ndim == 2 and weights.dtype in _CODES
    code = _CODES[weights.dtype]
    grad_output = np.ascontiguousarray(grad_output, dtype=weights.dtype)
    table_offsets, indices, offsets = _i32(table_offsets), _i32(indices), _i32(offsets)
    T = table_offsets.size
    B = (offsets.size - 1) // T
    D = weights.shape[1]
    assert grad_output.shape == (B, T, D)
    want = np.float64 if weights.dtype == np.float64 else np.float32
    assert optimizer_state.dtype == want and optimizer_state.flags["C_CONTIGUOUS"]
    psw = gpsw = None
    if per_sample_weights is not None:
        psw = np.ascontiguousarray(per_sample_weights, dtype=weights.dtype)
        gpsw = np.zeros(indices.size, dtype=weights.dtype)
    sr = stochastic_rounding
    lib().oracle_backward_approx(_p(grad_output), _p(weights), ctypes.c_int(code), ctypes.c_int64(weights.shape[0]),
                                 ctypes.c_int32(D), _p(table_offsets), None, None, None, ctypes.c_int32(0),
                                 ctypes.c_int32(T), _p(indices), _p(offsets), ctypes.c_int32(B), _p(psw),
                                 _p(optimizer_state), ctypes.c_float(lr), ctypes.c_float(eps), _p(gpsw),
                                 ctypes.c_int32(0 if sr is None else 1), ctypes.c_uint64(0 if sr is None else sr[0]),
                                 ctypes.c_uint64(0 if sr is None else sr[1]))
    return gpsw


def backward_approx_mixed(grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, indices, offsets, lr,
                          eps, optimizer_state, per_sample_weights=None, stochastic_rounding=None):
    """The same for tables with per-table dimension (flat 1-D weights, grad_output [B, total_D])."""
    assert weights.flags["C_CONTIGUOUS"] and weights.ndim == 1
    code = _CODES[weights.dtype]
    grad_output = np.ascontiguousarray(grad_output, dtype=weights.dtype)
    table_offsets = np.ascontiguousarray(table_offsets, dtype=np.int64)
    table_dim_offsets, dim_offsets = _i32(table_dim_offsets), _i32(dim_offsets)
    indices, offsets = _i32(indices), _i32(offsets)
    T = table_offsets.size - 1
    B = (offsets.size - 1) // T
    total_D = int(dim_offsets[-1])
    assert grad_output.shape == (B, total_D)
    psw = gpsw = None
    if per_sample_weights is not None:
        psw = np.ascontiguousarray(per_sample_weights, dtype=weights.dtype)
        gpsw = np.zeros(indices.size, dtype=weights.dtype)
    sr = stochastic_rounding
    lib().oracle_backward_approx(_p(grad_output), _p(weights), ctypes.c_int(code),
                                 ctypes.c_int64(int(table_dim_offsets[-1])), ctypes.c_int32(0), None,
                                 _p(table_offsets), _p(table_dim_offsets), _p(dim_offsets), ctypes.c_int32(total_D),
                                 ctypes.c_int32(T), _p(indices), _p(offsets), ctypes.c_int32(B), _p(psw),
                                 _p(optimizer_state), ctypes.c_float(lr), ctypes.c_float(eps), _p(gpsw),
                                 ctypes.c_int32(0 if sr is None else 1), ctypes.c_uint64(0 if sr is None else sr[0]),
                                 ctypes.c_uint64(0 if sr is None else sr[1]))
    return gpsw


def construct_offsets(batch_offsets_per_table, total_indices_per_table):
    per_table = _i32(batch_offsets_per_table)
    totals = _i32(total_indices_per_table)
    T, B = per_table.shape
    out = np.empty(1 + T * B, np.int32)
    lib().oracle_construct_offsets(_p(per_table), _p(totals), ctypes.c_int32(T), ctypes.c_int32(B), _p(out))
    return out


def half_to_float(bits):
    return lib().oracle_half_to_float(int(bits))


def float_to_half(value):
    return lib().oracle_float_to_half(float(value))


# ------------------------------------------------------------------ row cache model
class CacheModel:
    """State and step function of the row-cache specification (oracle/lxu_cache_model.c)."""

    WAYS = 64

    def __init__(self, num_sets, policy="lru"):
        self.num_sets = int(num_sets)
        self.policy = {"lru": 0, "lfu": 1}[policy]
        n = self.num_sets * self.WAYS
        self.tags = np.full(n, -1, np.int32)
        self.last_used = np.zeros(n, np.int32)
        self.use_count = np.zeros(n, np.int32)
        self.step_no = 0

    def step(self, unique_keys):
        """unique_keys: strictly ascending int32.  -> (unique_slots, evicted_keys, stats[6])"""
        keys = _i32(unique_keys)
        self.step_no += 1
        slots = np.empty(keys.size, np.int32)
        evicted = np.empty(keys.size, np.int32)
        stats = np.zeros(6, np.int32)
        lib().lxu_cache_step(_p(self.tags), _p(self.last_used), _p(self.use_count), ctypes.c_int64(self.num_sets),
                             ctypes.c_int32(self.policy), ctypes.c_int32(self.step_no), _p(keys),
                             ctypes.c_int64(keys.size), _p(slots), _p(evicted), _p(stats))
        return slots, evicted, stats

    def resident(self):
        return np.sort(self.tags[self.tags >= 0])


def cache_set_of(key, num_sets):
    fn = lib().lxu_set_of
    fn.restype = ctypes.c_uint32
    return fn(ctypes.c_uint32(int(key)), ctypes.c_uint32(int(num_sets)))


# ------------------------------------------------------------ per-table dimension
def forward_mixed(weights, table_offsets, dim_offsets, indices, offsets, per_sample_weights=None):
    """weights 1-D; table_offsets int64 [T+1]; dim_offsets int32 [T+1] -> output [B, total_D]."""
    weights = np.ascontiguousarray(weights)
    code = _CODES[weights.dtype]
    table_offsets = np.ascontiguousarray(table_offsets, dtype=np.int64)
    dim_offsets, indices, offsets = _i32(dim_offsets), _i32(indices), _i32(offsets)
    T = table_offsets.size - 1
    B = (offsets.size - 1) // T
    total_D = int(dim_offsets[-1])
    psw = None if per_sample_weights is None else np.ascontiguousarray(per_sample_weights, dtype=weights.dtype)
    out = np.empty((B, total_D), dtype=weights.dtype)
    lib().oracle_forward_mixed(_p(weights), ctypes.c_int(code), _p(table_offsets), _p(dim_offsets),
                               ctypes.c_int32(total_D), ctypes.c_int32(T), _p(indices), _p(offsets),
                               ctypes.c_int32(B), _p(psw), _p(out))
    return out


def backward_mixed(optimizer, grad_output, weights, table_offsets, table_dim_offsets, dim_offsets, indices, offsets,
                   lr, eps=0.0, optimizer_state=None, per_sample_weights=None):
    """In-place on `weights` (1-D) and `optimizer_state`; returns grad_psw or None."""
    assert weights.flags["C_CONTIGUOUS"] and weights.ndim == 1
    code = _CODES[weights.dtype]
    grad_output = np.ascontiguousarray(grad_output, dtype=weights.dtype)
    table_offsets = np.ascontiguousarray(table_offsets, dtype=np.int64)
    table_dim_offsets, dim_offsets = _i32(table_dim_offsets), _i32(dim_offsets)
    indices, offsets = _i32(indices), _i32(offsets)
    T = table_offsets.size - 1
    B = (offsets.size - 1) // T
    total_D = int(dim_offsets[-1])
    assert grad_output.shape == (B, total_D)
    psw = gpsw = None
    if per_sample_weights is not None:
        psw = np.ascontiguousarray(per_sample_weights, dtype=weights.dtype)
        gpsw = np.zeros(indices.size, dtype=weights.dtype)
    opt = {"sgd": 0, "adagrad": 1}[optimizer]
    lib().oracle_backward_mixed(ctypes.c_int(opt), _p(grad_output), _p(weights), ctypes.c_int(code),
                                ctypes.c_int64(int(table_dim_offsets[-1])), _p(table_offsets), _p(table_dim_offsets),
                                _p(dim_offsets), ctypes.c_int32(total_D), ctypes.c_int32(T), _p(indices),
                                ctypes.c_int64(indices.size), _p(offsets), ctypes.c_int32(B), _p(psw),
                                _p(optimizer_state), ctypes.c_float(lr), ctypes.c_float(eps), _p(gpsw))
    return gpsw


def philox4x32_10(counter, key):
    ctr = (ctypes.c_uint32 * 4)(*counter)
    k = (ctypes.c_uint32 * 2)(*key)
    out = (ctypes.c_uint32 * 4)()
    lib().oracle_philox4x32_10(ctr, k, out)
    return list(out)


def stochastic_round(value, random_bits):
    fn = lib().oracle_stochastic_round
    fn.restype = ctypes.c_uint16
    fn.argtypes = [ctypes.c_float, ctypes.c_uint32]
    return fn(float(value), int(random_bits))


def stochastic_round_many(values, random_bits):
    """oracle_stochastic_round over arrays: float32 values, uint32 words -> uint16 fp16 patterns."""
    values = np.ascontiguousarray(values, dtype=np.float32)
    random_bits = np.ascontiguousarray(random_bits, dtype=np.uint32)
    out = np.empty(values.shape, np.uint16)
    lib().oracle_stochastic_round_many(values.ctypes.data_as(ctypes.c_void_p), random_bits.ctypes.data_as(ctypes.c_void_p),
                                       out.ctypes.data_as(ctypes.c_void_p), ctypes.c_int64(values.size))
    return out


# ------------------------------------------------------ interleaved [E][T][D] tables
def forward_etd(weights, indices, offsets):
    """weights float32 [E, T, D]; offsets flattened [B*T+1] -> output [B, T, D]."""
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    E, T, D = weights.shape
    indices, offsets = _i32(indices), _i32(offsets)
    B = (offsets.size - 1) // T
    out = np.empty((B, T, D), np.float32)
    lib().oracle_forward_etd(_p(weights), ctypes.c_int32(E), ctypes.c_int32(T), ctypes.c_int32(D), _p(indices),
                             _p(offsets), ctypes.c_int32(B), _p(out))
    return out


def backward_etd(grad_output, weights, indices, offsets, lr):
    """In-place exact SGD on weights float32 [E, T, D]."""
    assert weights.dtype == np.float32 and weights.flags["C_CONTIGUOUS"]
    E, T, D = weights.shape
    indices, offsets = _i32(indices), _i32(offsets)
    B = (offsets.size - 1) // T
    grad_output = np.ascontiguousarray(grad_output, dtype=np.float32)
    lib().oracle_backward_etd(_p(grad_output), _p(weights), ctypes.c_int32(E), ctypes.c_int32(T), ctypes.c_int32(D),
                              _p(indices), _p(offsets), ctypes.c_int32(B), ctypes.c_float(lr))
