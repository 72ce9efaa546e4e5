"""fp16 stochastic rounding of the updated weights (tbe_backward_exact_adagrad_stochastic).

The reference's random stream (cuRAND Philox per thread, table_batched_embeddings_cuda.cu:627-631)
cannot be reproduced, so parity with the reference is statistical only -- the reference's own
test merely bounds the error (test_table_batched_embeddings.py:300-318, atol 1e-3).  Against
this repository's oracle, which uses the same counter layout, the result is compared exactly
wherever the fp32 value before rounding agrees."""
import ctypes

import numpy as np
import pytest
import torch

from conftest import make_problem
from gpu_util import DEV, dev

import table_batched_embeddings as ext
import table_batched_embeddings_ops as ops
import tbe_native

pytestmark = pytest.mark.gpu


def _run(p, seed, offset, weighted=False):
    w = dev(p["weights"])
    st = torch.zeros(w.shape[0], device=DEV)
    lay = tbe_native.backward_workspace_layout(p["n"], p["D"], tbe_native.DTYPE_F16, p["T"])
    ws = torch.empty(lay.total_bytes, dtype=torch.uint8, device=DEV)
    go, to, idx, off = dev(p["grad_output"]), dev(p["table_offsets"]), dev(p["indices"]), dev(p["offsets"])
    psw = dev(p["per_sample_weights"]) if weighted else None
    gpsw = torch.empty(p["n"], dtype=torch.float16, device=DEV) if weighted else None
    vp = lambda t: ctypes.c_void_p(t.data_ptr() if t is not None else 0)
    tbe_native.check(tbe_native.load().tbe_backward_exact_adagrad_stochastic(
        vp(go), vp(w), tbe_native.DTYPE_F16, w.shape[0], 0, p["D"], vp(to), p["T"], vp(idx), p["n"], vp(off), p["B"],
        vp(psw), vp(st), 0.05, 0.1, vp(gpsw), seed, offset, vp(ws), ws.numel(),
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    return w.cpu().numpy(), st.cpu().numpy()


@pytest.mark.parametrize("D", [8, 12, 64, 128, 520])
def test_matches_oracle_stream_and_stays_within_one_ulp(oracle, D):
    p = make_problem(40 + D, T=3, E=60, D=D, B=50, L=7, dtype=np.float16, zipf=1.2)
    got, got_state = _run(p, seed=1234, offset=8)
    w_sr = p["weights"].copy()
    st = np.zeros(180, np.float32)
    oracle.backward("adagrad", p["grad_output"], w_sr, p["table_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st,
                    stochastic_rounding=(1234, 8))
    w_rn = p["weights"].copy()
    st2 = np.zeros(180, np.float32)
    oracle.backward("adagrad", p["grad_output"], w_rn, p["table_offsets"], p["indices"], p["offsets"], 0.05, 0.1, st2)
    # the kernel sums a row's gradients in another order than the oracle, so the fp32 value before
    # rounding can differ in its last bits and flip a draw now and then; nearly all elements agree
    agree = (got.view(np.uint16) == w_sr.view(np.uint16)).mean()
    assert agree > 0.995, agree
    # both results are fp16 neighbours of the same fp32 value: at most one spacing apart (the
    # spacing of the larger of the two when they straddle a power of two)
    ulp = np.maximum(np.abs(np.spacing(w_rn)), np.abs(np.spacing(got))).astype(np.float32)
    assert (np.abs(got.astype(np.float32) - w_rn.astype(np.float32)) <= ulp).all()
    np.testing.assert_allclose(got_state, st, rtol=1e-3, atol=1e-12)
    touched = np.zeros(180, bool)
    touched[oracle.linearize(p["table_offsets"], p["indices"], p["offsets"])[0]] = True
    assert got[~touched].tobytes() == p["weights"][~touched].tobytes()
    assert (got[touched] != w_rn[touched]).any()                 # some element did round the other way


def test_reproducible_per_stream_and_unbiased():
    p = make_problem(77, T=1, E=4, D=64, B=2000, L=1, dtype=np.float16, ragged=False)
    p["grad_output"][:] = (np.random.RandomState(0).randn(2000, 1, 64) * 1e-3).astype(np.float16)
    a, _ = _run(p, 5, 0)
    b, _ = _run(p, 5, 0)
    c, _ = _run(p, 5, 4)
    assert a.tobytes() == b.tobytes() and a.tobytes() != c.tobytes()
    # average over many independent streams approaches the exact fp32 result
    draws = np.stack([_run(p, 5, 4 * k)[0].astype(np.float64) for k in range(64)])
    w32 = dev(p["weights"]).float()
    st = torch.zeros(4, device=DEV)
    ext.backward_exact_adagrad(dev(p["grad_output"]).float(), w32, dev(p["table_offsets"]), dev(p["indices"]),
                               dev(p["offsets"]), None, st, 0.05, 0.1, False, 1)
    exact = w32.cpu().numpy().astype(np.float64)
    nearest = exact.astype(np.float16).astype(np.float64)
    ulp = np.abs(np.spacing(exact.astype(np.float16))).astype(np.float64)
    bias_sr = np.abs(draws.mean(0) - exact) / ulp
    bias_rn = np.abs(nearest - exact) / ulp
    assert bias_sr.mean() < 0.08 and bias_sr.mean() < 0.5 * bias_rn.mean()


def test_rounding_rule_matches_the_oracle_bit_for_bit(oracle):
    """tbe_stochastic_round applies the kernels' element rule (random bits added to the fp32 pattern, then
    a conversion toward zero done on bit patterns) to arrays: four million patterns over all exponents with
    random words, the fp16 subnormal range, the largest finite values and the first that overflow."""
    rs = np.random.RandomState(6)
    bits = np.concatenate([
        rs.randint(0, 2 ** 32, size=4_000_000, dtype=np.uint64).astype(np.uint32),
        np.arange(0x33000000, 0x38900000, 211, dtype=np.uint32),
        np.arange(0xb3000000, 0xb8900000, 211, dtype=np.uint32),
        np.arange(0x477fc000, 0x47802000, dtype=np.uint32),
        np.array([0, 0x80000000, 0x7f7fffff, 0xff7fffff, 0x7f800000, 0xff800000, 1, 0x80000001], np.uint32)])
    words = rs.randint(0, 2 ** 32, size=bits.size, dtype=np.uint64).astype(np.uint32)
    words[::7] = 0
    words[3::7] = 0xffffffff
    values = bits.view(np.float32)
    out = torch.empty(bits.size, dtype=torch.int16, device=DEV)
    v, w = dev(values), torch.from_numpy(words.view(np.int32)).to(DEV)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    tbe_native.check(tbe_native.load().tbe_stochastic_round(vp(v), vp(w), vp(out), bits.size,
                                                            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)))
    torch.cuda.synchronize()
    got = out.cpu().numpy().view(np.uint16)
    want = oracle.stochastic_round_many(values, words)
    summed = (bits.astype(np.uint64) + (words >> 19)).astype(np.uint32).view(np.float32)   # what gets converted
    nan = np.isnan(summed)
    assert got[~nan].tobytes() == want[~nan].tobytes()
    assert bool(np.isnan(got[nan].view(np.float16)).all())


def test_module_with_stochastic_rounding_like_the_reference_test(oracle):
    """test_backward_adagrad with stochastic_rounding=True, fp16 (test_table_batched_embeddings.py:
    219-318): state and weights within the reference's own 1e-3 tolerances of the exact update."""
    T, E, D, B, L = 3, 100, 32, 64, 6
    p = make_problem(50, T, E, D, B, L, np.float16, ragged=False)
    cc = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.5,
                                       eps=0.2, fp16=True, stochastic_rounding=True).cuda()
    cc.embedding_weights.data.copy_(dev(p["weights"]))
    torch.manual_seed(3)
    offset_before = torch.cuda.default_generators[0].get_offset()
    cc(dev(p["indices"]), dev(p["offsets"])).backward(dev(p["grad_output"]))
    assert torch.cuda.default_generators[0].get_offset() == offset_before + 4
    w = p["weights"].copy()
    st = np.zeros(T * E, np.float32)
    oracle.backward("adagrad", p["grad_output"], w, p["table_offsets"], p["indices"], p["offsets"], 0.5, 0.2, st)
    np.testing.assert_allclose(cc.optimizer_state.cpu().numpy(), st, rtol=1e-3, atol=1e-3)
    np.testing.assert_allclose(cc.embedding_weights.detach().float().cpu().numpy(), w.astype(np.float32), rtol=1e-3,
                               atol=1e-3)
    # fp32 weights ignore the flag, as stochastic_rounding_vector's generic overload does (tbe.cu:557-562)
    cc32 = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=ops.Optimizer.EXACT_ROWWISE_ADAGRAD, learning_rate=0.5,
                                         eps=0.2, stochastic_rounding=True).cuda()
    cc32.embedding_weights.data.copy_(dev(p["weights"]).float())
    cc32(dev(p["indices"]), dev(p["offsets"])).backward(dev(p["grad_output"]).float())
    w32 = p["weights"].astype(np.float32)
    st32 = np.zeros(T * E, np.float32)
    oracle.backward("adagrad", p["grad_output"].astype(np.float32), w32, p["table_offsets"], p["indices"],
                    p["offsets"], 0.5, 0.2, st32)
    np.testing.assert_allclose(cc32.embedding_weights.detach().cpu().numpy(), w32, rtol=1e-5, atol=1e-7)
