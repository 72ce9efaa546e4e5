"""Writes tests/golden/*.npz: inputs and expected outputs of the table-batched
embedding-bag path, computed with the reference test-suite's own oracle --
per-table torch.nn.EmbeddingBag(mode="sum", sparse=True) on the CPU plus the
Python-side optimizer (test_table_batched_embeddings.py:127-160, 184-193, 296-318).
No reference code is imported or run; only torch library routines.

    python tests/golden/make_golden.py
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def draw(seed, T, E, D, B, L, dtype, ragged=False, weighted=False, dup_heavy=False):
    rs = np.random.RandomState(seed)
    if ragged:
        lengths = rs.randint(0, L + 1, size=(T, B))
    else:
        lengths = np.full((T, B), L)
    n = int(lengths.sum())
    offsets = np.concatenate([[0], np.cumsum(lengths.reshape(-1))]).astype(np.int32)
    if dup_heavy:
        indices = (rs.zipf(1.2, size=n) % E).astype(np.int32)
    else:
        indices = rs.randint(0, E, size=n).astype(np.int32)
    weights = rs.uniform(-0.01, 0.01, size=(T * E, D)).astype(dtype)
    grad_output = rs.randn(B, T, D).astype(dtype)
    psw = rs.uniform(0, 1, size=n).astype(dtype) if weighted else None
    return lengths, offsets, indices, weights, grad_output, psw


def torch_reference(T, E, D, B, lengths, offsets, indices, weights, grad_output, psw, optimizer, lr, eps):
    """Per-table EmbeddingBag forward/backward and the Python optimizer, in float32 math
    for float16 inputs (the CPU EmbeddingBag has no half kernels), rounded once at the end."""
    math_dtype = torch.float64 if weights.dtype == np.float64 else torch.float32
    out = np.zeros((B, T, D), dtype=np.float64)
    new_weights = np.zeros((T * E, D), dtype=np.float64)
    new_state = np.zeros(T * E, dtype=np.float64)
    grad_psw = np.zeros(indices.size, dtype=np.float64) if psw is not None else None
    for t in range(T):
        bag = torch.nn.EmbeddingBag(E, D, mode="sum", sparse=True).to(math_dtype)
        bag.weight.data.copy_(torch.from_numpy(weights[t * E:(t + 1) * E].astype(np.float64)).to(math_dtype))
        lo, hi = offsets[t * B], offsets[(t + 1) * B]
        idx_t = torch.from_numpy(indices[lo:hi].astype(np.int64))
        off_t = torch.from_numpy((offsets[t * B:(t + 1) * B] - lo).astype(np.int64))
        kwargs = {}
        if psw is not None:
            w_t = torch.from_numpy(psw[lo:hi].astype(np.float64)).to(math_dtype).requires_grad_(True)
            kwargs["per_sample_weights"] = w_t
        y = bag(idx_t, off_t, **kwargs)
        out[:, t, :] = y.detach().double().numpy()
        go_t = torch.from_numpy(grad_output[:, t, :].astype(np.float64)).to(math_dtype)
        y.backward(go_t)
        grad = bag.weight.grad.to_dense()
        if psw is not None:
            grad_psw[lo:hi] = w_t.grad.double().numpy()
        if optimizer == "sgd":
            new_w = bag.weight.detach() - grad * lr  # test_table_batched_embeddings.py:193
        else:
            state = grad.pow(2).sum(dim=1)  # :299, starting from a zero state
            new_state[t * E:(t + 1) * E] = state.double().numpy()
            new_w = torch.addcdiv(bag.weight.detach(), grad, (state.sqrt() + eps).view(E, 1), value=-lr)  # :307-315
        new_weights[t * E:(t + 1) * E] = new_w.double().numpy()
    return out, new_weights, new_state, grad_psw


CASES = {
    # the smallest benchmark configuration: tiny TBE, T=2, E=1000, D=32 fp32, B=64, L=4, uniform indices, SGD lr=0.1, seed 0
    "cfg1_sgd_f32": dict(seed=0, T=2, E=1000, D=32, B=64, L=4, dtype=np.float32, optimizer="sgd", lr=0.1, eps=0.0),
    "ragged_adagrad_f32": dict(seed=1, T=3, E=50, D=16, B=40, L=9, dtype=np.float32, ragged=True, dup_heavy=True,
                               optimizer="adagrad", lr=0.5, eps=0.2),
    "weighted_adagrad_f32": dict(seed=2, T=2, E=60, D=64, B=33, L=12, dtype=np.float32, ragged=True, weighted=True,
                                 dup_heavy=True, optimizer="adagrad", lr=0.01, eps=1e-8),
    "weighted_adagrad_f16": dict(seed=3, T=2, E=100, D=64, B=32, L=10, dtype=np.float16, ragged=True, weighted=True,
                                 dup_heavy=True, optimizer="adagrad", lr=0.01, eps=1e-8),
    "sgd_f64": dict(seed=4, T=2, E=30, D=8, B=16, L=6, dtype=np.float64, dup_heavy=True, optimizer="sgd", lr=0.05,
                    eps=0.0),
    "hot_row_sgd_f32": dict(seed=5, T=1, E=4, D=128, B=300, L=5, dtype=np.float32, optimizer="sgd", lr=0.01, eps=0.0),
}


def main():
    torch.manual_seed(0)
    torch.set_num_threads(1)
    for name, c in CASES.items():
        c = dict(c)
        opt, lr, eps = c.pop("optimizer"), c.pop("lr"), c.pop("eps")
        T, E, D, B = c["T"], c["E"], c["D"], c["B"]
        lengths, offsets, indices, weights, go, psw = draw(**c)
        out, new_w, new_state, grad_psw = torch_reference(T, E, D, B, lengths, offsets, indices, weights, go, psw,
                                                          opt, lr, eps)
        arrays = dict(T=T, E=E, D=D, B=B, lr=lr, eps=eps, optimizer=opt, offsets=offsets, indices=indices,
                      weights=weights, grad_output=go, expected_output=out, expected_weights=new_w,
                      expected_state=new_state)
        if psw is not None:
            arrays["per_sample_weights"] = psw
            arrays["expected_grad_psw"] = grad_psw
        np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)
        print(name, "N=%d" % indices.size, "%.1f KB" % (os.path.getsize(os.path.join(HERE, name + ".npz")) / 1e3))


if __name__ == "__main__":
    main()
