"""The reference test-suite's CPU path, restated with torch library routines only.

TEST INFRASTRUCTURE: used by bench.py's cpu_baseline leg (and nothing in the shipped
package).  Per table one torch.nn.EmbeddingBag(E, D, mode="sum", sparse=True) on the CPU,
forward, backward with the output gradient, then the Python-side optimizer exactly as
test_table_batched_embeddings.py writes it: SGD `weight - weight.grad * lr` (:184-193),
row-wise Adagrad `state += grad.to_dense().pow(2).sum(1)`,
`addcdiv(weight, grad.to_dense(), sqrt(state) + eps, value=-lr)` (:296-318).
"""
import time

import numpy as np
import torch


class CpuTables:
    def __init__(self, weights, rows, D, fill=None):
        """weights: float32 numpy [sum(rows), D]; or None, then every table is filled with the
        constant `fill` (timing runs on tables too large to draw and copy: values do not change
        the work)."""
        self.bags = []
        self.states = []
        r0 = 0
        for E in rows:
            if weights is None:
                init = torch.full((E, D), float(fill))
            else:
                init = torch.from_numpy(np.ascontiguousarray(weights[r0:r0 + E])).float()
            bag = torch.nn.EmbeddingBag(E, D, mode="sum", sparse=True, _weight=init)
            self.bags.append(bag)
            self.states.append(torch.zeros(E))
            r0 += E

    def step(self, indices, offsets, B, grad_output, optimizer, lr, eps=0.0, per_sample_weights=None,
             update="dense"):
        """One forward + backward + optimizer pass over all tables; returns output [B, T, D].
        update="dense" is the optimizer as the reference's test writes it (it touches every row of
        every table); update="index_add" applies the same SGD step to the rows of the coalesced
        sparse gradient only."""
        outs = []
        for t, bag in enumerate(self.bags):
            lo, hi = int(offsets[t * B]), int(offsets[(t + 1) * B])
            idx = torch.from_numpy(indices[lo:hi].astype(np.int64))
            off = torch.from_numpy((offsets[t * B:(t + 1) * B] - lo).astype(np.int64))
            kwargs = {}
            if per_sample_weights is not None:
                kwargs["per_sample_weights"] = torch.from_numpy(per_sample_weights[lo:hi]).float()
            bag.weight.grad = None
            out = bag(idx, off, **kwargs)
            out.backward(torch.from_numpy(np.ascontiguousarray(grad_output[:, t, :])).float())
            grad = bag.weight.grad
            with torch.no_grad():
                if optimizer == "sgd" and update == "index_add":
                    g = grad.coalesce()
                    bag.weight.data.index_add_(0, g.indices()[0], g.values(), alpha=-lr)
                elif optimizer == "sgd":
                    bag.weight.data = bag.weight - grad * lr
                else:
                    assert update == "dense"
                    dense = grad.to_dense()
                    self.states[t] += dense.pow(2).sum(dim=1)
                    bag.weight.data = torch.addcdiv(bag.weight, dense, (self.states[t].sqrt() + eps).view(-1, 1),
                                                    value=-lr)
            outs.append(out.detach())
        return torch.stack(outs, dim=1)


def time_steps(tables, step_args, warmup=1, iters=3, update="dense", seconds=None):
    """Seconds per step.  With `seconds`, at least `iters` steps and as many more as that much time
    allows (judged by the first timed steps); returns (seconds per step, steps timed)."""
    for _ in range(warmup):
        tables.step(*step_args, update=update)
    t0 = time.perf_counter()
    for _ in range(iters):
        tables.step(*step_args, update=update)
    done = iters
    if seconds is not None:
        more = int((seconds - (time.perf_counter() - t0)) / ((time.perf_counter() - t0) / iters))
        for _ in range(max(more, 0)):
            tables.step(*step_args, update=update)
        done += max(more, 0)
        return (time.perf_counter() - t0) / done, done
    return (time.perf_counter() - t0) / done
