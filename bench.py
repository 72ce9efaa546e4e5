"""Headline benchmark: table-batched embedding bags, forward + fused exact-SGD backward.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2|3|4] [--no-cpu]

One step = one pass of the hot path over one batch of seeded synthetic input: the
module's forward (pooled gather-sum) and its backward (linearize, radix sort, segments,
fused update) through autograd, as the reference's tests drive it
(test_table_batched_embeddings.py:197-212).  Inputs are resident in HBM before the timed
region.  Prints ONE JSON line.  Everything runs on one GPU.

Default workload = BASELINE config 3 (the shape the target is quoted on):
T=64 tables x 100k rows x D=128 fp32, B=4096 bags per table, L=20, Zipf(1.05) indices,
exact SGD lr=0.01.  --config 2 times the forward alone on uniform indices; --config 4 the
fp16 / weighted / exact row-wise Adagrad shape.
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
for _p in (ROOT, os.path.join(ROOT, "sparse-ads-baselines_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK = 8.0e12  # bytes/s, MI355X

# Bytes that crossed the L2 <-> memory-fabric boundary per launch, from two rocprofv3 --pmc runs of
# this script (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter
# reads for a plain 1 GiB device copy (FETCH_SIZE x2.0, WRITE_SIZE x1.0).  Keyed by (kernel, config).
MEASURED_TRAFFIC = {
    ("update_short", 3): int((1901850.8 * 2.0 + 1283608.9) * 1024),
    ("forward", 3): int((836316.6 * 2.0 + 131072.0) * 1024),
}


def make_workload(config, seed=0):
    rs = np.random.RandomState(seed)
    if config in (2, 3):
        T, E, D, B, L = 64, 100000, 128, 4096, 20
        lengths = np.full(T * B, L, dtype=np.int64)
        n = T * B * L
        if config == 2:
            indices = rs.randint(0, E, size=n)
            name = "cfg2 forward only: T=64 E=100k D=128 fp32 B=4096 L=20 uniform"
        else:
            indices = rs.zipf(1.05, size=n) % E
            name = "cfg3 fwd + exact SGD: T=64 E=100k D=128 fp32 B=4096 L=20 Zipf(1.05) lr=0.01"
        w = dict(T=T, E=E, D=D, B=B, fp16=False, weighted=False, optimizer="sgd" if config == 3 else None,
                 lr=0.01, eps=0.0)
    elif config == 4:
        T, E, D, B = 32, 1000000, 64, 8192
        lengths = rs.randint(0, 41, size=T * B).astype(np.int64)
        n = int(lengths.sum())
        indices = rs.zipf(1.2, size=n) % E
        name = ("cfg4 fwd + weighted exact row-wise Adagrad: T=32 E=1M D=64 fp16 B=8192 L~U[0,40] Zipf(1.2) "
                "lr=0.01 eps=1e-8")
        w = dict(T=T, E=E, D=D, B=B, fp16=True, weighted=True, optimizer="adagrad", lr=0.01, eps=1e-8)
    else:
        raise SystemExit("bench.py: --config must be 2, 3 or 4")
    w["name"] = name
    w["indices"] = indices.astype(np.int32)
    w["offsets"] = np.concatenate([[0], np.cumsum(lengths)]).astype(np.int32)
    w["n"] = n
    w["seed"] = seed
    return w


def algorithmic_bytes(w, U):
    """Bytes the path must move per step (weights element S, N lookups, BT bags, U unique rows):
    A_fwd = N*D*S + 4N + 4(BT+1) + BT*D*S (+ N*S weighted)
    A_bwd = N*D*S + 2*U*D*S + 4N + 4(BT+1) (+ 8U Adagrad state) (+ 2*N*S weighted)"""
    S = 2 if w["fp16"] else 4
    N, BT, D = w["n"], w["T"] * w["B"], w["D"]
    a_fwd = N * D * S + 4 * N + 4 * (BT + 1) + BT * D * S + (N * S if w["weighted"] else 0)
    a_bwd = 0
    a_update = 0
    if w["optimizer"]:
        a_update = N * D * S + 2 * U * D * S
        if w["optimizer"] == "adagrad":
            a_update += 8 * U
        if w["weighted"]:
            a_update += 2 * N * S
        a_bwd = a_update + 4 * N + 4 * (BT + 1)
    return a_fwd, a_bwd, a_update


def cpu_baseline(w, torch, tables=8, iters=3):
    """The reference's CPU path (per-table torch.nn.EmbeddingBag + Python optimizer) on a bounded
    sample: the first `tables` tables of the same workload, all host cores."""
    from oracle import torch_cpu_path

    T = min(tables, w["T"])
    E, D, B = w["E"], w["D"], w["B"]
    rs = np.random.RandomState(w["seed"] + 1)
    hi = int(w["offsets"][T * B])
    weights = rs.uniform(-0.01, 0.01, size=(T * E, D)).astype(np.float32)
    go = rs.randn(B, T, D).astype(np.float32)
    psw = rs.uniform(0, 1, size=hi).astype(np.float32) if w["weighted"] else None
    torch.set_num_threads(os.cpu_count() or 1)
    cpu = torch_cpu_path.CpuTables(weights, [E] * T, D)
    opt = w["optimizer"] or "sgd"
    sec = torch_cpu_path.time_steps(cpu, (w["indices"][:hi], w["offsets"][:T * B + 1], B, go, opt, w["lr"],
                                          w["eps"], psw), warmup=1, iters=iters)
    return {"value": T * B / sec, "unit": "bags/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": "first %d of %d tables of the same workload (%d bags/step), 1 warm-up + %d timed steps, "
                      "per-table torch.nn.EmbeddingBag(sparse=True) forward+backward + Python %s update, fp32"
                      % (T, w["T"], T * B, iters, opt),
            "ms_per_step": sec * 1e3}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--config", type=int, default=3)
    ap.add_argument("--profile-steps", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 1 GiB device-to-device copy 5 times, as the known-size "
                         "reference for rocprofv3 FETCH_SIZE / WRITE_SIZE counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU; --gpus %d is not supported (run with --gpus 1)" % args.gpus,
              file=sys.stderr)
        sys.exit(2)

    import torch

    import table_batched_embeddings as ext
    import table_batched_embeddings_ops as ops
    import tbe_native

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    w = make_workload(args.config)
    T, E, D, B = w["T"], w["E"], w["D"], w["B"]
    optimizer = {"sgd": ops.Optimizer.SGD, "adagrad": ops.Optimizer.EXACT_ROWWISE_ADAGRAD,
                 None: ops.Optimizer.SGD}[w["optimizer"]]
    module = ops.TableBatchedEmbeddingBags(T, E, D, optimizer=optimizer, learning_rate=w["lr"], eps=w["eps"],
                                           fp16=w["fp16"]).cuda()
    gen = torch.Generator(device=dev).manual_seed(w["seed"])
    module.embedding_weights.data.uniform_(-0.01, 0.01, generator=gen)
    dtype = module.embedding_weights.dtype
    indices = torch.from_numpy(w["indices"]).to(dev)
    offsets = torch.from_numpy(w["offsets"]).to(dev)
    grad_output = torch.randn(B, T, D, device=dev, generator=gen).to(dtype)
    psw = None
    if w["weighted"]:
        psw = torch.rand(w["n"], device=dev, generator=gen).to(dtype).requires_grad_(True)

    if w["optimizer"]:
        def step():
            module(indices, offsets, psw).backward(grad_output)
    else:
        def step():
            with torch.no_grad():
                ext.forward(module.embedding_weights.data, module.table_offsets, indices, offsets, None, 200, 1,
                            False)

    if args.calibrate_copy:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    bags = T * B

    # unique rows of the batch, for the byte count (read back from the backward workspace)
    U = 0
    if w["optimizer"]:
        lay = tbe_native.backward_workspace_layout(w["n"], D, tbe_native.DTYPE_F16 if w["fp16"] else
                                                   tbe_native.DTYPE_F32)
        ws = ext.backward_workspace(dev)
        U = int(ws[lay.num_unique:lay.num_unique + 4].view(torch.int32)[0])
    a_fwd, a_bwd, a_update = algorithmic_bytes(w, U)

    # per-kernel durations from HIP events recorded by the library on the launch stream
    per_kernel = {}
    if args.profile_steps > 0:
        with tbe_native.profile() as prof:
            for _ in range(args.profile_steps):
                step()
        for name, ms in prof.launches:
            per_kernel.setdefault(name, []).append(ms)
    kernels = {k: {"launches_per_step": len(v) / max(args.profile_steps, 1), "avg_us": 1e3 * sum(v) / len(v)}
               for k, v in per_kernel.items()}
    kernel_bytes = {"forward": a_fwd, "update_short": a_update}
    roofline = None
    if kernels:
        dominant = max((k for k in kernels if k in kernel_bytes and kernel_bytes[k]),
                       key=lambda k: kernels[k]["avg_us"] * kernels[k]["launches_per_step"])
        achieved = kernel_bytes[dominant] / (kernels[dominant]["avg_us"] * 1e-6) / 1e9
        roofline = {"bound": "hbm", "kernel": dominant, "achieved": achieved, "peak": HBM_PEAK / 1e9,
                    "unit": "GB/s", "frac": achieved / (HBM_PEAK / 1e9),
                    "traffic": MEASURED_TRAFFIC.get((dominant, args.config)),
                    "algorithmic_bytes_per_launch": kernel_bytes[dominant],
                    "avg_launch_us": kernels[dominant]["avg_us"]}

    result = {
        "metric": "tbe_fwd_bwd_bags_per_sec" if w["optimizer"] else "tbe_fwd_bags_per_sec",
        "value": bags / (elapsed / args.steps),
        "unit": "bags/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16" if w["fp16"] else "f32",
        "data": "synthetic",
        "config": {"workload": w["name"], "T": T, "rows_per_table": E, "D": D, "B": B, "lookups": w["n"],
                   "unique_rows": U, "seed": w["seed"]},
        "effective_GBps": (a_fwd + a_bwd) / (elapsed / args.steps) / 1e9,
        "effective_frac_of_hbm_peak": (a_fwd + a_bwd) / (elapsed / args.steps) / HBM_PEAK,
        "algorithmic_bytes": {"forward": a_fwd, "backward": a_bwd},
        "roofline": roofline,
        "kernels": kernels,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(w, torch)
    else:
        result["cpu_baseline"] = None
    print(json.dumps(result))


if __name__ == "__main__":
    main()
