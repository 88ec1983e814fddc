#!/usr/bin/env python3
"""Benchmark of the ctct_loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

One step = forward + backward of warp_ctct.ctct_loss on one resident batch of
the "typical ASR batch" workload: N=32, frames 150..250, labels 30..60,
V=1024, fp32 joint log-probs already in HBM, padded regions zero-filled.
Prints ONE JSON line: whole-job lattices/s, the roofline of the dominant
kernel (the dense gradient write, timed with HIP events on its stream inside
the timed region) and a CPU baseline (the C oracle with OpenMP, on the host
cores, same batch).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "warp-ctct_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X HBM3E, published
# HBM bytes per launch of the dense-gradient kernel from rocprofv3 --pmc
# (WRITE_SIZE + FETCH_SIZE, calibrated on a copy kernel); None until measured.
DENSE_GRAD_TRAFFIC_BYTES = None


def make_batch(torch, N, T, U, V, seed=2024):
    import numpy as np
    rng = np.random.default_rng(seed)
    lx = rng.integers(150 * T // 250, T + 1, N).astype(np.int32)
    ly = rng.integers(U // 2, U + 1, N).astype(np.int32)
    lx[0], ly[1] = T, U
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 3] = ys[:, 2]                       # one adjacent repeat per sample
    g = torch.Generator(device="cuda").manual_seed(seed)
    joint = torch.randn(N, T, U + 1, V, device="cuda", generator=g).log_softmax(-1)
    d_lx = torch.as_tensor(lx).cuda()
    d_ly = torch.as_tensor(ly).cuda()
    t_idx = torch.arange(T, device="cuda")[None, :, None, None]
    u_idx = torch.arange(U + 1, device="cuda")[None, None, :, None]
    joint.masked_fill_((t_idx >= d_lx[:, None, None, None]) | (u_idx > d_ly[:, None, None, None]), 0.0)
    return joint, torch.as_tensor(ys).cuda(), d_lx, d_ly, ys, lx, ly


def algorithmic_bytes(N, T, U, V, lx, ly):
    """Compulsory HBM bytes of one loss+grad step: the dense gradient write,
    the three gathered reads per live cell, labels / lengths / costs."""
    dense = 4 * N * T * (U + 1) * V
    gathered = 12 * int(sum(int(a) * (int(b) + 1) for a, b in zip(lx, ly)))
    small = 4 * N * (U + 3)
    return dense, gathered, small


def cpu_baseline(joint, ys, lx, ly, budget_s=20.0):
    """C oracle (oracle/ctct_oracle.c, fp32, OpenMP over lattices) on the host
    copy of the same batch: gather + lattice + dense gradient."""
    from oracle import c_oracle as C
    threads = max(1, min(16, os.cpu_count() or 1))
    C.set_num_threads(threads)
    host = joint.cpu().numpy()
    N = host.shape[0]
    C.ctct_loss_dense(host, ys, lx, ly)                  # warm-up (page faults, libm)
    times = []
    t_end = time.perf_counter() + budget_s
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 10):
        t0 = time.perf_counter()
        C.ctct_loss_dense(host, ys, lx, ly)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": N / med, "unit": "lattices/s", "cores": threads, "kind": "port",
            "sample": "the same N=%d batch, %d runs, median %.3f s per batch "
                      "(C oracle, fp32, OpenMP)" % (N, len(times), med)}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (lattices are independent; a multi-GPU "
                 "run would only split the batch) - use --gpus 1")

    import torch
    import warp_ctct

    N, T, U, V = 32, 250, 60, 1024
    joint, d_ys, d_lx, d_ly, ys, lx, ly = make_batch(torch, N, T, U, V)
    joint.requires_grad_(True)

    dense_events = []

    def observer(name, fn):
        if name != "dense_grad":
            return fn()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn()
        e1.record()
        dense_events.append((e0, e1))
        return out

    def step():
        loss = warp_ctct.ctct_loss(joint, d_ys, d_lx, d_ly, reduction="mean")
        (grad,) = torch.autograd.grad(loss, joint)
        return loss, grad

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    warp_ctct.set_kernel_observer(observer)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss, grad = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    warp_ctct.set_kernel_observer(None)

    ms_per_step = elapsed / args.steps * 1e3
    value = N * args.steps / elapsed
    dense_ms = sum(a.elapsed_time(b) for a, b in dense_events) / max(1, len(dense_events))
    dense_b, gathered_b, small_b = algorithmic_bytes(N, T, U, V, lx, ly)
    achieved = dense_b / (dense_ms * 1e-3) / 1e9
    result = {
        "metric": "lattices/sec (loss+grad) at N=32,T=250,U=60,V=1024 fp32; % of HBM roofline",
        "value": value,
        "unit": "lattices/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "ctct_loss fwd+bwd, typical ASR batch: N=32, lx in [150,250], "
                               "ly in [30,60], V=1024, fp32 joint resident in HBM",
                   "N": N, "T": T, "U": U, "V": V,
                   "algorithmic_bytes_per_step": dense_b + gathered_b + small_b,
                   "step_frac_of_hbm_roofline":
                       (dense_b + gathered_b + small_b) / (ms_per_step * 1e-3) / 1e9 / HBM_PEAK_GBS},
        "roofline": {"bound": "hbm", "kernel": "dense_grad_kernel", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": DENSE_GRAD_TRAFFIC_BYTES, "avg_launch_us": dense_ms * 1e3,
                     "algorithmic_bytes_per_launch": dense_b},
        "loss": float(loss),
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(joint.detach(), ys, lx, ly)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
