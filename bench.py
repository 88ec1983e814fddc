#!/usr/bin/env python3
"""Benchmark of the ctct_loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

One step = forward + backward of warp_ctct.ctct_loss on one resident batch of
the "typical ASR batch" workload: N=32, frames 150..250, labels 30..60,
V=1024, fp32 joint log-probs already in HBM, padded regions zero-filled.
Prints ONE JSON line: whole-job lattices/s, the roofline of the dominant
kernel (the zero-fill of the dense gradient, timed with HIP events on its
stream inside the timed region) and a CPU baseline (the C oracle with OpenMP, on the host
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
# HBM bytes per launch of zero_fill_vec_kernel from two rocprofv3 --pmc runs
# (profiles/ctct_loss_typical_batch_pmc.md): WRITE_SIZE 1 952 000 KiB x 1.0 +
# FETCH_SIZE 12.8 KiB x 2.0, the factors being what the same counters read for
# a plain 1 GiB -> 1 GiB elementwise kernel (WRITE_SIZE 1 048 576, FETCH_SIZE
# 524 300 KiB).
ZERO_FILL_TRAFFIC_BYTES = 1952000 * 1024 + int(12.8 * 2 * 1024)


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


def cpu_baseline(joint, ys, lx, ly, budget_s=10.0):
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
    while len(times) < 3 or (time.perf_counter() < t_end and len(times) < 500):
        t0 = time.perf_counter()
        C.ctct_loss_dense(host, ys, lx, ly)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    return {"value": N / med, "unit": "lattices/s", "cores": threads, "kind": "port",
            "sample": "the same N=%d batch, %d runs, median %.3f s per batch "
                      "(C oracle, fp32, OpenMP)" % (N, len(times), med)}


OTHER = {
    # name: (kind, N, T, U, V, sigma)
    "c1": ("full", 2, 40, 10, 32, 1.0),
    "c2": ("full", 32, 250, 60, 1024, 1.0),   # only with --graph; the headline line is main()'s
    "c3": ("full", 8, 500, 120, 4096, 2.0),
    "c4": ("simple_norm", 32, 400, 80, 2048, 1.0),
    "c5": ("simple_unnorm", 4, 1500, 300, 8192, 1.0),
    # the typical batch with a half-precision joint (half the bytes at both ends)
    "c2_bf16": ("full", 32, 250, 60, 1024, 1.0),
    "c2_f16": ("full", 32, 250, 60, 1024, 1.0),
    # the typical batch from logits: log_softmax inside the loss (fused), and
    # torch.log_softmax followed by ctct_loss (what a caller of the reference does)
    "c2_logits": ("logits", 32, 250, 60, 1024, 1.0),
    "c2_logits_bf16": ("logits", 32, 250, 60, 1024, 1.0),
    "c2_logits_unfused": ("logits_unfused", 32, 250, 60, 1024, 1.0),
}
IO_DTYPE = {"c2_bf16": "bfloat16", "c2_f16": "float16", "c2_logits_bf16": "bfloat16"}


def other_config(args, torch, warp_ctct):
    """The remaining benchmark configurations: same timing discipline, a
    reduced JSON line (value, ms_per_step, per-operator HIP-event times)."""
    import numpy as np
    kind, N, T, U, V, sigma = OTHER[args.config]
    rng = np.random.default_rng(7)
    gen = torch.Generator(device="cuda").manual_seed(7)
    if args.config == "c1":
        lx = np.full(N, T, np.int32)
        ly = np.full(N, U, np.int32)
    else:
        lo_t = {"c3": 400, "c4": 300, "c5": 1200}.get(args.config, 150)
        lo_u = {"c3": 80, "c4": 50, "c5": 250}.get(args.config, 30)
        lx = rng.integers(lo_t, T + 1, N).astype(np.int32)
        ly = rng.integers(lo_u, U + 1, N).astype(np.int32)
        lx[0], ly[1] = T, U
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 3] = ys[:, 2]
    d_ys, d_lx, d_ly = (torch.as_tensor(a).cuda() for a in (ys, lx, ly))
    live = int(sum(int(a) * (int(b) + 1) for a, b in zip(lx, ly)))
    if kind == "full":
        joint = torch.randn(N, T, U + 1, V, device="cuda", generator=gen).mul_(sigma).log_softmax(-1)
        t_idx = torch.arange(T, device="cuda")[None, :, None, None]
        u_idx = torch.arange(U + 1, device="cuda")[None, None, :, None]
        joint.masked_fill_((t_idx >= d_lx[:, None, None, None]) | (u_idx > d_ly[:, None, None, None]), 0.0)
        io = getattr(torch, IO_DTYPE.get(args.config, "float32"))
        joint = joint.to(io).requires_grad_(True)
        leaves = (joint,)
        alg_bytes = joint.element_size() * (N * T * (U + 1) * V + 3 * live) + 4 * N * (U + 3)

        def loss_fn():
            return warp_ctct.ctct_loss(joint, d_ys, d_lx, d_ly)
    elif kind in ("logits", "logits_unfused"):
        io = getattr(torch, IO_DTYPE.get(args.config, "float32"))
        logits = torch.randn(N, T, U + 1, V, device="cuda", generator=gen).mul_(3.0).to(io)
        logits.requires_grad_(True)
        leaves = (logits,)
        # algorithmic bytes: live rows read twice (forward, backward), gradient written once
        alg_bytes = logits.element_size() * V * (2 * live + N * T * (U + 1))

        if kind == "logits":
            def loss_fn():
                return warp_ctct.ctct_loss_with_logits(logits, d_ys, d_lx, d_ly)
        else:
            def loss_fn():
                return warp_ctct.ctct_loss(logits.log_softmax(-1), d_ys, d_lx, d_ly)
    else:
        f = torch.randn(N, T, V, device="cuda", generator=gen)
        g = torch.randn(N, U + 1, V, device="cuda", generator=gen)
        normalized = kind == "simple_norm"
        if normalized:
            f, g = f.log_softmax(-1), g.log_softmax(-1)
        f.requires_grad_(True)
        g.requires_grad_(True)
        leaves = (f, g)
        alg_bytes = 8 * N * V * (T + U + 1) if normalized else \
            4 * live + 12 * int(sum(int(b) + 1 for b in ly)) + 4 * N * V * (T + U + 1)

        def loss_fn():
            return warp_ctct.ctct_simple_loss(f, g, d_ys, d_lx, d_ly, normalized=normalized)

    events = {}

    def observer(name, fn):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        out = fn()
        e1.record()
        events.setdefault(name, []).append((e0, e1))
        return out

    def step():
        return torch.autograd.grad(loss_fn(), leaves)

    run = step
    if args.graph:
        # the whole step as one HIP graph: one submission per step instead of
        # 4-12 launches and the autograd bookkeeping around them
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = step()
        run = graph.replay
    for _ in range(args.warmup):
        run()
    torch.cuda.synchronize()
    if not args.graph:
        warp_ctct.set_kernel_observer(observer)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    warp_ctct.set_kernel_observer(None)
    ms = elapsed / args.steps * 1e3
    ops = {k: sum(a.elapsed_time(b) for a, b in v) / len(v) * 1e3 for k, v in events.items()}
    print(json.dumps({
        "metric": "lattices/sec (loss+grad)", "value": N * args.steps / elapsed,
        "unit": "lattices/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms, "higher_is_better": True, "dtype": "f32", "data": "synthetic",
        "io_dtype": IO_DTYPE.get(args.config, "float32"), "hip_graph": bool(args.graph),
        "config": {"workload": args.config, "kind": kind, "N": N, "T": T, "U": U, "V": V,
                   "algorithmic_bytes_per_step": alg_bytes,
                   "step_frac_of_hbm_roofline": alg_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                   "max_frames": int(lx.max()), "ns_per_frame_step": ms * 1e6 / int(lx.max())},
        "operator_us": ops}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--config", default="c2", choices=["c1", "c2", "c3", "c4", "c5", "c2_bf16", "c2_f16", "c2_logits",
                             "c2_logits_bf16", "c2_logits_unfused"],
                    help="workload: c2 (default) is the configuration the headline metric is "
                         "quoted on; the others are the remaining benchmark configurations "
                         "and print a reduced line (no cpu_baseline)")
    ap.add_argument("--graph", action="store_true",
                    help="capture one step in a HIP graph and time its replays (reduced line, "
                         "for any --config)")
    ap.add_argument("--calibrate", action="store_true",
                    help="also launch one plain copy kernel of known size (1 GiB read + 1 GiB "
                         "written) so that rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE readings can "
                         "be scaled to bytes")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE GPU (lattices are independent; a multi-GPU "
                 "run would only split the batch) - use --gpus 1")

    import torch
    import warp_ctct

    if args.config != "c2" or args.graph:
        other_config(args, torch, warp_ctct)
        return

    N, T, U, V = 32, 250, 60, 1024
    joint, d_ys, d_lx, d_ly, ys, lx, ly = make_batch(torch, N, T, U, V)
    joint.requires_grad_(True)

    dense_events = []

    def observer(name, fn):
        if name != "dense_zero_fill":
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
    if args.calibrate:
        src = torch.zeros(1 << 28, device="cuda")          # 2^28 floats = 1 GiB
        dst = torch.empty_like(src)
        torch.add(src, 1.0, out=dst)                        # elementwise kernel: 1 GiB in, 1 GiB out
        torch.cuda.synchronize()
        del src, dst
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
        "roofline": {"bound": "hbm", "kernel": "zero_fill_vec_kernel", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": ZERO_FILL_TRAFFIC_BYTES, "avg_launch_us": dense_ms * 1e3,
                     "algorithmic_bytes_per_launch": dense_b},
        "loss": float(loss),
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(joint.detach(), ys, lx, ly)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
