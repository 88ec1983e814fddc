#!/usr/bin/env python3
"""Benchmark of the CTC-Transducer loss hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-configs]

One step = forward + backward of warp_ctct.ctct_loss on one resident batch of
the "typical ASR batch" workload: N=32, frames 150..250, labels 30..60,
V=1024, fp32 joint log-probs already in HBM, padded regions zero-filled.
Prints ONE JSON line: whole-job lattices/s, the roofline of the dominant
kernel (lattice_fill_kernel: the clear of the dense gradient with the lattice
sweeps riding in the same launch, timed with HIP events on its stream inside
the timed region), a CPU baseline (the C oracle with OpenMP, on
the host cores, same batch) and, under "configs", the same measurement for all
five benchmark configurations with the HIP-event duration of every kernel of
a step (the library's own per-kernel timing, warpctct_profile).

    python bench.py --config c4 [--graph]      one configuration alone (reduced line)
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "warp-ctct_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3   # MI355X dense fp32 matrix, published
# HBM bytes per launch of lattice_fill_kernel (the clear of the dense gradient
# with the lattice sweeps in the same launch) from two rocprofv3 --pmc runs
# (profiles/ctct_loss_typical_batch_pmc.md): WRITE_SIZE 1 964 748 KiB x 1.0 +
# FETCH_SIZE 9 710.3 KiB x 2.0, the factors being what the same counters read
# for a plain 1 GiB -> 1 GiB elementwise kernel (WRITE_SIZE 1 048 576,
# FETCH_SIZE 524 300 KiB).
LATTICE_FILL_TRAFFIC_BYTES = 1964748 * 1024 + int(9710.3 * 2 * 1024)


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
    host_cores = os.cpu_count() or 1
    threads = max(1, min(16, host_cores))
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
    return {"value": N / med, "unit": "lattices/s", "cores": threads, "host_cores": host_cores,
            "kind": "port",
            "sample": "the same N=%d batch, %d runs, median %.3f s per batch "
                      "(C oracle, fp32, OpenMP on %d threads; the host reports %d cores)"
                      % (N, len(times), med, threads, host_cores)}


# ---- per-kernel HIP-event timing through the library's own hook ---------------
_LIB = None


def kernel_library():
    global _LIB
    if _LIB is None:
        _LIB = ctypes.CDLL(os.path.join(ROOT, "warp-ctct_amd", "warp_ctct", "libwarpctct_hip.so"))
    return _LIB


def profile_kernels(torch, run, steps):
    """Average duration in microseconds, per step, of every kernel of the
    library that `run` launches (HIP events on the stream of each launch)."""
    lib = kernel_library()
    for _ in range(3):                 # the clocks drop while the GPU idles (CPU baseline leg)
        run()
    torch.cuda.synchronize()
    lib.warpctct_profile(1)
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    lib.warpctct_profile(0)
    name, us = ctypes.c_char_p(), ctypes.c_float()
    total, calls = {}, {}
    for i in range(lib.warpctct_profile_count()):
        if lib.warpctct_profile_read(i, ctypes.byref(name), ctypes.byref(us)) != 0:
            continue
        k = name.value.decode().strip("()")
        total[k] = total.get(k, 0.0) + us.value
        calls[k] = calls.get(k, 0) + 1
    return {k: {"us_per_step": total[k] / steps, "launches_per_step": calls[k] / steps} for k in total}


OTHER = {
    # name: (kind, N, T, U, V, sigma)
    "c1": ("full", 2, 40, 10, 32, 1.0),
    "c2": ("full", 32, 250, 60, 1024, 1.0),
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
    "c2_logits_f16": ("logits", 32, 250, 60, 1024, 1.0),
    "c2_logits_unfused": ("logits_unfused", 32, 250, 60, 1024, 1.0),
    # the typical batch handed over in compact form: costs and the (N,T,U+1,3) unit
    # gradients of ctct_loss_compact, no dense gradient at all
    "c2_compact": ("compact", 32, 250, 60, 1024, 1.0),
}
IO_DTYPE = {"c2_bf16": "bfloat16", "c2_f16": "float16", "c2_logits_bf16": "bfloat16",
            "c2_logits_f16": "float16"}
WORKLOAD = {
    "c1": "ctct_loss fp32, N=2, T=40, U=10, V=32, full lengths (the reference's CPU-sized case)",
    "c2": "ctct_loss fp32, typical ASR batch: N=32, lx in [150,250], ly in [30,60], V=1024",
    "c3": "ctct_loss fp32, large vocabulary / long lattice: N=8, lx in [400,500], ly in [80,120], V=4096, N(0,2) logits",
    "c4": "ctct_simple_loss fp32 normalized (log-add joiner): N=32, lx in [300,400], ly in [50,80], V=2048",
    "c5": "ctct_simple_loss fp32 unnormalized, long-utterance stress: N=4, lx in [1200,1500], ly in [250,300], V=8192",
    "c2_bf16": "ctct_loss on a bfloat16 joint (gradient written in bfloat16), typical ASR batch: N=32, lx in [150,250], ly in [30,60], V=1024",
    "c2_logits": "ctct_loss_with_logits on fp32 logits (log_softmax and its backward inside), typical ASR batch: N=32, lx in [150,250], ly in [30,60], V=1024",
    "c2_logits_bf16": "ctct_loss_with_logits on bfloat16 logits, typical ASR batch: N=32, lx in [150,250], ly in [30,60], V=1024",
    "c2_compact": "ctct_loss_compact on the fp32 joint (costs + unit gradients (N,T,U+1,3), no dense gradient), typical ASR batch: N=32, lx in [150,250], ly in [30,60], V=1024",
}


def build_config(name, torch, warp_ctct):
    """Synthetic inputs of one configuration, resident on the GPU.  Returns
    (step function, facts) where facts holds sizes and algorithmic work."""
    import numpy as np
    kind, N, T, U, V, sigma = OTHER[name]
    rng = np.random.default_rng(7)
    gen = torch.Generator(device="cuda").manual_seed(7)
    if name == "c1":
        lx = np.full(N, T, np.int32)
        ly = np.full(N, U, np.int32)
    else:
        lo_t = {"c3": 400, "c4": 300, "c5": 1200}.get(name, 150)
        lo_u = {"c3": 80, "c4": 50, "c5": 250}.get(name, 30)
        lx = rng.integers(lo_t, T + 1, N).astype(np.int32)
        ly = rng.integers(lo_u, U + 1, N).astype(np.int32)
        lx[0], ly[1] = T, U
    ys = rng.integers(1, V, (N, U)).astype(np.int32)
    ys[:, 3] = ys[:, 2]
    d_ys, d_lx, d_ly = (torch.as_tensor(a).cuda() for a in (ys, lx, ly))
    live = int(sum(int(a) * (int(b) + 1) for a, b in zip(lx, ly)))
    # cells that a complete alignment can pass through: t >= u and lx - t >= ly - u
    band = int(sum(sum(max(0, min(int(b), t) - max(0, int(b) - (int(a) - t)) + 1) for t in range(int(a)))
                   for a, b in zip(lx, ly)))
    facts = {"kind": kind, "N": N, "T": T, "U": U, "V": V, "max_frames": int(lx.max()),
             "live_cells": live, "band_cells": band}
    if kind == "full":
        joint = torch.randn(N, T, U + 1, V, device="cuda", generator=gen).mul_(sigma).log_softmax(-1)
        t_idx = torch.arange(T, device="cuda")[None, :, None, None]
        u_idx = torch.arange(U + 1, device="cuda")[None, None, :, None]
        joint.masked_fill_((t_idx >= d_lx[:, None, None, None]) | (u_idx > d_ly[:, None, None, None]), 0.0)
        io = getattr(torch, IO_DTYPE.get(name, "float32"))
        joint = joint.to(io).requires_grad_(True)
        leaves = (joint,)
        facts["algorithmic_bytes_per_step"] = (joint.element_size() * (N * T * (U + 1) * V + 3 * live)
                                               + 4 * N * (U + 3))
        facts["dense_gradient_bytes"] = joint.element_size() * N * T * (U + 1) * V

        def loss_fn():
            return warp_ctct.ctct_loss(joint, d_ys, d_lx, d_ly)
    elif kind == "compact":
        joint = torch.randn(N, T, U + 1, V, device="cuda", generator=gen).log_softmax(-1)
        # algorithmic bytes: three gathered reads and three unit gradients per cell
        facts["algorithmic_bytes_per_step"] = 12 * live + 12 * N * T * (U + 1) + 4 * N * (U + 3)

        def step():
            return warp_ctct.ctct_loss_compact(joint, d_ys, d_lx, d_ly)

        return step, facts
    elif kind in ("logits", "logits_unfused"):
        io = getattr(torch, IO_DTYPE.get(name, "float32"))
        logits = torch.randn(N, T, U + 1, V, device="cuda", generator=gen).mul_(3.0).to(io)
        logits.requires_grad_(True)
        leaves = (logits,)
        # algorithmic bytes: live rows read twice (forward, backward), gradient written once
        facts["algorithmic_bytes_per_step"] = logits.element_size() * V * (2 * live + N * T * (U + 1))
        # the backward's kernel: rows inside the band read, every row written
        facts["logits_grad_bytes"] = logits.element_size() * V * (band + N * T * (U + 1))

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
        facts["algorithmic_bytes_per_step"] = 8 * N * V * (T + U + 1) if normalized else \
            4 * live + 12 * int(sum(int(b) + 1 for b in ly)) + 4 * N * V * (T + U + 1)
        if normalized:
            # log-add terms of the forward and of each of the two gradients, 2 flop each
            facts["algorithmic_flops_per_step"] = 3 * 2 * N * T * (U + 1) * V

        def loss_fn():
            return warp_ctct.ctct_simple_loss(f, g, d_ys, d_lx, d_ly, normalized=normalized)

    def step():
        return torch.autograd.grad(loss_fn(), leaves)

    return step, facts


def time_steps(torch, run, steps, warmup):
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        run()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def summarise(name, facts, sec_per_step, kernels):
    """The figures of one configuration: step time, throughput, and the
    fraction of the roofline that bounds it."""
    us = {k: round(v["us_per_step"], 2) for k, v in sorted(kernels.items(), key=lambda kv: -kv[1]["us_per_step"])}
    out = {"workload": WORKLOAD.get(name, name), "ms_per_step": sec_per_step * 1e3,
           "value": facts["N"] / sec_per_step, "unit": "lattices/s",
           "kernel_us_per_step": us, "kernel_us_total": round(sum(us.values()), 2)}
    if "algorithmic_bytes_per_step" in facts:
        out["algorithmic_bytes_per_step"] = facts["algorithmic_bytes_per_step"]
        out["step_frac_of_hbm_roofline"] = (facts["algorithmic_bytes_per_step"] / sec_per_step / 1e9
                                            / HBM_PEAK_GBS)
    # (lattice_fill_kernel, the sweeps with the clear of the dense gradient in
    # the same launch, is as long as the clear: no figure per frame from it)
    # (with the sweeps done in the linear domain, lattice_lin_kernel does the
    # work and lattice_kernel, launched behind it as the fall-back, returns at
    # once: the figure per frame is the sweeping kernel's)
    lattice = sum(v for k, v in us.items() if k.startswith("lattice_kernel"))
    lattice_name = "lattice_kernel"
    if us.get("lattice_lin_kernel", 0.0) > lattice:
        lattice, lattice_name = us["lattice_lin_kernel"], "lattice_lin_kernel"
    if lattice > 0:
        out["lattice_kernel_us"] = lattice
        out["lattice_ns_per_frame"] = lattice * 1e3 / facts["max_frames"]
    fill = us.get("lattice_fill_kernel")
    grad_us = sum(v for k, v in us.items() if k.startswith("logits_grad_kernel"))
    if facts["kind"] == "logits" and grad_us > 0:
        gbs = facts["logits_grad_bytes"] / (grad_us * 1e-6) / 1e9
        out["roofline"] = {"bound": "hbm", "kernel": "logits_grad_kernel (rows inside the band of "
                           "complete alignments read, every row of the gradient written)",
                           "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                           "frac": gbs / HBM_PEAK_GBS, "avg_launch_us": grad_us,
                           "algorithmic_bytes_per_launch": facts["logits_grad_bytes"]}
    elif name == "c1" or facts["kind"] in ("simple_unnorm", "compact"):
        out["roofline"] = {"bound": "latency", "kernel": lattice_name,
                           "note": "serial recursion over max_frames dependent steps; reported as "
                                   "ns per frame, an HBM fraction would be structurally low",
                           "max_frames": facts["max_frames"]}
    elif facts["kind"] == "full" and fill:
        gbs = facts["dense_gradient_bytes"] / (fill * 1e-6) / 1e9
        out["roofline"] = {"bound": "hbm", "kernel": "lattice_fill_kernel", "achieved": gbs,
                           "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": gbs / HBM_PEAK_GBS,
                           "avg_launch_us": fill,
                           "algorithmic_bytes_per_launch": facts["dense_gradient_bytes"]}
    elif facts["kind"] == "simple_norm":
        # every kernel of the three products: the forward's partial-sum pass counts too
        gemm = {k: v for k, v in us.items() if k.startswith(("logmm_fwd", "logmm_bwd"))
                and "zero" not in k}
        gemm_us = sum(gemm.values())
        flops = facts["algorithmic_flops_per_step"]
        tf = flops / (gemm_us * 1e-6) / 1e12 if gemm_us > 0 else 0.0
        out["algorithmic_flops_per_step"] = flops
        out["roofline"] = {"bound": "mfma", "kernel": "the three matrix products of the log-matmul "
                           "(forward, gradient wrt f, gradient wrt g; the forward's pass over its "
                           "slabs' partial sums runs inside simple_gather_units_kernel<true>, which it "
                           "lengthens by 4 us, not counted here): "
                           "fp32 operands split on the fly into three bfloat16 planes, six bf16 "
                           "matrix instructions per fp32 product, priced against the fp32 peak",
                           "achieved": tf, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                           "frac": tf / MFMA_FP32_PEAK_TFLOPS, "avg_launch_us": gemm,
                           "algorithmic_flops_per_launch": flops // 3}
        out["step_frac_of_mfma_roofline"] = flops / sec_per_step / 1e12 / MFMA_FP32_PEAK_TFLOPS
    return out


def measure_config(name, torch, warp_ctct, steps, warmup=3, profile_steps=3):
    step, facts = build_config(name, torch, warp_ctct)
    sec = time_steps(torch, step, steps, warmup)
    kernels = profile_kernels(torch, step, profile_steps)
    out = summarise(name, facts, sec, kernels)
    out["steps"] = steps
    del step
    torch.cuda.empty_cache()
    return out


def other_config(args, torch, warp_ctct):
    """One configuration alone: same timing discipline, a reduced JSON line."""
    kind, N, T, U, V, sigma = OTHER[args.config]
    step, facts = build_config(args.config, torch, warp_ctct)
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
            captured = step()   # noqa: F841  (keeps the captured outputs alive)
        run = graph.replay
    sec = time_steps(torch, run, args.steps, args.warmup)
    kernels = {} if args.graph else profile_kernels(torch, step, 3)
    out = summarise(args.config, facts, sec, kernels)
    print(json.dumps({
        "metric": "lattices/sec (loss+grad)", "value": out["value"],
        "unit": "lattices/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": out["ms_per_step"], "higher_is_better": True, "dtype": "f32",
        "data": "synthetic", "io_dtype": IO_DTYPE.get(args.config, "float32"),
        "hip_graph": bool(args.graph),
        "config": dict(out, workload=args.config, kind=kind, N=N, T=T, U=U, V=V)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the per-configuration figures under \"configs\"")
    ap.add_argument("--config", default="c2", choices=sorted(OTHER),
                    help="workload: c2 (default) is the configuration the headline metric is "
                         "quoted on; any other prints a reduced line for that one alone")
    ap.add_argument("--graph", action="store_true",
                    help="capture one step in a HIP graph and time its replays (reduced line, "
                         "for any --config)")
    ap.add_argument("--joiner-sweeps", choices=["default", "log", "linear"], default="default",
                    help="domain of the log-add joiner's lattice sweeps (ctct_simple_loss): the "
                         "library's choice by the number of frames, the log domain only, or the "
                         "linear domain, checked, with the log domain as fall-back, for every input")
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

    if args.joiner_sweeps != "default":
        warp_ctct.joiner_linear_lattice({"log": 0, "linear": 1}[args.joiner_sweeps])
    if args.config != "c2" or args.graph:
        other_config(args, torch, warp_ctct)
        return

    N, T, U, V = 32, 250, 60, 1024
    joint, d_ys, d_lx, d_ly, ys, lx, ly = make_batch(torch, N, T, U, V)
    joint.requires_grad_(True)

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
    # The dominant kernel (the clear of the dense gradient, with the lattice
    # sweeps riding in the same launch) is bracketed with HIP events on its own
    # stream inside the timed region, through the library's timing hook.
    lib = kernel_library()
    lib.warpctct_profile_filter(b"lattice_fill")
    lib.warpctct_profile(1)
    t0 = time.perf_counter()
    for _ in range(args.steps):
        loss, grad = step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    lib.warpctct_profile(0)
    lib.warpctct_profile_filter(None)
    name, us = ctypes.c_char_p(), ctypes.c_float()
    fills = []
    for i in range(lib.warpctct_profile_count()):
        if lib.warpctct_profile_read(i, ctypes.byref(name), ctypes.byref(us)) == 0:
            fills.append(us.value)
    if len(fills) != min(args.steps, 8192):             # the hook keeps 8192 records
        sys.exit("bench.py: expected one clearing launch per step, the timing hook saw %d in %d steps"
                 % (len(fills), args.steps))

    ms_per_step = elapsed / args.steps * 1e3
    value = N * args.steps / elapsed
    dense_ms = sum(fills) / len(fills) * 1e-3
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
        "roofline": {"bound": "hbm", "kernel": "lattice_fill_kernel", "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "traffic": LATTICE_FILL_TRAFFIC_BYTES, "avg_launch_us": dense_ms * 1e3,
                     "algorithmic_bytes_per_launch": dense_b},
        "loss": float(loss),
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(joint.detach(), ys, lx, ly)
    if not args.no_configs:
        # every kernel of a headline step, then the other four configurations
        kernels = profile_kernels(torch, step, 3)
        configs = {"c2": {"workload": WORKLOAD["c2"], "ms_per_step": ms_per_step,
                          "kernel_us_per_step": {k: round(v["us_per_step"], 2) for k, v in sorted(
                              kernels.items(), key=lambda kv: -kv[1]["us_per_step"])}}}
        for name, steps in (("c1", 50), ("c3", 8), ("c4", 20), ("c5", 20), ("c2_bf16", 20),
                            ("c2_logits", 10), ("c2_logits_bf16", 10), ("c2_compact", 30)):
            # (this batch's tensors go before the next configuration's are made: c3 alone holds 16 GB)
            if name == "c1":
                del joint, loss, grad, step
                torch.cuda.empty_cache()
            configs[name] = measure_config(name, torch, warp_ctct, steps)
        result["configs"] = configs
    print(json.dumps(result))


if __name__ == "__main__":
    main()
