#!/usr/bin/env python3
"""Benchmark of the neural-field hot paths on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

The headline workload is BASELINE.json ``configs[1]``: multiresolution hash encoding,
forward + backward, N = 2^20 points, L = 16, F = 2, T = 2^19, fp16 tables, fp16 upstream
gradient, float32 table gradient.  One step = forward launch + clearing the float32
gradient table + backward launch(es), inputs resident in HBM.  ``value`` is Mpoints/s.

Extra objects in the same line:
  roofline      the dominant kernel of the step (the forward gather kernel: the backward is a
                chain of five shorter kernels), algorithmic bytes per launch / launch time measured
                here with events against the 8 TB/s HBM peak; ``traffic`` is that kernel's HBM
                traffic from the FETCH_SIZE / WRITE_SIZE counters of a profiler run;
  cpu_baseline  the CPU oracle (a port of the reference's PyTorch path) timed on this host
                on a 65536-point sample of the same workload;
  workloads     the other BASELINE configs (fused MLP, reversible MLP, end-to-end step) with
                their own throughput and MFMA roofline fraction.
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16

# geometry of BASELINE configs[1] ("base 16, growth 1.5, L=16" == min_res 16, max_res 7006)
T, L, F, D, MIN_RES, MAX_RES = 2**19, 16, 2, 3, 16, 7006
N_POINTS = 2**20
# algorithmic bytes per point: fwd = 4D + L*2^D*F*2 + L*F*2 ; bwd = 4D + L*F*2 + L*2^D*F*4
FWD_BYTES_PER_POINT = 4 * D + L * 8 * F * 2 + L * F * 2  # 588
BWD_BYTES_PER_POINT = 4 * D + L * F * 2 + L * 8 * F * 4  # 1100
# HBM bytes per forward launch at N = 2^20 measured with rocprofv3 --pmc FETCH_SIZE (x2.0, the factor a 256 MiB copy
# kernel gives for that counter) + WRITE_SIZE (x1.0): 842 MB + 67 MB
FWD_TRAFFIC_BYTES = 9.10e8


def event_times(fn, reps):
    """Per-call GPU duration (ms) of ``fn`` measured with events on the current stream."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return [a.elapsed_time(b) for a, b in evs]


def wall_time(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3  # ms per step


def graph_time(fn, steps, warmup, check):
    """ms per replay of ``fn`` captured into one HIP graph (the host then issues one launch per step instead of six).
    ``check()`` returns tensors written by ``fn``; every one of three spaced replays must reproduce the eager values."""
    try:
        fn()
        torch.cuda.synchronize()
        want = [t.clone() for t in check()]
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):
                fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            fn()
        for _ in range(3):
            g.replay()
            torch.cuda.synchronize()
            got = check()
            if not all(torch.equal(a, b) for a, b in zip(got, want)):
                # dW sums are float atomics: their order may differ between runs; allow rounding-level differences
                if not all(torch.allclose(a.float(), b.float(), rtol=2e-2, atol=1e-2 * float(b.float().abs().max())) for a, b in zip(got, want)):
                    return None
        return wall_time(g.replay, steps, warmup)
    except Exception as e:  # capture is an extra, never the headline
        print(f"bench: HIP graph capture skipped: {e!r}", file=sys.stderr)
        return None


def bench_hash(steps, warmup):
    from triton_helpers_amd.layers.hash_encoding import kernel as hk
    from triton_helpers_amd.layers.hash_encoding.helpers import total_rows

    dev = torch.device("cuda", 0)
    E = total_rows(T, L, D, MIN_RES, MAX_RES)
    torch.manual_seed(0)
    x = torch.rand(N_POINTS, D).to(dev)
    table = ((torch.rand(E, F) * 2 - 1) * 1e-4).half().to(dev)
    do = torch.randn(N_POINTS, L * F).half().to(dev)
    grad = torch.zeros(E, F, dtype=torch.float32, device=dev)
    pi = torch.tensor([hk.PI_1, hk.PI_2, hk.PI_3], dtype=torch.int64, device=dev)

    def fwd():
        with torch.no_grad():
            return hk.hash_encoding(x, table, None, pi, T, MIN_RES, MAX_RES, L)

    def zero():
        grad.zero_()

    def bwd():
        hk.hash_encoding_table_grad(x, do, E, F, pi, T, MIN_RES, MAX_RES, L, out=grad)

    def step():
        fwd()
        zero()
        bwd()

    ms = wall_time(step, steps, warmup)
    reps = max(10, min(steps, 50))
    t_fwd = statistics.mean(event_times(fwd, reps))
    t_zero = statistics.mean(event_times(zero, reps))
    t_bwd = statistics.mean(event_times(bwd, reps))

    # the same step through autograd (table grad rounded to fp16 by the engine), for information
    e = table.clone().requires_grad_(True)

    def step_autograd():
        e.grad = None
        hk.hash_encoding(x, e, None, pi, T, MIN_RES, MAX_RES, L).backward(do)

    ms_autograd = wall_time(step_autograd, max(5, steps // 5), 3)
    return dict(ms=ms, t_fwd=t_fwd, t_zero=t_zero, t_bwd=t_bwd, ms_autograd=ms_autograd, E=E)


def cpu_baseline_hash():
    """CPU oracle (port of the reference's PyTorch path) on a 65536-point sample of the workload."""
    from oracle import hash_encoding as O

    n = 65536
    threads = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(threads)
    torch.manual_seed(0)
    E = O.level_row_offsets(L, T, D, MIN_RES, MAX_RES)[-1]
    x = torch.rand(n, D)
    table = ((torch.rand(E, F) * 2 - 1) * 1e-4).half()
    do = torch.randn(n, L * F).half()

    def run():
        O.encode_forward(x, table, None, T, L, MIN_RES, MAX_RES)
        O.encode_backward(x, do, E, F, None, T, L, MIN_RES, MAX_RES)

    run()
    times = []
    t_start = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < 10 and len(times) < 20):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    med = statistics.median(times)
    return {
        "value": n / med / 1e6,
        "unit": "Mpoints/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": f"fwd+bwd of {n} points, same geometry (L=16,F=2,T=2^19), fp16 table, fp32 grad; median of {len(times)} runs",
    }


def bench_mlp(steps, warmup, d_out=16, rows=2**20):
    from triton_helpers_amd.layers.fully_fused_mlp import kernel as mk

    dev = torch.device("cuda", 0)
    torch.manual_seed(0)

    def u(shape, fan_in):
        return ((torch.rand(*shape) * 2 - 1) / fan_in**0.5).bfloat16().to(dev).requires_grad_(True)

    w_in, w_hid, w_out = u((64, 32), 32), u((64, 64), 64), u((d_out, 64), 64)
    x = torch.randn(1, rows, 32).bfloat16().to(dev).requires_grad_(True)
    dy = torch.randn(1, rows, d_out).bfloat16().to(dev)

    def step():
        x.grad = w_in.grad = w_hid.grad = w_out.grad = None
        mk.fully_fused_mlp(x, w_in, None, w_out, None, w_hid, None, "relu").backward(dy)

    # By default the autograd engine runs the backward on a device thread of its own: two hand-overs between host
    # threads per step, which on some runs of this process cost more than the kernels (160 us against 110 us per
    # step).  torch.autograd.set_multithreading_enabled(False) runs it on the calling thread; both are reported.
    with torch.autograd.set_multithreading_enabled(True):
        ms_engine_thread = wall_time(step, steps, warmup)
    with torch.autograd.set_multithreading_enabled(False):
        ms = wall_time(step, steps, warmup)
    flop_row = 3 * 2 * (32 * 64 + 64 * 64 + 64 * d_out)
    tflops = rows * flop_row / (ms * 1e-3) / 1e12
    out = {
        "workload": f"fused MLP 32->64->64->{d_out} ReLU bf16 fwd+bwd, {rows} rows (through autograd)",
        "value": rows / ms / 1e3, "unit": "Mrows/s", "ms_per_step": ms,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None},
        "hbm_GBs": rows * 256 / (ms * 1e-3) / 1e9,
        "autograd": "backward on the calling thread (torch.autograd.set_multithreading_enabled(False))",
        "ms_per_step_engine_thread": ms_engine_thread,
    }
    # the same autograd step replayed from a HIP graph: what the kernels take once the host is out of the way
    gms = graph_time(step, steps, warmup, lambda: [x.grad, w_in.grad, w_hid.grad, w_out.grad])
    if gms is not None:
        gt = rows * flop_row / (gms * 1e-3) / 1e12
        out["hip_graph"] = {"ms_per_step": gms, "achieved": gt, "unit": "TFLOP/s", "frac": gt / MFMA_BF16_PEAK_TFLOPS}
    return out


def bench_rev(steps, warmup, rows=2**20):
    from triton_helpers_amd.layers.reversible_mlp import kernel as rk

    dev = torch.device("cuda", 0)
    torch.manual_seed(0)
    H, blocks = 64, 4
    w1 = ((torch.rand(blocks * 2 * H, H) * 2 - 1) / 8).bfloat16().to(dev).requires_grad_(True)
    w2 = ((torch.rand(blocks * 2 * H, H) * 2 - 1) / 8).bfloat16().to(dev).requires_grad_(True)
    x = torch.randn(rows, 2 * H).bfloat16().to(dev).requires_grad_(True)
    dy = torch.randn(rows, 2 * H).bfloat16().to(dev)

    def step():
        x.grad = w1.grad = w2.grad = None
        rk.reversible_mlp(x, w1, None, w2, None, "gelu").backward(dy)

    ms = wall_time(step, steps, warmup)
    flop_row = 3 * 2 * blocks * 4 * H * H
    tflops = rows * flop_row / (ms * 1e-3) / 1e12
    return {
        "workload": f"reversible MLP width 128, 4 couplings, GELU bf16 fwd+bwd, {rows} rows (through autograd)",
        "value": rows / ms / 1e3, "unit": "Mrows/s", "ms_per_step": ms,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None},
    }


def bench_e2e(steps, warmup, n=2**21):
    """BASELINE configs[4]: encode -> MLP 32->64->64->4 -> MSE, forward + backward through autograd."""
    from triton_helpers_amd.layers.fully_fused_mlp import kernel as mk
    from triton_helpers_amd.layers.hash_encoding import kernel as hk
    from triton_helpers_amd.layers.hash_encoding.helpers import total_rows

    dev = torch.device("cuda", 0)
    torch.manual_seed(0)
    E = total_rows(T, L, D, MIN_RES, MAX_RES)
    table = ((torch.rand(E, F) * 2 - 1) * 1e-4).half().to(dev).requires_grad_(True)
    x = torch.rand(n, D).to(dev)
    target = torch.rand(n, 4).to(dev)

    def u(shape, fan_in):
        return ((torch.rand(*shape) * 2 - 1) / fan_in**0.5).bfloat16().to(dev).requires_grad_(True)

    w_in, w_hid, w_out = u((64, 32), 32), u((64, 64), 64), u((4, 64), 64)

    def step():
        table.grad = w_in.grad = w_hid.grad = w_out.grad = None
        enc = hk.hash_encoding(x, table, None, None, T, MIN_RES, MAX_RES, L)
        # the fp16 encoding goes straight into the bf16 MLP, which converts it while loading (and writes dx as fp16)
        y = mk.fully_fused_mlp(enc.unsqueeze(0), w_in, None, w_out, None, w_hid, None, "relu")
        # summed (not averaged) squared error: keeps the fp16 gradient that reaches the encoder out of underflow
        loss = torch.nn.functional.mse_loss(y.float().squeeze(0), target, reduction="sum")
        loss.backward()

    ms = wall_time(step, steps, warmup)
    return {"workload": f"end-to-end step: {n} points -> hash encoding -> MLP 32->64->64->4 -> summed squared error, fwd+bwd",
            "value": n / ms / 1e3, "unit": "Mpoints/s", "ms_per_step": ms}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extras", action="store_true", help="skip the MLP / end-to-end workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one out-of-place add over 256 MiB (a copy kernel of known traffic, for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--hash-kernel-flags", type=int, default=0,
                    help="NF_HASH_* flag bits passed to the hash-encoding entry points (profiling the alternative "
                         "kernels, e.g. 8 = LDS-staged forward); the default 0 is what the bench line is quoted on")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (points are independent, so the work "
              "would shard over points with one gradient all-reduce). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    torch.cuda.set_device(0)
    if args.hash_kernel_flags:
        from triton_helpers_amd.layers.hash_encoding import kernel as hk
        hk._FLAGS = args.hash_kernel_flags

    h = bench_hash(args.steps, args.warmup)
    # The forward is one kernel (hash_fwd_sweep_k); the backward is zero + count + offsets + fill + accumulate, each
    # shorter than the forward kernel.
    dom, dom_ms, dom_bytes = ("hash_fwd_tiled_k" if args.hash_kernel_flags & 8 else "hash_fwd_sweep_k"), h["t_fwd"], FWD_BYTES_PER_POINT * N_POINTS
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    bwd_achieved = BWD_BYTES_PER_POINT * N_POINTS / (h["t_bwd"] * 1e-3) / 1e9
    step_bytes = (FWD_BYTES_PER_POINT + BWD_BYTES_PER_POINT) * N_POINTS + h["E"] * F * 4
    out = {
        "metric": "Mpoints/s fwd+bwd: hash-enc+fused MLP @2^20 pts; % HBM / MFMA peak",
        "value": N_POINTS / h["ms"] / 1e3,
        "unit": "Mpoints/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": h["ms"],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[1]: hash encoding fwd+bwd, N=2^20 3-D points, L=16, F=2, T=2^19, res 16..7006, "
                        "fp16 tables and upstream grad, float32 table gradient (zero-fill included in the step)",
            "points": N_POINTS, "levels": L, "features": F, "table_rows_per_level": T,
        },
        "roofline": {
            "bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": achieved / HBM_PEAK_GBS, "traffic": FWD_TRAFFIC_BYTES,
            "launch_ms": dom_ms, "algorithmic_bytes_per_launch": dom_bytes,
        },
        "phases_ms": {"hash_fwd": h["t_fwd"], "grad_zero_fill": h["t_zero"], "hash_bwd": h["t_bwd"]},
        "bwd_roofline_frac": bwd_achieved / HBM_PEAK_GBS,
        "step_roofline_frac": step_bytes / (h["ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "autograd_ms_per_step": h["ms_autograd"],
    }
    # What a plain stream reaches on this GPU, next to the 8 TB/s of the data sheet: a 256 MiB out-of-place add
    # (reads 256 MiB, writes 256 MiB) timed with events, median of 20.
    ca = torch.zeros(64 * 2**20, dtype=torch.float32, device="cuda")
    cb = torch.empty_like(ca)
    copy_ms = statistics.median(event_times(lambda: torch.add(ca, 1.0, out=cb), 20)[5:])
    copy_gbs = 2 * ca.numel() * 4 / (copy_ms * 1e-3) / 1e9
    del ca, cb
    out["achievable"] = {
        "stream_GBs": copy_gbs, "how": "256 MiB read + 256 MiB write elementwise add, event-timed",
        "fwd_frac_of_stream": achieved / copy_gbs,
        "bwd_frac_of_stream": bwd_achieved / copy_gbs,
        "step_frac_of_stream": step_bytes / (h["ms"] * 1e-3) / 1e9 / copy_gbs,
    }
    if not args.no_extras:
        s, w = max(5, args.steps // 2), max(3, args.warmup // 2)
        with torch.autograd.set_multithreading_enabled(False):  # backward on the calling thread, see bench_mlp
            out["workloads"] = {
                "configs[2]": bench_mlp(s, w, 16),
                "configs[3]": bench_rev(max(3, s // 2), 2),
                "configs[4]": bench_e2e(max(3, s // 2), 2),
            }
    if args.calibrate_copy:
        a = torch.zeros(64 * 2**20, dtype=torch.float32, device="cuda")
        b = torch.empty_like(a)
        for _ in range(3):
            torch.add(a, 1.0, out=b)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_hash()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
