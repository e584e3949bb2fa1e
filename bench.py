#!/usr/bin/env python3
"""Benchmark of the neural-field hot paths on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W]`` prints ONE JSON line.

The headline workload is BASELINE.json ``configs[1]``: multiresolution hash encoding,
forward + backward, N = 2^20 points, L = 16, F = 2, T = 2^19, fp16 tables, fp16 upstream
gradient, float32 table gradient.  One step = forward launch + clearing the float32
gradient table + backward launch(es), inputs resident in HBM.  ``value`` is Mpoints/s over
exactly K steps of wall time; ``event_ms`` gives the median and the 20 % / 80 % quantiles of the
same K steps timed one by one with events (the reference's ``do_bench`` statistics,
triton_helpers/benchmark.py:151-153, 179-184: warm-up 20, 100 repetitions, median, quantiles).

Extra objects in the same line:
  roofline      the dominant kernel of the step (the forward gather kernel: the backward is a
                chain of five shorter kernels), algorithmic bytes per launch / launch time measured
                here with events against the 8 TB/s HBM peak; ``traffic`` (HBM bytes per launch) and
                the L2 request count are counter figures of a separate profiler run, kept in the
                committed profile summary together with that run's kernel time: they are quoted
                (``traffic_source`` says from where) only while this run's launch time is within 10 %
                of it, and are null otherwise;
  cpu_baseline  the CPU oracle (a port of the reference's PyTorch path) timed on this host
                on a 65536-point sample of the same workload; ``cpu_baselines`` holds the same for
                the other configurations (configs[0] is the reference's own CPU-runnable case);
  workloads     the other BASELINE configs (fused MLP, reversible MLP, end-to-end step) with
                their own throughput and MFMA roofline fraction.

``--only 2`` (= ``configs[2]``; also 1, 3, 4) runs that workload alone, W warm-up + K steps, and prints its object: the
command to put behind ``rocprofv3 ... --`` for per-kernel counters.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16
# L2: 16 channels per XCD, 128 bytes per clock each, 8 XCDs, 2.4 GHz
L2_PEAK_GBS = 16 * 128 * 8 * 2.4

# geometry of BASELINE configs[1] ("base 16, growth 1.5, L=16" == min_res 16, max_res 7006)
T, L, F, D, MIN_RES, MAX_RES = 2**19, 16, 2, 3, 16, 7006
N_POINTS = 2**20
# algorithmic bytes per point: fwd = 4D + L*2^D*F*2 + L*F*2 ; bwd = 4D + L*F*2 + L*2^D*F*4
FWD_BYTES_PER_POINT = 4 * D + L * 8 * F * 2 + L * F * 2  # 588
BWD_BYTES_PER_POINT = 4 * D + L * F * 2 + L * 8 * F * 4  # 1100
PROFILE_SUMMARY = os.path.join(ROOT, "profiles", "hash_encoding_fwd_bwd_2p20.md")
E2E_LOSS_SCALE = 2.0**20
CPU_SAMPLE = 65536


def profile_figures(kernel, launch_ms):
    """Counter-derived figures of the forward kernel.  They cannot be measured in this run (hardware counters need
    the profiler), so the committed profile summary keeps them in a line
    ``<!-- bench-figures: kernel=<name> kernel_us=<its duration in the counter run> key=value ... -->`` next to the
    tables they come from.  Returns (figures, source): the figures are used only when the line names the kernel this
    run launches and its duration then is within 10 % of the duration measured now; otherwise ({}, why)."""
    rel = os.path.relpath(PROFILE_SUMMARY, ROOT)
    try:
        text = open(PROFILE_SUMMARY).read()
    except OSError:
        return {}, f"{rel} is missing"
    m = re.search(r"<!--\s*bench-figures:(.*?)-->", text, flags=re.S)
    if not m:
        return {}, f"{rel} holds no bench-figures line"
    name = re.search(r"kernel=(\S+)", m.group(1))
    figs = {k: float(v) for k, v in re.findall(r"(\w+)=([0-9.eE+-]+)(?=\s|$)", m.group(1))}
    if name is None or name.group(1) != kernel or "kernel_us" not in figs:
        return {}, f"{rel}: the counter figures are for {name.group(1) if name else 'an unnamed kernel'}, this run launches {kernel}"
    then_us, now_us = figs["kernel_us"], launch_ms * 1e3
    if abs(then_us - now_us) > 0.10 * now_us:
        return {}, f"{rel}: stale -- {kernel} took {then_us:.1f} us in the counter run and {now_us:.1f} us now"
    return figs, f"{rel}: rocprofv3 --pmc run of {kernel} ({then_us:.1f} us per launch there, {now_us:.1f} us here)"


def quantiles(ms):
    s = sorted(ms)
    pick = lambda q: s[min(len(s) - 1, int(q * (len(s) - 1) + 0.5))]  # noqa: E731
    return {"median": statistics.median(s), "p20": pick(0.2), "p80": pick(0.8), "n": len(s)}


def event_times(fn, reps):
    """Per-call GPU duration (ms) of ``fn`` measured with events on the current stream (the stream the library
    launches on)."""
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


# ------------------------------------------------------------------------------------------------ GPU workloads
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
    step_ev = quantiles(event_times(step, steps))
    reps = max(10, min(steps, 100))
    fwd_ev = quantiles(event_times(fwd, reps))
    t_zero = statistics.median(event_times(zero, reps))
    bwd_ev = quantiles(event_times(bwd, reps))

    # the same step through autograd (table grad rounded to fp16 by the engine), for information
    e = table.clone().requires_grad_(True)

    def step_autograd():
        e.grad = None
        hk.hash_encoding(x, e, None, pi, T, MIN_RES, MAX_RES, L).backward(do)

    ms_autograd = wall_time(step_autograd, max(5, steps // 5), 3)
    return dict(ms=ms, step_ev=step_ev, fwd_ev=fwd_ev, t_zero=t_zero, bwd_ev=bwd_ev, ms_autograd=ms_autograd, E=E)


def bench_mlp(steps, warmup, d_out=16, rows=2**20, graph=True):
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

    # The headline is the step as torch runs it by default: the autograd engine executes the backward on a device
    # thread of its own, two hand-overs between host threads per step.  With
    # torch.autograd.set_multithreading_enabled(False) the backward runs on the calling thread; that figure and the
    # replay of the captured step from a HIP graph are reported beside it.
    with torch.autograd.set_multithreading_enabled(True):
        ms = wall_time(step, steps, warmup)
        ev = quantiles(event_times(step, steps))
    with torch.autograd.set_multithreading_enabled(False):
        ms_calling_thread = wall_time(step, steps, warmup)
    flop_row = 3 * 2 * (32 * 64 + 64 * 64 + 64 * d_out)

    def tf(t_ms):
        return rows * flop_row / (t_ms * 1e-3) / 1e12

    out = {
        "workload": f"configs[2]: fused MLP 32->64->64->{d_out} ReLU bf16 fwd+bwd, {rows} rows (through autograd, default engine)",
        "value": rows / ms / 1e3, "unit": "Mrows/s", "ms_per_step": ms, "event_ms": ev,
        "roofline": {"bound": "mfma", "achieved": tf(ms), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tf(ms) / MFMA_BF16_PEAK_TFLOPS, "traffic": None},
        "hbm_GBs": rows * 256 / (ms * 1e-3) / 1e9,
        "backward_on_calling_thread": {"ms_per_step": ms_calling_thread, "achieved": tf(ms_calling_thread), "unit": "TFLOP/s",
                                       "frac": tf(ms_calling_thread) / MFMA_BF16_PEAK_TFLOPS,
                                       "how": "torch.autograd.set_multithreading_enabled(False)"},
    }
    if graph:
        with torch.autograd.set_multithreading_enabled(False):
            gms = graph_time(step, steps, warmup, lambda: [x.grad, w_in.grad, w_hid.grad, w_out.grad])
        if gms is not None:
            out["hip_graph"] = {"ms_per_step": gms, "achieved": tf(gms), "unit": "TFLOP/s", "frac": tf(gms) / MFMA_BF16_PEAK_TFLOPS}
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
    ev = quantiles(event_times(step, steps))
    flop_row = 3 * 2 * blocks * 4 * H * H
    tflops = rows * flop_row / (ms * 1e-3) / 1e12
    return {
        "workload": f"configs[3]: reversible MLP width 128, 4 couplings, GELU bf16 fwd+bwd, {rows} rows (through autograd)",
        "value": rows / ms / 1e3, "unit": "Mrows/s", "ms_per_step": ms, "event_ms": ev,
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / MFMA_BF16_PEAK_TFLOPS, "traffic": None},
    }


def bench_e2e(steps, warmup, n=2**21):
    """BASELINE configs[4]: encode -> MLP 32->64->64->4 -> MSE (mean), forward + backward through autograd."""
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
        loss = torch.nn.functional.mse_loss(y.float().squeeze(0), target)
        # Mean over n * 4 elements: the gradient that reaches the fp16 encoding is ~1e-9 and would underflow, as in
        # any fp16 training step; a constant loss scale (what torch.amp.GradScaler applies dynamically) keeps it in
        # range.  The gradients come out multiplied by it (an optimiser step would divide them).
        (loss * E2E_LOSS_SCALE).backward()

    ms = wall_time(step, steps, warmup)
    ev = quantiles(event_times(step, steps))
    return {"workload": f"configs[4]: end-to-end step: {n} points -> hash encoding -> MLP 32->64->64->4 -> MSE (mean), "
                        f"loss scale 2^20, fwd+bwd",
            "value": n / ms / 1e3, "unit": "Mpoints/s", "ms_per_step": ms, "event_ms": ev}


# ------------------------------------------------------------------------------------------------ CPU baselines
def _cpu_threads():
    """Threads for the CPU baselines: the host's cores, at most 16 -- a GPU box of this pool gives one GPU's job a share
    of 16 cores (its OMP_NUM_THREADS is preset to 16), whatever os.cpu_count() shows."""
    n = min(os.cpu_count() or 1, 16)
    torch.set_num_threads(n)
    return n


def _time_cpu(run, budget_s=6.0, max_reps=20):
    run()  # warm-up
    times, t_start = [], time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - t_start < budget_s and len(times) < max_reps):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    return statistics.median(times), len(times)


def _cpu_entry(n, med, reps, unit, sample):
    return {"value": n / med / 1e6, "unit": unit, "cores": torch.get_num_threads(), "host_cpu_count": os.cpu_count(),
            "kind": "port", "sample": f"{sample}; median of {reps} runs"}


def cpu_baseline_hash(backward=True, fp32=False):
    """CPU oracle (port of the reference's PyTorch path, triton_helpers/layers/hash_encoding/kernel.py:482-502) on a
    65536-point sample of the workload; ``fp32`` + forward only is BASELINE configs[0] at its full size."""
    from oracle import hash_encoding as O

    n = CPU_SAMPLE
    _cpu_threads()
    torch.manual_seed(0)
    E = O.level_row_offsets(L, T, D, MIN_RES, MAX_RES)[-1]
    x = torch.rand(n, D)
    table = (torch.rand(E, F) * 2 - 1) * 1e-4
    table = table if fp32 else table.half()
    do = torch.randn(n, L * F).half()

    def run():
        O.encode_forward(x, table, None, T, L, MIN_RES, MAX_RES)
        if backward:
            O.encode_backward(x, do, E, F, None, T, L, MIN_RES, MAX_RES)

    med, reps = _time_cpu(run)
    what = "fwd+bwd" if backward else "forward"
    tab = "fp32 table" if fp32 else "fp16 table, fp32 grad"
    return _cpu_entry(n, med, reps, "Mpoints/s", f"{what} of {n} points, same geometry (L=16,F=2,T=2^19), {tab}")


def cpu_baseline_mlp(d_out=16):
    """float32 F.linear chain with autograd (the reference tests' baseline, tests/test_layers/test_fully_fused_mlp.py:21-35)."""
    from oracle import mlp as M

    n = CPU_SAMPLE
    _cpu_threads()
    torch.manual_seed(0)
    w_in, w_hid, w_out = torch.randn(64, 32) / 6, torch.randn(64, 64) / 8, torch.randn(d_out, 64) / 8
    x, dy = torch.randn(n, 32), torch.randn(n, d_out)
    med, reps = _time_cpu(lambda: M.mlp_backward(x, dy, w_in, None, w_out, None, w_hid, None, "relu"))
    return _cpu_entry(n, med, reps, "Mrows/s", f"fwd+bwd of {n} rows, 32->64->64->{d_out} ReLU, float32")


def cpu_baseline_rev():
    from oracle import reversible as R

    n = CPU_SAMPLE
    _cpu_threads()
    torch.manual_seed(0)
    w1, w2 = torch.randn(4 * 2 * 64, 64) / 8, torch.randn(4 * 2 * 64, 64) / 8
    x, dy = torch.randn(n, 128), torch.randn(n, 128)
    med, reps = _time_cpu(lambda: R.rev_backward(x, dy, w1, None, w2, None, "gelu"))
    return _cpu_entry(n, med, reps, "Mrows/s", f"fwd+bwd of {n} rows, width 128, 4 couplings, GELU, float32, stored activations")


def cpu_baseline_e2e():
    from oracle import hash_encoding as O
    from oracle import mlp as M

    n = CPU_SAMPLE
    _cpu_threads()
    torch.manual_seed(0)
    E = O.level_row_offsets(L, T, D, MIN_RES, MAX_RES)[-1]
    x = torch.rand(n, D)
    table = ((torch.rand(E, F) * 2 - 1) * 1e-4).half()
    target = torch.rand(n, 4)
    w_in, w_hid, w_out = torch.randn(64, 32) / 6, torch.randn(64, 64) / 8, torch.randn(4, 64) / 8

    def run():
        enc = O.encode_forward(x, table, None, T, L, MIN_RES, MAX_RES).float().requires_grad_(True)
        leaves = [t.clone().requires_grad_(True) for t in (w_in, w_out, w_hid)]
        y = M.mlp_forward(enc, leaves[0], None, leaves[1], None, leaves[2], None, "relu")
        torch.nn.functional.mse_loss(y, target).backward()
        O.encode_backward(x, enc.grad, E, F, None, T, L, MIN_RES, MAX_RES)

    med, reps = _time_cpu(run)
    return _cpu_entry(n, med, reps, "Mpoints/s", f"fwd+bwd of {n} points: encode -> MLP 32->64->64->4 -> MSE, float32")


# ------------------------------------------------------------------------------------------------ main
def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--only", choices=["configs[1]", "configs[2]", "configs[3]", "configs[4]", "1", "2", "3", "4"], default=None,
                    help="run this workload alone (for per-kernel profiling) and print its object; a bare digit is "
                         "short for configs[digit]")
    ap.add_argument("--no-extras", action="store_true", help="skip the MLP / end-to-end workloads")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baselines")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one out-of-place add over 256 MiB (a copy kernel of known traffic, for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a profiler run)")
    ap.add_argument("--hash-kernel-flags", type=int, default=0,
                    help="NF_HASH_* flag bits passed to the hash-encoding entry points (profiling the alternative "
                         "kernels, e.g. 8 = LDS-staged forward); the default 0 is what the bench line is quoted on")
    args = ap.parse_args()
    if args.only and len(args.only) == 1:
        args.only = f"configs[{args.only}]"
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

    if args.only and args.only != "configs[1]":
        fn = {"configs[2]": lambda: bench_mlp(args.steps, args.warmup, 16, graph=False),
              "configs[3]": lambda: bench_rev(args.steps, args.warmup),
              "configs[4]": lambda: bench_e2e(args.steps, args.warmup)}[args.only]
        print(json.dumps(fn()))
        return

    h = bench_hash(args.steps, args.warmup)
    # The forward is one kernel (hash_fwd_sweep_k); the backward is zero + count + offsets + fill + accumulate, each
    # shorter than the forward kernel.
    dom = "hash_fwd_tiled_k" if args.hash_kernel_flags & 8 else "hash_fwd_sweep_k"
    dom_ms, dom_bytes = h["fwd_ev"]["median"], FWD_BYTES_PER_POINT * N_POINTS
    t_bwd = h["bwd_ev"]["median"]
    achieved = dom_bytes / (dom_ms * 1e-3) / 1e9
    bwd_achieved = BWD_BYTES_PER_POINT * N_POINTS / (t_bwd * 1e-3) / 1e9
    step_bytes = (FWD_BYTES_PER_POINT + BWD_BYTES_PER_POINT) * N_POINTS + h["E"] * F * 4
    figs, figs_source = profile_figures(dom, dom_ms)
    roofline = {
        "bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
        "frac": achieved / HBM_PEAK_GBS, "traffic": figs.get("fwd_traffic_bytes"), "traffic_source": figs_source,
        "launch_ms": dom_ms, "launch_ms_p20_p80": [h["fwd_ev"]["p20"], h["fwd_ev"]["p80"]],
        "algorithmic_bytes_per_launch": dom_bytes,
    }
    if "fwd_l2_read_requests" in figs:
        # the gathers are served by L2 (90 % hits): requests that leave the CUs x 128-byte lines over the launch time
        l2 = figs["fwd_l2_read_requests"] * 128 / (dom_ms * 1e-3) / 1e9
        roofline["l2"] = {"read_requests": figs["fwd_l2_read_requests"], "achieved": l2, "peak": L2_PEAK_GBS, "unit": "GB/s",
                          "frac": l2 / L2_PEAK_GBS, "peak_how": "16 channels x 128 B/clk x 8 XCDs x 2.4 GHz",
                          "source": "request count from the same counter run as traffic, time from this run"}
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
        "event_ms": h["step_ev"],
        "roofline": roofline,
        "phases_ms": {"hash_fwd": dom_ms, "grad_zero_fill": h["t_zero"], "hash_bwd": t_bwd,
                      "hash_bwd_p20_p80": [h["bwd_ev"]["p20"], h["bwd_ev"]["p80"]]},
        "bwd_roofline_frac": bwd_achieved / HBM_PEAK_GBS,
        "step_roofline_frac": step_bytes / (h["ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS,
        "autograd_ms_per_step": h["ms_autograd"],
    }
    if args.only == "configs[1]":
        print(json.dumps(out))
        return
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
        out["workloads"] = {
            "configs[2]": bench_mlp(s, w, 16),
            "configs[3]": bench_rev(max(20, s // 2), 5),
            "configs[4]": bench_e2e(max(20, s // 2), 5),
        }
    if args.calibrate_copy:
        a = torch.zeros(64 * 2**20, dtype=torch.float32, device="cuda")
        b = torch.empty_like(a)
        for _ in range(3):
            torch.add(a, 1.0, out=b)  # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline_hash()
        out["cpu_baselines"] = {
            "configs[0]": cpu_baseline_hash(backward=False, fp32=True),
            "configs[2]": cpu_baseline_mlp(16),
            "configs[3]": cpu_baseline_rev(),
            "configs[4]": cpu_baseline_e2e(),
        }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
