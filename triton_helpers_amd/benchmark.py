"""Benchmark / profile command line for the layers of this package.

The command line is the reference's (``triton_helpers/benchmark.py``, ``layers/*/__main__.py``): sub-commands
``benchmark`` and ``profile``; ``-p`` providers, ``-m`` modes (``fwd`` / ``bwd`` / ``fwd-bwd``), ``-d`` dtypes
(``fp16`` / ``bf16`` / ``fp32``), ``-w`` warm-up and ``-r`` repetition budgets in milliseconds, one flag per swept
dimension with ``--<dim>-mode values|linspace|logspace``, ``-l`` line argument, ``-x`` x dimension, ``-o`` output
directory.  So are the statistics (median and 20 % / 80 % quantiles of event-timed calls, the L2 cache overwritten before
every call) and the files written: one ``<task>-<mode>-<dims>-<dtype>.csv`` per table, a column per line value followed
by its ``-min`` / ``-max`` quantile columns.  Plots are not drawn.

The machinery behind it is this package's own and small: a *workload* is a name plus two functions (``make`` builds
the inputs of one sweep point, ``run`` calls the layer), a *sweep* is a dictionary of axes, and a table is filled by
timing one closure per cell.  Nothing here depends on Triton.

Usage: ``python -m triton_helpers.layers.hash_encoding benchmark -m fwd bwd -L 65536 131072 -o out/``.
"""
from __future__ import annotations

import argparse
import csv
import itertools
import statistics
from pathlib import Path
from typing import Any, Callable, Dict, List, NamedTuple, Optional, Sequence, Tuple

import torch
from torch import Tensor

MODES = {"fwd": "Forward", "bwd": "Backward", "fwd-bwd": "Forward-Backward"}
DTYPES = {"fp16": torch.float16, "bf16": torch.bfloat16, "fp32": torch.float32}
AXIS_MODES = ("values", "linspace", "logspace")


class Workload(NamedTuple):
    """One implementation under test.  ``make(device=, dtype=, requires_grad=, **dims)`` returns the keyword arguments
    of ``run``; ``run(**inputs)`` returns the output tensor of one forward call."""

    provider: str
    make: Callable[..., Dict[str, Any]]
    run: Callable[..., Tensor]

    @property
    def title(self) -> str:
        return self.provider.title()


class Timing(NamedTuple):
    median: float
    low: float
    high: float


class Table(NamedTuple):
    name: str
    header: List[str]
    rows: List[List[float]]


# ------------------------------------------------------------------------------------------------ axes
def axis_values(values: Sequence[int], how: str) -> List[int]:
    """``values``: the numbers themselves; ``linspace``: ``start stop step`` (stop included); ``logspace``:
    ``start stop count`` as exponents of two."""
    if how == "values":
        return list(values)
    if len(values) != 3:
        raise ValueError(f"{how} takes three numbers (start, stop, step or count), got {list(values)}")
    a, b, c = values
    if how == "linspace":
        return list(range(a, b + 1, c))
    if how == "logspace":
        return [int(round(2.0 ** (a + (b - a) * i / max(c - 1, 1)))) for i in range(c)]
    raise ValueError(f"unknown axis mode {how!r}")


# ------------------------------------------------------------------------------------------------ timing
_flush_buffers: Dict[int, Tensor] = {}


def _flush_cache() -> None:
    """Overwrite 256 MiB, more than the GPU's L2 and memory-side cache keep, so that every timed call starts cold."""
    dev = torch.cuda.current_device()
    buf = _flush_buffers.get(dev)
    if buf is None:
        buf = _flush_buffers[dev] = torch.empty(64 * 2**20, dtype=torch.int32, device=f"cuda:{dev}")
    buf.zero_()


def _timed(fn: Callable[[], Any], n: int, cold: bool) -> List[float]:
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n)]
    for begin, end in pairs:
        if cold:
            _flush_cache()
        begin.record()
        fn()
        end.record()
    torch.cuda.synchronize()
    return [begin.elapsed_time(end) for begin, end in pairs]


def time_calls(fn: Callable[[], Any], warmup_ms: float = 20, rep_ms: float = 100, cold: bool = True) -> Timing:
    """Milliseconds per call: median and the 20 % / 80 % quantiles.  The two budgets are times, not counts: the number
    of warm-up and timed calls is the budget over the duration of a few probe calls (at least one each)."""
    fn()
    torch.cuda.synchronize()
    probe = max(statistics.fmean(_timed(fn, 5, cold)), 1e-4)
    for _ in range(max(1, int(warmup_ms / probe))):
        fn()
    ms = sorted(_timed(fn, max(1, int(rep_ms / probe)), cold))

    def at(q: float) -> float:
        pos = q * (len(ms) - 1)
        i = int(pos)
        j = min(i + 1, len(ms) - 1)
        return ms[i] + (ms[j] - ms[i]) * (pos - i)

    return Timing(at(0.5), at(0.2), at(0.8))


# ------------------------------------------------------------------------------------------------ what is timed
def step_closure(work: Workload, mode: str, dtype: torch.dtype, device: str, dims: Dict[str, int]) -> Callable[[], Any]:
    """The call that is timed.  ``fwd``: the forward on inputs without gradients.  ``bwd``: one forward up front, then
    only ``backward`` of its output with a fixed upstream gradient.  ``fwd-bwd``: forward, a fresh random upstream
    gradient and backward per call (the reference times the same three things, ``benchmark.py:189-215``)."""
    if mode not in MODES:
        raise ValueError(f"unknown mode {mode!r}")
    inputs = work.make(device=device, dtype=dtype, requires_grad=mode != "fwd", **dims)
    if mode == "fwd":
        return lambda: work.run(**inputs)
    if mode == "bwd":
        out = work.run(**inputs)
        upstream = torch.randn_like(out)
        return lambda: out.backward(upstream, retain_graph=True)

    def both():
        out = work.run(**inputs)
        out.backward(torch.randn_like(out), retain_graph=True)
        return out

    return both


def profile_once(work: Workload, mode: str, dtype_name: str, device: str, dims: Dict[str, int], warmup: int) -> None:
    """Warm up, then one call inside a named range (for ``rocprofv3 --kernel-trace`` / ``--marker-trace``)."""
    fn = step_closure(work, mode, DTYPES[dtype_name], device, dims)
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    label = f"{work.provider}-{mode}-{dtype_name}"
    try:
        torch.cuda.nvtx.range_push(label)  # roctx on ROCm builds of torch
        ranged = True
    except Exception:
        ranged = False
    fn()
    torch.cuda.synchronize()
    if ranged:
        torch.cuda.nvtx.range_pop()


# ------------------------------------------------------------------------------------------------ the sweep
_LINE_NAMES = {
    "kernel": lambda w: w.title,
    "dtype": lambda d: d.upper(),
    "mode": lambda m: MODES[m],
}


def sweep(task: str, workloads: Sequence[Workload], axes: Dict[str, List[int]], modes: Sequence[str], dtypes: Sequence[str],
          x_dim: str, line_arg: str = "kernel", measure: Optional[Callable[[Workload, str, str, Dict[str, int]], Timing]] = None,
          output: Optional[Path] = None, quiet: bool = False) -> List[Table]:
    """One table per combination of everything that is neither the x dimension nor the line argument; ``measure`` fills
    a cell (``None``: cells stay NaN, as for ``profile``)."""
    if output is not None and not Path(output).is_dir():
        raise NotADirectoryError(f"Output path {output} is not a directory")
    if not workloads or not axes or not modes or not dtypes:
        raise ValueError("a sweep needs at least one kernel, one dimension, one mode and one dtype")
    varied: Dict[str, List[Any]] = {"kernel": list(workloads), "dtype": list(dtypes), "mode": list(modes)}
    varied.update({k: v for k, v in axes.items() if k != x_dim})
    if line_arg not in varied:
        raise ValueError(f"Unsupported line arg {line_arg}")
    line_values = varied.pop(line_arg)
    line_name = _LINE_NAMES.get(line_arg, lambda v: f"{line_arg}={v}")
    header = [x_dim]
    for v in line_values:
        header += [line_name(v), f"{line_name(v)}-min", f"{line_name(v)}-max"]
    tables = []
    keys = list(varied)
    for combo in itertools.product(*(varied[k] for k in keys)):
        fixed = dict(zip(keys, combo))
        dims_part = "-".join(f"{k}={v}" for k, v in fixed.items() if k in axes)
        parts = [task, fixed["kernel"].title if "kernel" in fixed else "", fixed.get("mode", ""), dims_part, fixed.get("dtype", "")]
        name = "-".join(p for p in parts if p)
        rows = []
        for x in axes[x_dim]:
            row = [float(x)]
            for v in line_values:
                cell = dict(fixed, **{line_arg: v, x_dim: x})
                work, mode, dtype = cell.pop("kernel"), cell.pop("mode"), cell.pop("dtype")
                row += list(measure(work, mode, dtype, cell)) if measure is not None else [float("nan")] * 3
            rows.append(row)
        tables.append(Table(name, header, rows))
        if measure is not None and not quiet:
            print(f"{name}:\n{_format(header, rows)}", flush=True)
        if measure is not None and output is not None:
            with open(Path(output) / f"{name}.csv", "w", newline="") as f:
                csv.writer(f).writerows([header] + rows)
    return tables


def _format(header: Sequence[str], rows: Sequence[Sequence[float]]) -> str:
    cells = [list(header)] + [[f"{v:.6g}" for v in r] for r in rows]
    widths = [max(len(r[i]) for r in cells) for i in range(len(header))]
    return "\n".join("  ".join(c.rjust(w) for c, w in zip(r, widths)) for r in cells)


# ------------------------------------------------------------------------------------------------ command line
def run_cli(task: str, workloads: Sequence[Workload], dims: Dict[str, Tuple[Any, str]], argv: Optional[Sequence[str]] = None) -> List[Table]:
    """Parse the command line and run it.  ``dims``: name -> (default value or values, default axis mode), the first
    one being the default x dimension."""
    parser = argparse.ArgumentParser(description="Benchmark the gfx950 kernels.", formatter_class=argparse.ArgumentDefaultsHelpFormatter)
    commands = parser.add_subparsers(help="Sub-commands", dest="command", required=True)
    bench = commands.add_parser("benchmark", help="Benchmark kernels")
    prof = commands.add_parser("profile", help="Profile kernels")
    names = [w.provider for w in workloads]
    for sub in (bench, prof):
        sub.add_argument("-p", "--providers", nargs="+", default=names, choices=names, help="Providers to evaluate.")
        sub.add_argument("-m", "--modes", nargs="+", default=["fwd"], choices=list(MODES), help="Modes to evaluate.")
        sub.add_argument("-d", "--dtypes", nargs="+", default=["fp16"], choices=list(DTYPES), help="Data types to evaluate.")
        sub.add_argument("-w", "--warmup", type=int, default=20, help="Warmup budget (ms); for profile: warm-up calls.")
        sub.add_argument("--device", default="cuda", help="Device to use for benchmarking or profiling.")
        for name, (default, how) in dims.items():
            flag = f"-{name}" if len(name) == 1 else f"--{name}"
            sub.add_argument(flag, type=int, nargs="+", default=[default] if isinstance(default, int) else list(default),
                             help=f"Value(s) for {name} dimension.")
            sub.add_argument(f"--{name}-mode", choices=AXIS_MODES, default=how,
                             help=f"How to read {flag}: the values, start stop step (linspace) or start stop count as powers of two (logspace).")
    first = next(iter(dims))
    bench.add_argument("-l", "--line-arg", default="kernel", choices=["kernel", "dtype", "mode"] + list(dims), help="Line argument")
    bench.add_argument("-x", "--x-dim", default=first, choices=list(dims), help="Dimension to use as table X axis")
    bench.add_argument("--x-label", default="Input Size", help="Label for the x axis (kept for command-line compatibility).")
    bench.add_argument("-r", "--rep", type=int, default=100, help="Repetition budget (ms).")
    bench.add_argument("-o", "--output", type=Path, default=None, help="Output directory")
    args = parser.parse_args(argv)

    axes = {name: axis_values(getattr(args, name), getattr(args, f"{name}_mode")) for name in dims}
    chosen = [w for w in workloads if w.provider in args.providers]
    if args.command == "profile":
        tables = sweep(task, chosen, axes, args.modes, args.dtypes, first)
        for t_work, t_mode, t_dtype, cell in _cells(chosen, axes, args.modes, args.dtypes):
            profile_once(t_work, t_mode, t_dtype, args.device, cell, args.warmup)
        return tables

    def measure(work: Workload, mode: str, dtype: str, cell: Dict[str, int]) -> Timing:
        return time_calls(step_closure(work, mode, DTYPES[dtype], args.device, cell), args.warmup, args.rep)

    return sweep(task, chosen, axes, args.modes, args.dtypes, args.x_dim, args.line_arg, measure, args.output)


def _cells(workloads, axes, modes, dtypes):
    names = list(axes)
    for work, mode, dtype in itertools.product(workloads, modes, dtypes):
        for values in itertools.product(*(axes[n] for n in names)):
            yield work, mode, dtype, dict(zip(names, values))
