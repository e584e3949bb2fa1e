"""Benchmark / profile command line for the layers of this package.

Mirrors the harness of the reference (``triton_helpers/benchmark.py``): the same sub-commands (``benchmark``,
``profile``), the same flags (``-p`` providers, ``-m`` modes ``fwd`` / ``bwd`` / ``fwd-bwd``, ``-d`` dtypes, ``-w`` warm-up,
``-r`` repetitions, one flag per dimension with ``--<dim>-mode values|linspace|logspace``, ``-l`` line argument, ``-x`` x
dimension, ``-o`` output directory), the same three closures per mode (reference ``benchmark.py:189-215``) and the same
statistics: median and the 20 % / 80 % quantiles of event-timed runs after a timed warm-up, with the L2 cache cleared
before every run (what ``triton.testing.do_bench`` does, reference ``benchmark.py:175-187``).  Results are printed as a
table per (mode, dtype, other dimensions) and written as ``<task>-<mode>-<dims>-<dtype>.csv`` with one column per line
value plus its ``-min`` / ``-max`` quantile columns, the layout of the reference's published CSV files.  Plots are not
drawn.  Nothing here depends on Triton.

Usage: ``python -m triton_helpers.layers.hash_encoding benchmark -m fwd bwd -L 65536 131072 -o out/``.
"""
from __future__ import annotations

import csv
import statistics
import sys
from abc import abstractmethod
from argparse import ArgumentDefaultsHelpFormatter, ArgumentParser, Namespace
from dataclasses import dataclass, field
from enum import Enum
from itertools import product
from pathlib import Path
from typing import Any, Callable, Dict, Iterator, List, Optional, Sequence, Tuple

import torch
from torch import Tensor


class _StrEnum(str, Enum):
    def __str__(self) -> str:
        return str(self.value)


class Dtype(_StrEnum):
    FP16 = "fp16"
    BF16 = "bf16"
    FP32 = "fp32"

    @property
    def torch(self) -> torch.dtype:
        return {Dtype.FP16: torch.float16, Dtype.BF16: torch.bfloat16, Dtype.FP32: torch.float32}[self]


class Endpoint(_StrEnum):
    PROFILE = "profile"
    BENCHMARK = "benchmark"


class Mode(_StrEnum):
    FORWARD = "fwd"
    BACKWARD = "bwd"
    FORWARD_BACKWARD = "fwd-bwd"

    @property
    def long_name(self) -> str:
        return {Mode.FORWARD: "Forward", Mode.BACKWARD: "Backward", Mode.FORWARD_BACKWARD: "Forward-Backward"}[self]


@dataclass
class DimConfig:
    """One swept dimension (reference ``benchmark.py:64-143``)."""

    name: str
    values: Sequence[int]

    def __len__(self) -> int:
        return len(self.values)

    def __iter__(self) -> Iterator[int]:
        yield from self.values

    @classmethod
    def from_range(cls, name: str, start: int, stop: int, step: int, logspace: bool = False) -> "DimConfig":
        if logspace:
            vals = torch.logspace(start, stop, step, base=2).int().tolist()
        else:
            vals = list(range(start, stop + 1, step))
        return cls(name, vals)

    @staticmethod
    def add_argument(parser: ArgumentParser, name: str, default_val, default_mode: str = "values") -> None:
        key = f"-{name}" if len(name) == 1 else f"--{name}"
        parser.add_argument(key, type=int, nargs="+", default=[default_val] if isinstance(default_val, int) else list(default_val),
                            help=f"Value(s) for {name} dimension.")
        parser.add_argument(f"--{name}-mode", type=str, choices=["values", "linspace", "logspace"], default=default_mode,
                            help=f"How to read {key}: the values themselves, or start stop step (linspace) / start stop steps as powers of two (logspace).")

    @classmethod
    def from_namespace(cls, args: Namespace, name: str) -> "DimConfig":
        if name not in args:
            raise ValueError(f"Cannot find values for {name} dimension.")
        values = getattr(args, name)
        mode = getattr(args, f"{name}_mode")
        if mode == "values":
            return cls(name, values)
        if mode == "linspace":
            return cls.from_range(name, *values)
        if mode == "logspace":
            return cls.from_range(name, *values, logspace=True)
        raise ValueError(f"Unsupported mode {mode}")


_l2_flush: Dict[torch.device, Tensor] = {}


def do_bench(fn: Callable[[], Any], warmup: float = 20, rep: float = 100, quantiles: Sequence[float] = (0.5, 0.2, 0.8),
             clear_l2: bool = True) -> Tuple[float, ...]:
    """Milliseconds per call of ``fn`` at the given quantiles.  ``warmup`` and ``rep`` are time budgets in milliseconds, as
    in ``triton.testing.do_bench``: the run count is the budget over an estimate of one call (at least one)."""
    fn()
    torch.cuda.synchronize()
    dev = torch.device("cuda", torch.cuda.current_device())
    if clear_l2 and dev not in _l2_flush:
        _l2_flush[dev] = torch.empty(256 * 2**20 // 4, dtype=torch.int32, device=dev)
    flush = _l2_flush.get(dev)
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        if clear_l2:
            flush.zero_()
        fn()
    end.record()
    torch.cuda.synchronize()
    estimate = max(start.elapsed_time(end) / 5, 1e-4)
    n_warmup, n_repeat = max(1, int(warmup / estimate)), max(1, int(rep / estimate))
    for _ in range(n_warmup):
        fn()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(n_repeat)]
    for a, b in events:
        if clear_l2:
            flush.zero_()
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    times = sorted(a.elapsed_time(b) for a, b in events)
    return tuple(_quantile(times, q) for q in quantiles)


def _quantile(sorted_vals: Sequence[float], q: float) -> float:
    if len(sorted_vals) == 1:
        return sorted_vals[0]
    pos = q * (len(sorted_vals) - 1)
    lo = int(pos)
    hi = min(lo + 1, len(sorted_vals) - 1)
    return sorted_vals[lo] + (sorted_vals[hi] - sorted_vals[lo]) * (pos - lo)


@dataclass
class KernelExecutor:
    """One implementation under test (reference ``benchmark.py:144-247``): subclasses say how to build the inputs and run
    the forward; the three modes are derived here."""

    provider: str
    callback: Optional[Callable] = None
    warmup: int = 20
    rep: int = 100
    quantiles: Tuple[float, float, float] = field(default_factory=lambda: (0.5, 0.2, 0.8))

    def __str__(self) -> str:
        return str.title(self.provider)

    def profile(self, mode: Mode, dtype: Dtype, *args, **kwargs) -> None:
        """Warm up, then one call inside a named range, for ``rocprofv3 --marker-trace`` / ``--kernel-trace``."""
        func = self._get_closure(mode, *args, dtype=dtype.torch, **kwargs)
        for _ in range(self.warmup):
            func()
        torch.cuda.synchronize()
        pushed = False
        try:
            torch.cuda.nvtx.range_push(f"{self.provider}-{mode}-{dtype}")  # roctx on ROCm builds of torch
            pushed = True
        except Exception:
            pass
        func()
        torch.cuda.synchronize()
        if pushed:
            torch.cuda.nvtx.range_pop()
        if self.callback:
            self.callback()

    def benchmark(self, mode: Mode, dtype: Dtype, *args, **kwargs) -> Tuple[float, float, float]:
        func = self._get_closure(mode, *args, dtype=dtype.torch, **kwargs)
        ms, min_ms, max_ms = do_bench(func, quantiles=self.quantiles, warmup=self.warmup, rep=self.rep)
        if self.callback:
            self.callback()
        return ms, min_ms, max_ms

    def _get_closure(self, mode: Mode, *args, **kwargs) -> Callable:
        if mode == Mode.FORWARD:
            _kwargs = self.prepare_inputs(*args, **kwargs, requires_grad=False)
            return lambda: self.forward(**_kwargs)
        if mode == Mode.BACKWARD:
            _kwargs = self.prepare_inputs(*args, **kwargs, requires_grad=True)
            output = self.prepare_backward(self.forward(**_kwargs))
            do = torch.randn_like(output)
            return lambda: self.backward(output, do)
        if mode == Mode.FORWARD_BACKWARD:
            _kwargs = self.prepare_inputs(*args, **kwargs, requires_grad=True)

            def func():
                output = self.prepare_backward(self.forward(**_kwargs))
                do = torch.randn_like(output)
                self.backward(output, do)
                return output

            return func
        raise ValueError(f"Unsupported mode {mode}")

    @abstractmethod
    def prepare_inputs(self, *args, requires_grad: bool = False, **kwargs) -> Dict[str, Any]:
        raise NotImplementedError

    def prepare_backward(self, forward_output: Any) -> Tensor:
        if isinstance(forward_output, Tensor):
            return forward_output
        raise TypeError(f"Unsupported forward output {type(forward_output)}; override prepare_backward to return a tensor.")

    @abstractmethod
    def forward(self, *args, **kwargs) -> Tensor:
        raise NotImplementedError

    def backward(self, output: Tensor, do: Tensor) -> None:
        output.backward(do, retain_graph=True)

    def randn(self, *args, **kwargs) -> Tensor:
        return torch.randn(*args, **kwargs)

    def rand(self, *args, **kwargs) -> Tensor:
        return torch.rand(*args, **kwargs)


@dataclass
class CLI:
    """Runs every (kernel, mode, dtype, dimension values) combination (reference ``benchmark.py:250-580``)."""

    task: str
    kernels: Sequence[KernelExecutor]
    dims: Sequence[DimConfig]
    modes: Sequence[Mode] = field(default_factory=lambda: (Mode.FORWARD,))
    dtypes: Sequence[Dtype] = field(default_factory=lambda: (Dtype.FP16,))
    x_label: str = "Input size"
    output: Optional[Path] = None
    line_arg: str = "kernel"
    x_dim: Optional[str] = None
    device: str = "cuda"

    def __post_init__(self):
        if self.output is not None and not Path(self.output).is_dir():
            raise NotADirectoryError(f"Output path {self.output} is not a directory")
        if not self.kernels:
            raise ValueError("At least one kernel must be provided")
        if not self.dims:
            raise ValueError("At least one dimension must be provided")
        if not self.modes:
            raise ValueError("At least one mode must be provided")
        if not self.dtypes:
            raise ValueError("At least one dtype must be provided")
        if self.x_dim is None:
            self.x_dim = self.dims[0].name

    def tables(self) -> Iterator[Tuple[str, Dict[str, Any], List[Tuple[str, Any]]]]:
        """(table name, fixed arguments, [(line name, line value)]) for every table of the sweep: one table per
        combination of everything that is neither the x dimension nor the line argument."""
        other = [d for d in self.dims if d.name != self.x_dim]
        axes: Dict[str, Sequence[Any]] = {"kernel": list(self.kernels), "dtype": list(self.dtypes), "mode": list(self.modes)}
        for d in other:
            axes[d.name] = list(d)
        if self.line_arg not in axes:
            raise ValueError(f"Unsupported line arg {self.line_arg}")
        line_vals = axes.pop(self.line_arg)
        names = {"kernel": str, "dtype": lambda d: str(d).upper(), "mode": lambda m: m.long_name}
        namer = names.get(self.line_arg, lambda v: f"{self.line_arg}={v}")
        lines = [(namer(v), v) for v in line_vals]
        keys = list(axes)
        for combo in product(*(axes[k] for k in keys)):
            fixed = dict(zip(keys, combo))
            dim_name = "-".join(f"{k}={v}" for k, v in fixed.items() if k not in ("kernel", "dtype", "mode"))
            parts = (self.task, str(fixed["kernel"]) if "kernel" in fixed else None, str(fixed["mode"]) if "mode" in fixed else None,
                     dim_name or None, str(fixed["dtype"]) if "dtype" in fixed else None)
            yield "-".join(p for p in parts if p), fixed, lines

    def __call__(self, endpoint: Endpoint) -> List[Tuple[str, List[str], List[List[float]]]]:
        x_dim = next(d for d in self.dims if d.name == self.x_dim)
        results = []
        for name, fixed, lines in self.tables():
            header = [x_dim.name]
            for ln, _ in lines:
                header += [ln, f"{ln}-min", f"{ln}-max"]
            rows: List[List[float]] = []
            for x in x_dim:
                row: List[float] = [float(x)]
                for _, lv in lines:
                    call = dict(fixed)
                    call[self.line_arg] = lv
                    call[x_dim.name] = x
                    kernel, dtype, mode = call.pop("kernel"), call.pop("dtype"), call.pop("mode")
                    if endpoint == Endpoint.PROFILE:
                        kernel.profile(mode, dtype, device=self.device, **call)
                        row += [float("nan")] * 3
                    else:
                        row += list(kernel.benchmark(mode, dtype, device=self.device, **call))
                rows.append(row)
            results.append((name, header, rows))
            if endpoint == Endpoint.BENCHMARK:
                print(f"{name}:")
                print(_format_table(header, rows), flush=True)
                if self.output is not None:
                    with open(Path(self.output) / f"{name}.csv", "w", newline="") as f:
                        w = csv.writer(f)
                        w.writerow(header)
                        w.writerows(rows)
        return results

    @classmethod
    def entrypoint(cls, task: str, kernels: Sequence[KernelExecutor], dims: Dict[str, Tuple[Any, str]],
                   argv: Optional[Sequence[str]] = None):
        parser = ArgumentParser(description="Benchmark the gfx950 kernels.", formatter_class=ArgumentDefaultsHelpFormatter)
        subparsers = parser.add_subparsers(help="Sub-commands", dest="command", required=True)
        benchmark = subparsers.add_parser("benchmark", help="Benchmark kernels")
        benchmark.set_defaults(endpoint=Endpoint.BENCHMARK)
        profile = subparsers.add_parser("profile", help="Profile kernels")
        profile.set_defaults(endpoint=Endpoint.PROFILE)
        providers = [p.provider for p in kernels]
        for sub in (benchmark, profile):
            sub.add_argument("-p", "--providers", type=str, nargs="+", default=providers, choices=providers, help="Providers to evaluate.")
            sub.add_argument("-m", "--modes", type=Mode, nargs="+", default=[Mode.FORWARD], choices=list(Mode), help="Modes to evaluate.")
            sub.add_argument("-d", "--dtypes", type=Dtype, nargs="+", default=[Dtype.FP16], choices=list(Dtype), help="Data types to evaluate.")
            sub.add_argument("-w", "--warmup", type=int, default=20, help="Warmup repetitions.")
            sub.add_argument("--device", type=str, default="cuda", help="Device to use for benchmarking or profiling.")
            for name, (values, mode) in dims.items():
                DimConfig.add_argument(sub, name, values, mode)
        default_dim = next(iter(dims.keys()))
        benchmark.add_argument("-l", "--line-arg", type=str, default="kernel", choices=["kernel", "dtype", "mode"] + list(dims.keys()), help="Line argument")
        benchmark.add_argument("-x", "--x-dim", type=str, default=default_dim, choices=list(dims.keys()), help="Dimension to use as table X axis")
        benchmark.add_argument("--x-label", type=str, default="Input Size", help="Label for the x axis.")
        benchmark.add_argument("-r", "--rep", type=int, default=100, help="Number of repetitions.")
        benchmark.add_argument("-o", "--output", type=Path, default=None, help="Output directory")
        args = parser.parse_args(argv)

        parsed_dims = [DimConfig.from_namespace(args, name) for name in dims.keys()]
        chosen = [k for k in kernels if k.provider in args.providers]
        for kernel in chosen:
            kernel.rep = getattr(args, "rep", 100)
            kernel.warmup = args.warmup
        cli = cls(task, chosen, parsed_dims, [Mode(m) for m in args.modes], [Dtype(d) for d in args.dtypes],
                  getattr(args, "x_label", "Input size"), output=getattr(args, "output", None),
                  line_arg=getattr(args, "line_arg", "kernel"), x_dim=getattr(args, "x_dim", default_dim), device=args.device)
        return cli(args.endpoint)


def _format_table(header: Sequence[str], rows: Sequence[Sequence[float]]) -> str:
    cells = [list(header)] + [[f"{v:.6g}" for v in r] for r in rows]
    widths = [max(len(r[i]) for r in cells) for i in range(len(header))]
    return "\n".join("  ".join(c.rjust(w) for c, w in zip(r, widths)) for r in cells)


def median_ms(values: Sequence[float]) -> float:
    return statistics.median(values)


if __name__ == "__main__":  # pragma: no cover
    print(__doc__)
    sys.exit(0)
