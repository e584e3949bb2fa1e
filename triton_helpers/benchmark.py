"""Alias of ``triton_helpers_amd.benchmark`` (the benchmark / profile command line of the layers)."""
from triton_helpers_amd.benchmark import (  # noqa: F401
    DTYPES, MODES, Table, Timing, Workload, axis_values, profile_once, run_cli, step_closure, sweep, time_calls,
)
