"""The benchmark command line (reference triton_helpers/benchmark.py, layers/*/__main__.py; its tests: tests/test_benchmark.py).

CPU part: argument parsing, axis sweeps, the three timed closures, table / CSV layout with a stub workload and a
stubbed timer.  GPU part: the two layers' entry points run a small sweep in every mode and write their CSV files.
"""
import csv

import pytest
import torch

from triton_helpers_amd import benchmark as B

CALLS = []


def _stub_inputs(L, D, device="cpu", dtype=torch.float32, requires_grad=False):
    return {"x": torch.ones(L, D, dtype=dtype, requires_grad=requires_grad), "scale": 2.0}


def _stub_run(x, scale):
    CALLS.append(("forward", tuple(x.shape), x.requires_grad))
    return x * scale


def _stub(name):
    return B.Workload(name, _stub_inputs, _stub_run)


def test_axis_modes_and_names():
    assert B.axis_values([2, 10, 4], "linspace") == [2, 6, 10]
    assert B.axis_values([4, 6, 3], "logspace") == [16, 32, 64]
    assert B.axis_values([5, 7], "values") == [5, 7]
    with pytest.raises(ValueError):
        B.axis_values([1, 2], "linspace")
    assert list(B.MODES) == ["fwd", "bwd", "fwd-bwd"] and B.MODES["fwd-bwd"] == "Forward-Backward"
    assert B.DTYPES["bf16"] == torch.bfloat16 and _stub("stub-a").title == "Stub-A"


def test_timed_closures_follow_the_reference():
    """fwd: inputs without grad, forward only; bwd: one forward up front, the closure only back-propagates a fixed
    gradient; fwd-bwd: both per call (reference benchmark.py:189-215)."""
    k = _stub("stub")
    CALLS.clear()
    B.step_closure(k, "fwd", torch.float32, "cpu", {"L": 3, "D": 2})()
    assert CALLS == [("forward", (3, 2), False)]
    CALLS.clear()
    f = B.step_closure(k, "bwd", torch.float32, "cpu", {"L": 3, "D": 2})
    assert len(CALLS) == 1 and CALLS[0][2] is True
    f(), f()
    assert len(CALLS) == 1
    CALLS.clear()
    f = B.step_closure(k, "fwd-bwd", torch.float32, "cpu", {"L": 3, "D": 2})
    f(), f()
    assert len(CALLS) == 2
    with pytest.raises(ValueError):
        B.step_closure(k, "sideways", torch.float32, "cpu", {"L": 3, "D": 2})


def test_cli_sweep_and_csv(tmp_path, monkeypatch):
    timed = []

    def fake_timer(fn, warmup_ms, rep_ms, cold=True):
        fn()
        timed.append((warmup_ms, rep_ms))
        return B.Timing(1.0, 0.5, 2.0)

    monkeypatch.setattr(B, "time_calls", fake_timer)
    res = B.run_cli(
        "Stub task", [_stub("stub-a"), _stub("stub-b")], dims={"L": ((4, 8), "values"), "D": (2, "values")},
        argv=["benchmark", "-m", "fwd", "bwd", "-d", "fp32", "-L", "2", "4", "3", "--L-mode", "logspace", "-w", "7", "-r", "9", "-o", str(tmp_path),
              "--device", "cpu"])
    # one table per (mode, dtype, D), lines = kernels, x = L in {4, 8, 16}
    assert [r.name for r in res] == ["Stub task-fwd-D=2-fp32", "Stub task-bwd-D=2-fp32"]
    for name, header, rows in res:
        assert header == ["L", "Stub-A", "Stub-A-min", "Stub-A-max", "Stub-B", "Stub-B-min", "Stub-B-max"]
        assert [r[0] for r in rows] == [4.0, 8.0, 16.0] and all(r[1:] == [1.0, 0.5, 2.0] * 2 for r in rows)
        with open(tmp_path / f"{name}.csv") as f:
            got = list(csv.reader(f))
        assert got[0] == header and len(got) == 4
    assert len(timed) == 2 * 2 * 3 and set(timed) == {(7, 9)}
    # line argument = mode: one table per (kernel, dtype, D)
    res = B.run_cli("T", [_stub("only")], dims={"L": (4, "values"), "D": ((2, 3), "values")},
                    argv=["benchmark", "-m", "fwd", "fwd-bwd", "-l", "mode", "--device", "cpu"])
    assert [r.name for r in res] == ["T-Only-D=2-fp16", "T-Only-D=3-fp16"]
    assert res[0].header == ["L", "Forward", "Forward-min", "Forward-max", "Forward-Backward", "Forward-Backward-min", "Forward-Backward-max"]
    # a swept dimension as the line argument
    res = B.run_cli("T", [_stub("only")], dims={"L": (4, "values"), "D": ((2, 3), "values")}, argv=["benchmark", "-l", "D", "--device", "cpu"])
    assert [r.name for r in res] == ["T-Only-fwd-fp16"] and res[0].header[1::3] == ["D=2", "D=3"]
    with pytest.raises(SystemExit):
        B.run_cli("T", [_stub("only")], dims={"L": (4, "values")}, argv=["benchmark", "-m", "sideways"])
    with pytest.raises(NotADirectoryError):
        B.sweep("T", [_stub("only")], {"L": [1]}, ["fwd"], ["fp16"], "L", output=tmp_path / "missing")


def test_alias_modules_exist():
    import triton_helpers.benchmark as alias
    from triton_helpers.layers.fully_fused_mlp.__main__ import main as m1
    from triton_helpers.layers.hash_encoding.__main__ import main as m2

    assert alias.run_cli is B.run_cli and callable(m1) and callable(m2)


@pytest.mark.gpu
def test_layer_entry_points_run_every_mode(tmp_path):
    from triton_helpers_amd.layers.fully_fused_mlp.__main__ import main as mlp_main
    from triton_helpers_amd.layers.hash_encoding.__main__ import main as hash_main

    res = hash_main(["benchmark", "-m", "fwd", "bwd", "fwd-bwd", "-d", "fp16", "fp32", "-L", "64", "2048", "-w", "2", "-r", "5", "-o", str(tmp_path)])
    assert len(res) == 6
    for name, header, rows in res:
        assert header[:2] == ["L", "Hip-Hash"] and len(rows) == 2
        assert all(r[1] > 0 and r[2] <= r[1] <= r[3] for r in rows), (name, rows)
        assert (tmp_path / f"{name}.csv").exists()
    res = mlp_main(["benchmark", "-m", "fwd", "fwd-bwd", "-d", "bf16", "-L", "256", "-H", "1", "3", "-l", "kernel", "-w", "2", "-r", "5"])
    assert [r.name for r in res] == ["MLP-fwd-D=64-H=1-bf16", "MLP-fwd-D=64-H=3-bf16", "MLP-fwd-bwd-D=64-H=1-bf16", "MLP-fwd-bwd-D=64-H=3-bf16"]
    for name, header, rows in res:
        assert header[1] == "Baseline" and header[4] == "Fully-Fused" and rows[0][1] > 0 and rows[0][4] > 0
    # profile: one ranged call per combination, no timing
    res = mlp_main(["profile", "-m", "fwd", "-d", "bf16", "-L", "256", "-H", "1", "-w", "1", "-p", "fully-fused"])
    assert len(res) == 1
