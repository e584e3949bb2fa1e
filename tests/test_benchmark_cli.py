"""The benchmark command line (reference triton_helpers/benchmark.py, layers/*/__main__.py; its tests: tests/test_benchmark.py).

CPU part: argument parsing, dimension sweeps, the three mode closures, table / CSV layout with a stub executor and a
stubbed timer.  GPU part: the two layers' entry points run a small sweep in every mode and write their CSV files.
"""
import csv

import pytest
import torch

from triton_helpers_amd import benchmark as B


class _Stub(B.KernelExecutor):
    calls = []

    def prepare_inputs(self, L, D, requires_grad=False, **kwargs):
        return {"x": torch.ones(L, D, requires_grad=requires_grad), "scale": 2.0}

    def forward(self, x, scale):
        _Stub.calls.append(("forward", tuple(x.shape), x.requires_grad))
        return x * scale


def test_dim_config_modes():
    assert list(B.DimConfig.from_range("L", 2, 10, 4)) == [2, 6, 10]
    assert list(B.DimConfig.from_range("L", 4, 6, 3, logspace=True)) == [16, 32, 64]
    assert [str(m) for m in B.Mode] == ["fwd", "bwd", "fwd-bwd"] and B.Mode("fwd-bwd").long_name == "Forward-Backward"
    assert B.Dtype("bf16").torch == torch.bfloat16


def test_mode_closures_follow_the_reference():
    """fwd: inputs without grad, forward only; bwd: one forward up front, the closure only back-propagates a fixed
    gradient; fwd-bwd: both per call (reference benchmark.py:189-215)."""
    k = _Stub("stub")
    _Stub.calls.clear()
    k._get_closure(B.Mode.FORWARD, L=3, D=2, dtype=torch.float32)()
    assert _Stub.calls == [("forward", (3, 2), False)]
    _Stub.calls.clear()
    f = k._get_closure(B.Mode.BACKWARD, L=3, D=2, dtype=torch.float32)
    assert len(_Stub.calls) == 1 and _Stub.calls[0][2] is True
    f(), f()
    assert len(_Stub.calls) == 1
    _Stub.calls.clear()
    f = k._get_closure(B.Mode.FORWARD_BACKWARD, L=3, D=2, dtype=torch.float32)
    f(), f()
    assert len(_Stub.calls) == 2


def test_cli_sweep_and_csv(tmp_path, monkeypatch):
    timed = []

    def fake_bench(fn, warmup, rep, quantiles, clear_l2=True):
        fn()
        timed.append((warmup, rep))
        return (1.0, 0.5, 2.0)

    monkeypatch.setattr(B, "do_bench", fake_bench)
    res = B.CLI.entrypoint(
        "Stub task", [_Stub("stub-a"), _Stub("stub-b")], dims={"L": ((4, 8), "values"), "D": (2, "values")},
        argv=["benchmark", "-m", "fwd", "bwd", "-d", "fp32", "-L", "2", "4", "3", "--L-mode", "logspace", "-w", "7", "-r", "9", "-o", str(tmp_path)])
    # one table per (mode, dtype, D), lines = kernels, x = L in {4, 8, 16}
    assert [r[0] for r in res] == ["Stub task-fwd-D=2-fp32", "Stub task-bwd-D=2-fp32"]
    for name, header, rows in res:
        assert header == ["L", "Stub-A", "Stub-A-min", "Stub-A-max", "Stub-B", "Stub-B-min", "Stub-B-max"]
        assert [r[0] for r in rows] == [4.0, 8.0, 16.0] and all(r[1:] == [1.0, 0.5, 2.0] * 2 for r in rows)
        with open(tmp_path / f"{name}.csv") as f:
            got = list(csv.reader(f))
        assert got[0] == header and len(got) == 4
    assert len(timed) == 2 * 2 * 3 and set(timed) == {(7, 9)}
    # line argument = mode: one table per (kernel, dtype, D)
    res = B.CLI.entrypoint("T", [_Stub("only")], dims={"L": (4, "values"), "D": ((2, 3), "values")},
                           argv=["benchmark", "-m", "fwd", "fwd-bwd", "-l", "mode"])
    assert [r[0] for r in res] == ["T-Only-D=2-fp16", "T-Only-D=3-fp16"]
    assert res[0][1] == ["L", "Forward", "Forward-min", "Forward-max", "Forward-Backward", "Forward-Backward-min", "Forward-Backward-max"]
    with pytest.raises(SystemExit):
        B.CLI.entrypoint("T", [_Stub("only")], dims={"L": (4, "values")}, argv=["benchmark", "-m", "sideways"])
    with pytest.raises(NotADirectoryError):
        B.CLI("T", [_Stub("only")], [B.DimConfig("L", [1])], output=tmp_path / "missing")


def test_alias_modules_exist():
    import triton_helpers.benchmark as alias
    from triton_helpers.layers.fully_fused_mlp.__main__ import main as m1
    from triton_helpers.layers.hash_encoding.__main__ import main as m2

    assert alias.CLI is B.CLI and callable(m1) and callable(m2)


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
    assert [r[0] for r in res] == ["MLP-fwd-D=64-H=1-bf16", "MLP-fwd-D=64-H=3-bf16", "MLP-fwd-bwd-D=64-H=1-bf16", "MLP-fwd-bwd-D=64-H=3-bf16"]
    for name, header, rows in res:
        assert header[1] == "Baseline" and header[4] == "Fully-Fused" and rows[0][1] > 0 and rows[0][4] > 0
    # profile: one ranged call per combination, no timing
    res = mlp_main(["profile", "-m", "fwd", "-d", "bf16", "-L", "256", "-H", "1", "-w", "1", "-p", "fully-fused"])
    assert len(res) == 1
