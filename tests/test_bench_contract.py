"""Host-side checks of bench.py (no GPU): where the counter-derived figures of the JSON line come from, and what the
script does when asked for more than one GPU."""
import subprocess
import sys

import bench


def test_counter_figures_belong_to_the_named_kernel_and_duration():
    """``roofline.traffic`` / ``roofline.l2`` cannot be measured in the run: they are quoted from the committed profile
    summary only while that summary names the kernel the run launches and a duration within 10 % of the run's."""
    figs, source = bench.profile_figures("hash_fwd_sweep_k", 0.001)
    assert figs == {} and "stale" in source  # a launch of 1 us is no kernel of that summary
    figs, source = bench.profile_figures("some_other_kernel", 0.33)
    assert figs == {} and "some_other_kernel" in source
    import re

    text = open(bench.PROFILE_SUMMARY).read()
    m = re.search(r"kernel=(\S+)\s+kernel_us=([0-9.]+)", text)
    assert m, "the profile summary holds a bench-figures line with its kernel and duration"
    figs, source = bench.profile_figures(m.group(1), float(m.group(2)) * 1e-3)
    assert figs["fwd_traffic_bytes"] > 1e8 and figs["fwd_l2_read_requests"] > 1e7
    assert "rocprofv3" in source and m.group(1) in source
    # the figures are the ones of the summary's own tables: fetched x 2.0 + written, in bytes
    fetch = re.search(r"hash_fwd_sweep_k<[^|]*\|\s*(\d+)\s*\|\s*\d+\s*\|\s*(\d+)\s*\|", text)
    assert fetch, "HBM traffic table of the forward kernel"
    want = (int(fetch.group(1)) * 2.0 + int(fetch.group(2))) * 1024
    assert abs(figs["fwd_traffic_bytes"] - want) <= 0.01 * want


def test_quantiles_are_the_reference_statistics():
    q = bench.quantiles([5.0, 1.0, 2.0, 4.0, 3.0])
    assert q["median"] == 3.0 and q["n"] == 5 and q["p20"] <= q["median"] <= q["p80"]


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, bench.__file__, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert r.returncode != 0
    assert "one GPU" in (r.stdout + r.stderr) or "--gpus" in (r.stdout + r.stderr)
