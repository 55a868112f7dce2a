"""bench.py prints one JSON line with the fields the driver reads, and refuses more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in (r.stdout + r.stderr)


def test_traffic_figures_come_from_the_committed_profile_summary():
    sys.path.insert(0, ROOT)
    import bench
    table = bench.measured_traffic()
    text = open(os.path.join(ROOT, bench.TRAFFIC_SOURCE)).read()
    assert "rocprofv3 --pmc FETCH_SIZE" in text and "rocprofv3 --pmc WRITE_SIZE" in text    # the commands that made it
    for w, target in bench.SUMMARY.items():
        assert w in bench.WORKLOADS
        if target is not None:
            assert w in table, f"{w}: a workload with a roofline target needs a counter row in {bench.TRAFFIC_SOURCE}"
    for w, row in table.items():
        assert w in bench.WORKLOADS, w
        assert f"| {row['traffic']} |" in text                      # the very figure the summary states
        # no wasted re-reads: within 2 % of the algorithmic bytes, except the flat unpack (a counter artefact the summary
        # explains) and the transposing copies of rows that start inside cache lines, which re-read by design
        limit = 1.1 if w.startswith("tr_") and "8200" in w else 1.02
        assert (0.95 if w.startswith("c5_flat_unpack") else 0.999) < row["traffic"] / row["algorithmic"] < limit, (w, row)
    assert table["c2"]["algorithmic"] == 9 * 25_165_824 * 2 and table["c3_pack"]["algorithmic"] == 2 * 4096 * 14336 * 2


@pytest.mark.gpu
def test_default_bench_line():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "1", "--steps", "10", "--warmup", "3"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [ln for ln in r.stdout.splitlines() if ln.startswith("{")]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 10 and rec["warmup"] == 3 and rec["vs_baseline"] is None
    assert rec["unit"] == "GB/s" and rec["higher_is_better"] is True and rec["data"] == "synthetic"
    assert rec["config"]["workload"] == "c2_bf16_bucket_reduce_avg8" and "model" not in rec["config"]
    roof = rec["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9 and 0.3 < roof["frac"] < 1.0
    assert abs(rec["config"]["algorithmic_bytes_per_step"] - 9 * 25_165_824 * 2) == 0
    assert 0.9 < roof["traffic"] / rec["config"]["algorithmic_bytes_per_step"] < 1.1
    cpu = rec["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] == 1 and cpu["unit"] == "GB/s" and cpu["value"] > 0
    assert cpu["sample"] and cpu["all_cores"]["cores"] >= 1
    # wall-clock throughput cannot exceed the kernel-time throughput by more than timer noise
    assert rec["value"] <= roof["achieved"] * 1.10
    # the headline says how long its buffer rotation is, whether the Infinity Cache helps it, and what the same kernel does cold
    assert roof["rotation_bytes"] >= 3 * 9 * 25_165_824 * 2 and roof["cache_assisted"] is False
    assert 0.3 < roof["frac_cold"] <= roof["frac"] * 1.03
    # every class of the path is reported in the same line, measured in the same process, short enough for a reader
    # that keeps only the last 8 KB of output, rows that carry a target last
    assert len(lines[0]) < 7000, len(lines[0])
    sys.path.insert(0, ROOT)
    import bench
    wl = rec["workloads"]
    assert sorted(wl) == sorted(bench.SUMMARY)
    names = list(wl)
    first_target = min(i for i, w in enumerate(names) if bench.SUMMARY[w] is not None)
    assert all(bench.SUMMARY[w] is not None for w in names[first_target:])
    for w, e in wl.items():
        floor = 0.0 if w.startswith("c1_") else 0.2    # configuration 1 moves 1 MiB per call: launch-bound
        assert e["ms"] > 0 and abs(e["frac"] - e["bytes"] / (e["ms"] * 1e-3) / 8e12) < 2e-3 * e["frac"] and floor < e["frac"] < 1.0, (w, e)
        assert e["target"] == bench.SUMMARY[w] and e["bytes"] > 0 and e["rot_mb"] > 0
        if e["traffic_x"] is not None:
            assert 0.9 < e["traffic_x"] < 1.1, (w, e)
        assert e.get("cache_assisted", False) == (e["rot_mb"] < 512 or w in bench.PIPELINES), (w, e)
    assert abs(wl["c2"]["frac"] - roof["frac"]) < 1e-3 and wl["c2_cold"]["frac"] == roof["frac_cold"]
    assert wl["c3_reshard_e2e"]["cache_assisted"] is True and "cache_assisted" not in wl["c2_cold"]
    for w in ("c4", "c5_quantize"):
        assert wl[w]["cpu"]["torch"] > 0 and wl[w]["cpu"]["port"] > 0
