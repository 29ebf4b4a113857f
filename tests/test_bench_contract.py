"""bench.py's command-line contract: one JSON line with the metric, the roofline of the dominant kernel and the CPU baseline;
more than one GPU is refused with a message."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_more_than_one_gpu_is_refused():
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert p.returncode == 2 and "one GPU" in p.stderr and not p.stdout.strip()


@pytest.mark.gpu
def test_bench_line_of_the_tiny_workload():
    """The smallest workload through the whole bench path: tuning, timed region, per-dispatch events, parity against the oracle."""
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--workload", "tiny_128", "--steps", "20", "--warmup", "5"],
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    lines = [l for l in p.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1
    d = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 20 and d["warmup"] == 5 and d["unit"] == "Mpix/s" and d["dtype"] == "f16" and d["vs_baseline"] is None
    assert d["value"] > 0 and abs(d["value"] - 128 * 128 / (d["ms_per_step"] * 1e-3) * 1e-6) < 1e-6 * d["value"]
    assert "workload" in d["config"] and "model" not in d["config"]
    r = d["roofline"]
    assert r["bound"] in ("hbm", "mfma") and r["peak"] == 2500.0 and abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-9 and "traffic" in r
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and "sample" in c
    # outputs of this network stay below 2: the stated bar itself has to hold
    assert d["parity"]["ok"] and d["parity"]["meets_stated_bar"] and d["parity"]["max_abs"] <= 2e-2 and d["parity"]["mean_abs"] <= 2e-3
    assert "other_workloads" not in d  # only the headline workload appends the others
