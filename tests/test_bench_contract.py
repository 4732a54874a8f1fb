"""The benchmark's contract with its driver: one JSON line with the agreed keys, one GPU only."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "ONE GPU" in r.stderr and r.stdout.strip() == ""


@pytest.mark.gpu
def test_bench_prints_one_json_line_with_the_contract_keys():
    r = subprocess.run([sys.executable, BENCH, "--steps", "20", "--warmup", "5", "--no-model", "--no-cpu-baseline"],
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    rec = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in rec, key
    assert rec["n_gpus"] == 1 and rec["steps"] == 20 and rec["warmup"] == 5 and rec["unit"] == "GB/s"
    assert rec["vs_baseline"] is None and rec["dtype"] == "fp16" and "workload" in rec["config"]
    roof = rec["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    # achieved = algorithmic bytes of the dominant kernel / its measured duration
    assert abs(roof["achieved"] - roof["algorithmic_bytes"] / (roof["kernel_ms"] * 1e-3) / 1e9) < 0.01 * roof["achieved"]
    # value = algorithmic bytes of a step / time of a step
    assert abs(rec["value"] - rec["config"]["algorithmic_bytes_per_step"] / (rec["ms_per_step"] * 1e-3) / 1e9) < 0.01 * rec["value"]
    assert 0.2 < roof["frac"] < 1.0
