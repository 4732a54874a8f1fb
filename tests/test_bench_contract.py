"""The benchmark's contract with its driver: one JSON line with the agreed keys, one GPU only."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")
sys.path.insert(0, ROOT)
import bench  # noqa: E402


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
    # the dominant kernel is named as the library launched it; the HBM traffic figure comes from the committed
    # profiler summary and only from a row measured on exactly that kernel
    assert roof["kernel_name"].startswith("fused_bwd_kernel<FP16, 32, 2")
    assert roof["traffic"] is None or roof["traffic"] == bench.measured_traffic("cfg2", roof["kernel_name"])
    # every configuration shape, packed and in the projection layout, forward and (where it has one) backward
    recs = {(r["name"], r["layout"]): r for r in rec["configs"]}
    assert set(recs) == {(n, l) for n in ("cfg1", "cfg2", "cfg3", "cfg4", "cfg5") for l in ("packed", "strided")}
    for (name, layout), r in recs.items():
        kernels = [r["forward"]] + ([r["backward"]] if bench.WORKLOADS[name]["bwd"] else [])
        assert (r["backward"] is not None) == bench.WORKLOADS[name]["bwd"]
        for kr in kernels:
            assert kr["kernel"] and kr["kernel_us"] > 1.0
            assert abs(kr["GBps"] - kr["algorithmic_bytes"] / kr["kernel_us"] / 1e3) < 0.01 * kr["GBps"]
            assert abs(kr["frac_of_hbm_peak"] - kr["GBps"] / 8000.0) < 1e-3 and 0.05 < kr["frac_of_hbm_peak"] < 1.0
    assert recs[("cfg2", "packed")]["backward"]["algorithmic_bytes"] == 137625600
    assert recs[("cfg3", "packed")]["forward"]["algorithmic_bytes"] == 52428800
    # the reference's two-call API, reported apart from the fused operator: 4C + 4W bytes per token and call
    unf = {r["name"]: r for r in rec["unfused"]}
    assert set(unf) == {"cfg2", "cfg3"}
    for key in ("qk_forward", "av_forward", "k_backward"):
        assert unf["cfg2"][key]["algorithmic_bytes"] == 1024 * 300 * (4 * 32 + 4 * 15)
        assert unf["cfg3"][key]["kernel_us"] > 1.0
    # the streaming-copy yardstick of the same byte volumes
    assert rec["copy_yardstick"]["cfg2 backward"]["kernel_us"] > 1.0


def test_traffic_table_is_keyed_by_workload_and_kernel(tmp_path):
    """The HBM traffic of the roofline record is read from a profiler summary, and only from the row of exactly the
    kernel that was timed: a kernel whose name changed since the summary was written gets no figure."""
    f = tmp_path / "traffic.md"
    f.write_text("| Workload | Kernel | FETCH_SIZE KiB | x | WRITE_SIZE KiB | x | note |\n|---|---|---|---|---|---|---|\n"
                 "| cfg2 | `void na1d::mfma::fused_bwd_kernel<na1d::FP16, 32, 2, false>(char*, char*)` | 1000.0 | 2.0 | 500.0 | 1.0 | |\n")
    assert bench.measured_traffic("cfg2", "fused_bwd_kernel<FP16, 32, 2, false>", str(f)) == 2500 * 1024
    assert bench.measured_traffic("cfg2", "fused_bwd_kernel<FP16, 32, 3, false>", str(f)) is None
    assert bench.measured_traffic("cfg3", "fused_bwd_kernel<FP16, 32, 2, false>", str(f)) is None
    assert bench.measured_traffic("cfg2", "x", str(tmp_path / "absent.md")) is None


def test_committed_traffic_table_parses():
    """Every data row of the committed summary yields a figure under its own workload and kernel."""
    rows = 0
    for line in open(bench.TRAFFIC_FILE):
        cells = [c.strip() for c in line.strip().strip("|").split("|")]
        if len(cells) >= 6 and cells[0].startswith("cfg"):
            assert bench.measured_traffic(cells[0], cells[1].strip("`")) > 1e6, line
            rows += 1
    assert rows >= 2
