"""GPU: the benchmark's one-line JSON keeps the keys its readers depend on (short runs of the real script)."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = [pytest.mark.gpu, pytest.mark.timeout(400)]
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*flags: str) -> dict:
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], capture_output=True, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [l for l in res.stdout.splitlines() if l.startswith("{")]
    assert len(lines) == 1, res.stdout[-2000:]
    return json.loads(lines[0])


def check_roofline(r: dict, bound: str) -> None:
    assert r["bound"] == bound and r["unit"] in ("GB/s", "TOP/s")
    assert r["achieved"] > 0 and r["peak"] > 0
    assert abs(r["frac"] - r["achieved"] / r["peak"]) < 1e-3
    assert "traffic" in r and r["avg_launch_us"] > 0


def test_headline_line_short_run():
    d = run_bench("--steps", "40", "--warmup", "4", "--layers", "2", "--no-decode", "--cpu-seconds", "0.5")
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in d, key
    assert d["n_gpus"] == 1 and d["steps"] == 40 and d["warmup"] == 4 and d["unit"] == "GB/s" and d["higher_is_better"] is True
    assert d["vs_baseline"] is None and d["data"] == "synthetic" and "workload" in d["config"] and d["config"]["outputs_finite"] is True
    assert abs(d["value"] - d["config"]["bytes_per_step"] / (d["ms_per_step"] * 1e-3) / 1e9) < 0.01 * d["value"]
    check_roofline(d["roofline"], "hbm")
    c = d["cpu_baseline"]
    assert c["kind"] == "port" and c["cores"] >= 1 and c["value"] > 0 and c["unit"] == "GB/s" and c["sample"] and c["single_thread"]["cores"] == 1


@pytest.mark.parametrize("workload,bound", [("quantize", "hbm"), ("get_rows", "hbm"), ("f32act", "hbm"), ("prefill", "mfma")])
def test_side_workload_lines(workload, bound):
    d = run_bench("--workload", workload, "--steps", "20", "--warmup", "2")
    assert d["n_gpus"] == 1 and d["value"] > 0 and d["ms_per_step"] > 0 and "workload" in d["config"]
    check_roofline(d["roofline"], bound)
