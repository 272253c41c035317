"""The command-line contract of bench.py: one JSON line with the agreed keys; more than one GPU is refused."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          cwd=ROOT, timeout=600)


def test_more_than_one_gpu_is_refused_with_a_message():
    res = run_bench("--gpus", "2")
    assert res.returncode != 0 and "one GPU" in res.stderr and res.stdout.strip() == ""


@pytest.mark.gpu
def test_default_workload_prints_one_json_line_with_roofline_and_cpu_baseline():
    res = run_bench("--steps", "3", "--warmup", "1", "--cpu-rows", "128")
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [ln for ln in res.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 3 and out["warmup"] == 1 and out["vs_baseline"] is None
    assert out["config"]["workload"] == "dwn_k6_b4096_i16384_n8192" and out["dtype"] == "f32"
    roof = out["roofline"]
    assert roof["bound"] == "hbm" and roof["unit"] == "GB/s" and roof["peak"] == 8000.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-12 and roof["achieved"] > 0
    cpu = out["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and "sample" in cpu
    assert out["value"] > cpu["value"]
