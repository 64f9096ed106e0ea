"""The benchmark's one-line contract, on a graph shrunk to 1 % so that the whole default run takes seconds."""
import json
import os
import subprocess
import sys

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*flags, timeout=300):
    print("[case] bench.py " + " ".join(flags), flush=True)
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], cwd=ROOT, capture_output=True, text=True, timeout=timeout)


def test_default_run_prints_one_json_line_with_every_configuration():
    done = run_bench("--scale", "0.01", "--steps", "2", "--warmup", "1", "--spmm-iters", "3")
    assert done.returncode == 0, done.stderr[-2000:]
    lines = [l for l in done.stdout.splitlines() if l.strip()]
    assert len(lines) == 1  # everything else goes to stderr
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline", "side_configs"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 2 and line["warmup"] == 1 and line["dtype"] == "f32" and line["vs_baseline"] is None
    assert "workload" in line["config"] and "model" not in line["config"]
    roof = line["roofline"]
    assert roof["bound"] == "hbm" and roof["peak"] == 8000.0 and roof["unit"] == "GB/s"
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-12 and abs(roof["achieved"] - line["value"]) < 1e-9 * line["value"]
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] >= 1 and cpu["value"] > 0 and "sample" in cpu
    assert line["max_rel_err_gpu_vs_cpu"] <= 1e-5
    assert set(line["side_configs"]) == {"5", "2", "4", "1"}
    for name, side in line["side_configs"].items():
        assert side["ms_per_step"] > 0 and "workload" in side["config"], name
    assert line["side_configs"]["5"]["dtype"] == "bf16" and line["side_configs"]["5"]["max_rel_err_gpu_vs_cpu"] <= 2e-2


def test_more_than_one_gpu_is_refused_with_a_message():
    done = run_bench("--gpus", "2", timeout=120)
    assert done.returncode == 2 and "one GPU" in done.stderr
