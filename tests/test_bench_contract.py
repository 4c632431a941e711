"""bench.py's command-line contract: it measures one GPU and says so when asked for more, never falls back to the CPU,
and prints one JSON line with the agreed keys."""

import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run_bench(*args, timeout=600):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True, timeout=timeout,
                          cwd=ROOT)


def test_more_than_one_gpu_is_refused_with_a_message():
    out = run_bench("--gpus", "2", "--steps", "1", "--warmup", "0")
    assert out.returncode != 0 and out.stdout.strip() == ""
    assert "one GPU" in out.stderr


@pytest.mark.gpu
def test_one_json_line_with_the_agreed_keys():
    out = run_bench("--steps", "3", "--warmup", "2", "--skip-unet")
    assert out.returncode == 0, out.stderr[-2000:]
    lines = [ln for ln in out.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline",
                "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 3 and line["warmup"] == 2 and line["vs_baseline"] is None
    assert line["unit"] == "TFLOP/s" and line["dtype"] == "bf16" and line["data"] == "synthetic" and "workload" in line["config"]
    roof = line["roofline"]
    assert roof["bound"] == "mfma" and roof["unit"] == "TFLOP/s" and roof["peak"] == 2500.0
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9 and 0.05 < roof["frac"] < 1.0
    cpu = line["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    # value is three directions of the stated FLOPs over the step time
    flops = line["details"]["conv"]["flops_per_direction"]
    assert abs(line["value"] - 3 * flops / (line["ms_per_step"] * 1e-3) / 1e12) < 1e-6 * line["value"]
