"""bench.py's command line contract that can be checked without a GPU, and (on
a GPU) the shape of the JSON line on a small workload."""

import json
import subprocess
import sys
from pathlib import Path

import pytest

REPO_ROOT = Path(__file__).resolve().parent.parent


def run_bench(*args, timeout=600):
    return subprocess.run([sys.executable, str(REPO_ROOT / "bench.py"), *args],
                          capture_output=True, text=True, timeout=timeout)


def test_more_than_one_gpu_is_refused_with_a_message():
    result = run_bench("--gpus", "2")
    assert result.returncode != 0
    assert "one GPU" in result.stderr and result.stdout.strip() == ""


@pytest.mark.gpu
@pytest.mark.parametrize("gradients,contractions", [("forward", 3), ("recompute", 4)])
def test_json_line_on_a_small_workload(gpu_device, gradients, contractions):
    result = run_bench("--workload", "small_head", "--steps", "3", "--warmup", "1",
                       "--cpu-rows", "64", "--no-library-gemm", "--gradients", gradients)
    assert result.returncode == 0, result.stderr[-2000:]
    lines = [line for line in result.stdout.splitlines() if line.startswith("{")]
    assert len(lines) == 1
    record = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step",
                "higher_is_better", "scaling", "vs_baseline", "dtype", "data", "config",
                "roofline", "cpu_baseline"):
        assert key in record, key
    assert record["n_gpus"] == 1 and record["steps"] == 3 and record["warmup"] == 1
    assert record["vs_baseline"] is None and record["higher_is_better"] is True
    assert "workload" in record["config"] and "model" not in record["config"]
    assert record["config"]["gradients"] == gradients
    assert record["contractions_executed"] == contractions
    assert record["forward_only_ms"] > 0 and record["backward_only_ms"] > 0
    roofline = record["roofline"]
    assert roofline["bound"] == "mfma" and roofline["unit"] == "TFLOP/s"
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-9
    baseline = record["cpu_baseline"]
    assert baseline["kind"] == "port" and baseline["cores"] >= 1 and baseline["value"] > 0
