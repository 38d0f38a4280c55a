"""bench.py's command line: defaults that finish within minutes, and the refusal of more than one GPU (this build has
no multi-GPU path).  The JSON line itself is checked on the GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused_with_a_message():
    res = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_defaults():
    sys.path.insert(0, ROOT)
    import bench
    argv, sys.argv = sys.argv, ["bench.py"]
    try:
        args = bench.parse()
    finally:
        sys.argv = argv
    assert args.gpus == 1 and args.steps >= 1 and args.warmup >= 1


@pytest.mark.gpu
def test_json_line_has_the_contract_fields(device):
    res = subprocess.run([sys.executable, BENCH, "--steps", "40", "--warmup", "5", "--no-extras", "--no-cpu"],
                         capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stderr[-2000:]
    line = json.loads(res.stdout.strip().splitlines()[-1])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 40 and line["warmup"] == 5 and line["unit"] == "TFLOP/s"
    assert line["vs_baseline"] is None and "workload" in line["config"] and "model" not in line["config"]
    roof = line["roofline"]
    assert roof["bound"] == "mfma" and abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    # value = flops of the step / time of the step
    assert abs(line["value"] - line["config"]["flops_per_step"] / (line["ms_per_step"] * 1e-3) / 1e12) < 0.02 * line["value"]
