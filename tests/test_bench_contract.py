"""The contract of bench.py: one JSON line on stdout with the agreed fields, and a refusal of
more than one GPU (this build measures one GPU)."""

import json
import pathlib
import subprocess
import sys

import pytest

ROOT = pathlib.Path(__file__).resolve().parent.parent


def test_more_than_one_gpu_is_refused_with_a_message():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert run.returncode != 0
    assert run.stdout.strip() == ""
    assert "one GPU" in run.stderr and "--gpus 1" in run.stderr


@pytest.mark.gpu
def test_one_json_line_with_roofline_and_cpu_baseline():
    run = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "1", "--steps", "4", "--warmup", "2", "--skip-kernels",
                          "--replays", "5"], capture_output=True, text=True, timeout=900)
    assert run.returncode == 0, run.stderr[-2000:]
    lines = [line for line in run.stdout.splitlines() if line.strip()]
    assert len(lines) == 1
    result = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in result, key
    assert result["n_gpus"] == 1 and result["steps"] == 4 and result["warmup"] == 2
    assert result["higher_is_better"] is True and result["vs_baseline"] is None and result["unit"] == "GB/s"
    assert "workload" in result["config"] and "model" not in result["config"]
    # the step is the metric's configuration: ONE mk_packed_matvec call on one 4096 x 14336 matrix at M=1, and
    # the other row counts of the metric ride in the same record as flat scalars
    config = result["config"]
    assert config["matrices_per_step"] == 1 and "one mk_packed_matvec call" in config["workload"]
    assert abs(config["us_M1"] - result["ms_per_step"] * 1e3) < 1e-3 * config["us_M1"]
    assert result["roofline"]["algorithmic_bytes_per_launch"] == 30_314_496
    for samples in (1, 2, 4, 8):
        assert config[f"us_M{samples}"] > 0 and 0 < config[f"frac_M{samples}"] < 1
        assert config[f"group_of_8_us_per_matrix_M{samples}"] > 0
    roofline = result["roofline"]
    assert roofline["bound"] == "hbm" and roofline["peak"] == 8000.0 and roofline["unit"] == "GB/s"
    assert abs(roofline["frac"] - roofline["achieved"] / roofline["peak"]) < 1e-4      # the line keeps five digits
    assert 0.2 < roofline["frac"] < 1.0
    # whole-job throughput: algorithmic bytes per step over the step time
    assert abs(result["value"] - roofline["algorithmic_bytes_per_launch"] / (result["ms_per_step"] * 1e-3) / 1e9) < 0.02 * result["value"]
    baseline = result["cpu_baseline"]
    assert baseline["kind"] in ("port", "reference") and baseline["cores"] >= 1 and baseline["value"] > 0 and baseline["sample"]
