"""The benchmark's command line and the shape of its one JSON line.

CPU part: more than one GPU is refused with a message (every box of this build has one GPU) before anything touches a
device.  GPU part: a short run of one workload prints exactly one JSON line with the fields the driver reads, the
`roofline` and `cpu_baseline` objects, and figures that are consistent with each other."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(*flags, timeout=600):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *flags], cwd=ROOT, stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=timeout)


def test_more_than_one_gpu_is_refused():
    res = _run("--gpus", "2")
    assert res.returncode == 2
    assert "one GPU" in res.stderr and res.stdout.strip() == ""


def test_unknown_workload_is_refused():
    res = _run("--workload", "c9")
    assert res.returncode != 0 and "invalid choice" in res.stderr


@pytest.mark.gpu
def test_json_line_of_a_short_run():
    res = _run("--gpus", "1", "--steps", "3", "--warmup", "1", "--settle-steps", "2", "--kernel-reps", "10", "--workload", "c1",
               "--no-cache-variants")
    assert res.returncode == 0, res.stderr[-2000:]
    lines = [l for l in res.stdout.splitlines() if l.strip()]
    assert len(lines) == 1, lines
    line = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "workloads"):
        assert key in line, key
    assert line["n_gpus"] == 1 and line["steps"] == 3 and line["warmup"] == 1 and line["settle_steps"] == 2
    assert line["higher_is_better"] is True and line["vs_baseline"] is None
    assert "workload" in line["config"] and "model" not in line["config"]
    roof = line["roofline"]
    assert roof["bound"] in ("hbm", "mfma") and roof["unit"] in ("GB/s", "TFLOP/s", "TOP/s")
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert 0.0 < roof["frac"] < 1.0
    cpu = line["cpu_baseline"]
    assert cpu["kind"] == "port" and cpu["cores"] == 1 and cpu["value"] > 0 and "sample" in cpu
    (w,) = line["workloads"]
    assert w["config"] == "C1" and w["kernel"].startswith("mtrt_dynqdq_f32_i8")
    # value = ideal time of the step's kernels / measured step time, in per cent
    ideal_ms = w["work"] / (w["peak"] * 1e3) / 1e3
    assert abs(line["value"] - 100.0 * ideal_ms / line["ms_per_step"]) < 0.05 * line["value"] + 0.01
