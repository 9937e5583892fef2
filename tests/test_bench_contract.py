"""The measurement script's contract: one JSON line with the fields the driver reads,
a roofline object for the dominant kernel, a CPU baseline object, and a refusal of
more than one GPU."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _run(args, timeout):
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py")] + args, cwd=ROOT,
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=timeout)


def test_more_than_one_gpu_is_refused():
    proc = _run(["--gpus", "2"], 120)
    assert proc.returncode != 0
    assert "one GPU" in (proc.stdout + proc.stderr)


@pytest.mark.gpu
def test_default_workload_prints_the_contract_line():
    proc = _run(["--steps", "2", "--warmup", "1", "--stage-reps", "2", "--cpu-sample", "2"], 600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [ln for ln in proc.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    out = json.loads(lines[0])
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                "scaling", "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline"):
        assert key in out, key
    assert out["n_gpus"] == 1 and out["steps"] == 2 and out["warmup"] == 1
    assert out["unit"] == "TFLOP/s" and out["dtype"] == "f32" and out["vs_baseline"] is None
    assert out["higher_is_better"] is True and out["value"] > 0
    assert "workload" in out["config"] and "model" not in out["config"]
    roof = out["roofline"]
    assert roof["bound"] in ("hbm", "mfma") and roof["unit"] in ("GB/s", "TFLOP/s")
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-3
    assert roof["peak"] == 157.3 and roof["traffic"] > 0
    # the roofline figure is clocked inside real steps; every stage carries that clock and,
    # with --stage-reps > 0, the back-to-back one as well
    assert "inside" in roof["timing"] and roof["avg_launch_ms"] > 0
    for row in out["stages"]:
        assert row["ms_in_step"] > 0 and row["ms"] > 0 and 0 < row["frac_in_step"] < 1.2
    cpu = out["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    assert out["parity"]["ok"] is True


@pytest.mark.gpu
def test_in_step_clock_alone():
    # --stage-reps 0: only the in-step clock; the roofline figure still comes out
    proc = _run(["--steps", "2", "--warmup", "1", "--stage-reps", "0", "--no-cpu", "--no-op-api",
                 "--workload", "cifar_conv2_5x5_32x15x15_b128"], 600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads([ln for ln in proc.stdout.splitlines() if ln.strip()][0])
    assert out["roofline"]["achieved"] > 0 and "inside" in out["roofline"]["timing"]
    for row in out["stages"]:
        assert row["ms_in_step"] > 0 and "ms" not in row
