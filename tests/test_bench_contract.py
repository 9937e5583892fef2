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


def _traffic_by_hand(workload, stage):
    """2.0 x FETCH_SIZE + 1.0 x WRITE_SIZE megabytes of the stage's sgemm launch and the reduce
    kernel behind it, read from the summaries with nothing but string splitting."""
    prefix = {"vgg_mid_conv3x3_128x56x56_b64": "vgg_mid_conv3x3_b64",
              "vgg_mid_conv3x3_128x56x56_b64/im2col": "vgg_mid_conv3x3_b64_im2col"}[workload]
    nth = [["gemm_fwd", "gemm_dgrad", "gemm_wgrad"], ["gemm_fwd_NT", "gemm_dgrad_NN", "gemm_wgrad_TN"]][
        workload.endswith("/im2col")].index(stage)
    total = 0.0
    for counter, factor in (("FETCH_SIZE", 2.0), ("WRITE_SIZE", 1.0)):
        lines = open(os.path.join(ROOT, "profiles", "%s_pmc_%s.txt" % (prefix, counter))).read().splitlines()
        assert "factor: %s" % factor in lines
        seen, take = -1, False
        for ln in lines:
            if "_kernel" not in ln or ln.startswith(("command", "kernel ")):
                continue
            if "sgemm_kernel" in ln:
                seen += 1
                take = seen == nth
            elif "reduce_" not in ln:        # splitk_reduce_kernel, tail_reduce_kernel, tail_reduce_conv_kernel
                take = False
            if take:
                total += factor * float(ln.split()[-1]) * 1e6
    return int(round(total))


def test_traffic_is_read_from_the_profile_summaries():
    import bench
    w = "vgg_mid_conv3x3_128x56x56_b64"
    t = bench.traffic_from_profiles(w + "/im2col", "im2col")
    assert set(t) == {"gemm_fwd_NT", "gemm_dgrad_NN", "gemm_wgrad_TN"}
    for stage, v in t.items():
        assert v == _traffic_by_hand(w + "/im2col", stage)
        assert 1.0e9 < v < 1.3e9          # 1028 MB algorithmic per product with a column buffer
    # the fused ops read the image, not a column buffer: 206 MB algorithmic per product
    t = bench.traffic_from_profiles(w, "direct", ["gemm_fwd", "gemm_dgrad", "gemm_wgrad"])
    assert set(t) == {"gemm_fwd", "gemm_dgrad", "gemm_wgrad"}
    for stage, v in t.items():
        assert v == _traffic_by_hand(w, stage)
        assert 2.0e8 < v < 5.0e8
    assert bench.traffic_from_profiles("mnist_conv3x3_1x28x28_b64", "im2col") == {}


def _detail(proc):
    """The full JSON (stage tables of every workload) that the script writes to stderr."""
    lines = [ln for ln in proc.stderr.splitlines() if ln.startswith("detail {")]
    assert len(lines) == 1
    return json.loads(lines[0][len("detail "):])


def test_compact_line_stays_short_whatever_the_detail_holds():
    # the stdout line is built from the detail by dropping, never by cutting: a detail far larger
    # than any real one still gives a line a tail capture holds, with the contract fields intact
    import bench
    stage = {"stage": "s" * 30, "bound": "hbm", "ms_in_step": 0.1234, "frac_in_step": 0.5678, "bytes": 10 ** 8,
             "vs_copy_in_step": 0.987}
    gemm = {"stage": "gemm_fwd", "bound": "mfma", "ms_in_step": 0.4, "frac_in_step": 0.85}
    roof = {"bound": "mfma", "achieved": 130.0, "peak": 157.3, "unit": "TFLOP/s", "frac": 0.8264, "traffic": 3 * 10 ** 8,
            "kernel": "sgemm_kernel", "stage": "gemm_fwd", "flops_per_launch": 59190000000, "avg_launch_ms": 0.45,
            "timing": "HIP events around the launch inside 20 consecutive steps"}
    work = {"value": 100.0, "ms_per_step": 1.5, "roofline": roof, "parity": {"ok": True},
            "stages": [dict(stage, stage="stage_%d" % i) for i in range(40)] + [gemm]}
    out = {"metric": "m" * 80, "value": 122.0, "unit": "TFLOP/s", "n_gpus": 1, "steps": 20, "warmup": 5, "ms_per_step": 1.45,
           "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
           "device": "d" * 60, "config": {"workload": "w" * 40, "x": [64, 128, 56, 56], "filters": [128, 128, 3, 3], "pad": [1, 1],
                                          "stride": [1, 1], "conv_algo": "c" * 90, "value_is": "v" * 200},
           "roofline": roof, "frac_fp32_mfma_peak": 0.77, "parity": {"ok": True, "bit_exact": {"pad": True}, "rel_fro": {"conv_fwd": 1e-7}},
           "stages": work["stages"], "cpu_baseline": {"value": 0.2, "unit": "TFLOP/s", "cores": 16, "kind": "port", "sample": "s" * 900},
           "op_api_step": {"ms_per_step": 1.46, "TFLOPs": 121.0}, "hbm_reference": {"copy_kernel_1GiB": {"frac": 0.7}},
           "workloads": {"workload_%d_%s" % (i, "n" * 30): work for i in range(30)}}
    line = json.dumps(bench.compact_line(out), separators=(",", ":"))
    assert len(line) <= bench.MAX_LINE < 4000
    back = json.loads(line)
    for key in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling",
                "vs_baseline", "dtype", "data", "config", "roofline", "cpu_baseline", "parity"):
        assert key in back, key
    assert back["roofline"]["traffic"] == 3 * 10 ** 8 and len(back["cpu_baseline"]["sample"]) <= 220
    # a detail of ordinary size keeps every part
    out["workloads"] = {"workload_%d" % i: work for i in range(7)}
    out["stages"] = work["stages"][:8] + [gemm]
    back = bench.compact_line(out)
    assert set(back["workloads"]) == set(out["workloads"]) and "stages" in back and "hbm_reference" in back
    assert back["workloads"]["workload_0"]["hbm_worst"][0].startswith("stage_")
    assert back["workloads"]["workload_0"]["hbm_worst"][1:] == [0.568, 0.987] and back["stages"]["stage_0"] == [0.1234, 0.5678, 0.987]
    assert len(json.dumps(back, separators=(",", ":"))) <= bench.MAX_LINE


@pytest.mark.gpu
def test_default_workload_prints_the_contract_line():
    proc = _run(["--steps", "2", "--warmup", "1", "--stage-reps", "2", "--cpu-sample", "2"], 900)
    assert proc.returncode == 0, proc.stderr[-2000:]
    lines = [ln for ln in proc.stdout.splitlines() if ln.strip()]
    assert len(lines) == 1, "exactly one line on stdout"
    assert len(lines[0]) < 4000, "the stdout line must fit a tail capture (%d characters)" % len(lines[0])
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
    assert "inside" in roof["timing"] and roof["avg_launch_ms"] > 0
    cpu = out["cpu_baseline"]
    assert cpu["kind"] in ("port", "reference") and cpu["cores"] >= 1 and cpu["value"] > 0 and cpu["sample"]
    # the gate ran the timed stage list of every workload on a 2-image slice
    par = out["parity"]
    assert par["ok"] is True and par["bit_exact"] == {"pad": True, "pool_values": True, "pool_mask": True, "pool_bwd_padded": True}
    assert set(par["rel_fro"]) == {"conv_fwd", "conv_dgrad", "conv_wgrad"} and max(par["rel_fro"].values()) <= 1e-4
    assert "no column buffer" in out["config"]["conv_algo"]
    assert "im2col" not in out["config"]["value_is"] and "pad_x" in out["config"]["value_is"]
    assert set(out["workloads"]) == {"vgg_mid_conv3x3_128x56x56_b64/im2col", "alexnet_conv1_11x11s4_3x227x227_b128",
                                     "alexnet_conv1_11x11s4_3x227x227_b128/col", "raw_gemm_4096_and_batched_64x512",
                                     "cifar_conv1_5x5_3x32x32_b128", "cifar_conv2_5x5_32x15x15_b128", "mnist_conv3x3_1x28x28_b64"}
    for name, row in out["workloads"].items():
        assert row["value"] > 0 and row["ms_per_step"] > 0 and row["gemm_frac"] > 0 and row["parity_ok"] is True
        assert name.startswith("raw_gemm") or 0 < row["hbm_worst"][1] <= row["hbm_best"][1] < 1.2
    # untimed steps in front of the warm-up steps (the clock ramps for ~25 ms after an idle stretch) are declared
    assert out["clock_settle"]["ms"] == 60.0 and out["clock_settle"]["steps"] >= 5
    assert set(out["hbm_reference"]) == {"copy_kernel_1GiB", "runtime_memcpy_1GiB", "write_fill_1GiB", "read_sum_1GiB", "add_2r1w_1GiB"}
    assert all(0.2 < v < 1.0 for v in out["hbm_reference"].values())

    # ---- the full tables, on stderr
    full = _detail(proc)
    assert full["value"] == out["value"] and full["roofline"]["frac"] == roof["frac"]
    # the roofline figure is clocked inside real steps; every stage carries that clock and,
    # with --stage-reps > 0, the back-to-back one as well
    for row in full["stages"]:
        assert row["ms_in_step"] > 0 and row["ms"] > 0 and 0 < row["frac_in_step"] < 1.2
    # the traffic figure is what the committed counter summaries say, not a constant
    import bench
    assert roof["traffic"] == _traffic_by_hand(out["config"]["workload"], roof["stage"])
    assert roof["traffic"] == bench.traffic_from_profiles(out["config"]["workload"], "direct",
                                                          ["gemm_fwd", "gemm_dgrad", "gemm_wgrad"])[roof["stage"]]
    # the other configurations ride along: AlexNet conv1 (LRN both ways, k = 2), the raw products,
    # and the first layers whose GEMMs are priced against both roofs
    w = full["workloads"]
    assert "im2col" in w["vgg_mid_conv3x3_128x56x56_b64/im2col"]["config"]["conv_algo"]
    assert [r["stage"] for r in w["vgg_mid_conv3x3_128x56x56_b64/im2col"]["stages"]][:2] == ["im2col", "gemm_fwd_NT"]
    assert w["vgg_mid_conv3x3_128x56x56_b64/im2col"]["parity"]["bit_exact"]["col2im"] is True
    assert [r["stage"] for r in w["alexnet_conv1_11x11s4_3x227x227_b128/col"]["stages"]][:2] == ["im2col", "gemm_fwd"]
    alex = w["alexnet_conv1_11x11s4_3x227x227_b128"]
    assert alex["config"]["lrn"]["k"] == 2.0
    assert set(alex["parity"]["rel_fro"]) == {"conv_fwd", "lrn_fwd", "lrn_bwd", "conv_dgrad", "conv_wgrad"}
    assert alex["parity"]["bit_exact"] == {"pool_values": True, "pool_mask": True, "pool_bwd": True, "col2im": True}
    names = [r["stage"] for r in alex["stages"]]
    assert "lrn_fwd" in names and "lrn_bwd" in names and "max_pool_bwd" in names
    # a strided layer with 3 input channels: the forward product and the weight gradient gather their
    # patches from the image and write / read NCHW themselves -- no im2col, no transposes
    assert names[0] == "gemm_fwd" and "im2col" not in names and not any(n.startswith("transpose") for n in names)
    assert "col2im" in names and "no column buffer" in alex["config"]["conv_algo"]
    assert all(r["ms_in_step"] > 0 for r in alex["stages"])
    assert len(w["raw_gemm_4096_and_batched_64x512"]["stages"]) == 5
    assert w["raw_gemm_4096_and_batched_64x512"]["parity"]["mul22_x4_batched_rel_fro"] <= 1e-4
    for name in ("cifar_conv1_5x5_3x32x32_b128", "mnist_conv3x3_1x28x28_b64"):
        gemms = [r for r in w[name]["stages"] if r["bound"] == "mfma"]
        # both roofs in every row; the data gradient (which still writes a column buffer) sits under the HBM one
        assert len(gemms) == 3 and all(r["roof"] in ("hbm", "mfma") and r["frac_hbm"] > 0 and r["frac_in_step"] > 0 for r in gemms)
        assert [r["roof"] for r in gemms if r["stage"] == "gemm_dgrad"] == ["hbm"]
    assert all("vs_measured_copy" in r for r in full["stages"] if r["bound"] == "hbm")
    # ... and against a plain copy of the same bytes timed in the stage's place inside the step
    big = [r for r in full["stages"] if r["bound"] == "hbm" and r["bytes"] >= 4e6]
    assert big and all(0.5 < r["vs_copy_in_step"] < 1.5 and r["ms_copy_same_bytes_in_step"] > 0 for r in big)
    assert all(len(out["stages"][r["stage"]]) == 3 for r in big)
    assert full["cpu_baseline"]["stages"]


@pytest.mark.gpu
def test_in_step_clock_alone():
    # --stage-reps 0: only the in-step clock; the roofline figure still comes out
    proc = _run(["--steps", "2", "--warmup", "1", "--stage-reps", "0", "--no-cpu", "--no-op-api",
                 "--workload", "cifar_conv2_5x5_32x15x15_b128"], 600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads([ln for ln in proc.stdout.splitlines() if ln.strip()][0])
    assert out["roofline"]["achieved"] > 0 and "inside" in out["roofline"]["timing"]
    assert all(v[0] > 0 for v in out["stages"].values())
    for row in _detail(proc)["stages"]:
        assert row["ms_in_step"] > 0 and "ms" not in row
