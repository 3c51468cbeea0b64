"""bench.py's command-line contract: what can be checked without a GPU (the refusal of more than one GPU) and, on the GPU
box, that every workload prints one JSON line with the fields the driver reads."""
import json
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BENCH = os.path.join(ROOT, "bench.py")

REQUIRED = ["metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better", "scaling", "vs_baseline", "dtype",
            "data", "config", "roofline"]
ROOFLINE = ["bound", "achieved", "peak", "unit", "frac", "traffic"]


def test_more_than_one_gpu_is_refused_with_a_message():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def check_roofline(roof):
    for key in ROOFLINE:
        assert key in roof, key
    assert abs(roof["frac"] - roof["achieved"] / roof["peak"]) < 1e-9
    assert roof["bound"] in ("hbm", "mfma") and roof["unit"] in ("GB/s", "TFLOP/s")


@pytest.mark.gpu
def test_default_run_carries_the_whole_metric():
    """No --workload: the training step at the top level, inference and the 3-D encoding as sub-objects, each checked against
    the oracle before it is timed, each the median of the repetitions."""
    r = subprocess.run([sys.executable, BENCH, "--steps", "5", "--warmup", "2", "--reps", "3", "--prewarm-ms", "20", "--no-cpu-baseline"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in REQUIRED:
        assert key in out, key
    assert out["steps"] == 5 and out["warmup"] == 2 and out["reps"] == 3 and len(out["ms_per_step_reps"]) == 3
    assert sorted(out["ms_per_step_reps"])[1] == out["ms_per_step"]
    assert out["parity_checked"] is True and out["parity"]["dW_max_norm_rel"] < 1e-2
    check_roofline(out["roofline"])
    assert out["roofline"]["bound"] == "mfma" and "training step" in out["config"]["workload"]
    for leg, unit in (("infer", "samples/s"), ("grid", "points/s")):
        assert out[leg]["unit"] == unit and out[leg]["value"] > 0 and out[leg]["parity_checked"] is True
        check_roofline(out[leg]["roofline"])
        assert out[leg]["roofline"]["bound"] == "hbm"
    assert 0 < out["infer"]["roofline"]["mfma_frac"] < 1
    # config 1 at its own batch, and the 2^18 batch over enough buffers that no call finds its rows in the cache
    assert "2^17" in out["infer_2p17"]["config"]["workload"] and out["infer_2p17"]["config"]["batch"] == 1 << 17
    assert out["infer_hbm"]["roofline"]["buffers_in_rotation_bytes"] > 256e6
    for leg in ("infer_2p17", "infer_hbm"):
        check_roofline(out[leg]["roofline"])
        assert out[leg]["rows_bit_equal_to_checked_output"] is True
    # the step executes 14 of the 15 products the convention counts (no dL/dx buffer); both fractions and a timing with dL/dx
    roof = out["roofline"]
    assert roof["executed_flops_per_launch"] * 15 == roof["algorithmic_flops_per_launch"] * 14
    assert abs(roof["frac_executed"] * 15 - roof["frac"] * 14) < 1e-9
    assert out["with_dLdx"]["kernel_ms"] > 0 and 0 < out["with_dLdx"]["frac"] < 1
    # how many elements actually leave the strict elementwise bar
    for what in ("y", "dW", "dLdx"):
        rep = out["parity"]["strict_bar"][what]
        assert rep["n"] > 0 and rep["frac_outside"] <= 2e-3 and rep["worst_ratio"] <= 4.0
    assert "frac_lines_moved" in out["grid"]["roofline"]


@pytest.mark.gpu
@pytest.mark.parametrize("workload", ["train", "train_fb", "infer", "grid", "grid_mlp", "grid_train", "py_infer", "py_train", "py_grid_train"])
def test_every_workload_prints_the_contract_line(workload):
    r = subprocess.run([sys.executable, BENCH, "--workload", workload, "--steps", "5", "--warmup", "2", "--reps", "2", "--prewarm-ms", "20",
                        "--no-cpu-baseline"], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in REQUIRED:
        assert key in out, key
    check_roofline(out["roofline"])
    assert out["n_gpus"] == 1 and out["vs_baseline"] is None and out["data"] == "synthetic"
    assert "workload" in out["config"] and out["value"] > 0
    if workload.startswith("py_"):  # the drop-in's own legs carry the C-ABI call of the same work, timed in the same process
        assert out["c_abi_ms_per_step"] > 0 and abs(out["ratio_to_c_abi"] - out["ms_per_step"] / out["c_abi_ms_per_step"]) < 1e-9
