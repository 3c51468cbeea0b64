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


@pytest.mark.gpu
@pytest.mark.parametrize("workload", ["train", "train_fb", "infer", "grid", "grid_mlp", "grid_train"])
def test_every_workload_prints_the_contract_line(workload):
    r = subprocess.run([sys.executable, BENCH, "--workload", workload, "--steps", "5", "--warmup", "2", "--no-cpu-baseline"],
                       capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stderr[-2000:]
    lines = [l for l in r.stdout.splitlines() if l.strip()]
    assert len(lines) == 1
    out = json.loads(lines[0])
    for key in REQUIRED:
        assert key in out, key
    for key in ROOFLINE:
        assert key in out["roofline"], key
    assert out["n_gpus"] == 1 and out["vs_baseline"] is None and out["data"] == "synthetic"
    assert "workload" in out["config"] and out["value"] > 0
    assert abs(out["roofline"]["frac"] - out["roofline"]["achieved"] / out["roofline"]["peak"]) < 1e-9
    assert out["roofline"]["bound"] in ("hbm", "mfma") and out["roofline"]["unit"] in ("GB/s", "TFLOP/s")
