"""Runs the C++ test program of the native host API (tests/cpp/test_host_api.cpp).

The program mirrors the reference's doctests for SwiftNetMLP, DeviceMatrix, the L2 loss and the grid encoding
(test/doctests/doctest_swiftnet.cpp, doctest_devicematrix.cpp, doctest_losses.cpp, doctest_encodings.cpp) on the
classes in tiny-dpcpp-nn_amd/include/tnn and checks device results against the CPU oracle.
"""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "cpp", "test_host_api")


def _run(args):
    if not os.path.exists(BINARY):
        pytest.fail(f"{BINARY} is not built: run `make -C tests/cpp` (done by __graft_entry__.build())")
    proc = subprocess.run([BINARY] + args, capture_output=True, text=True, timeout=600)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout[-4000:] + proc.stderr[-2000:]
    assert "0 failed" in proc.stdout


def test_host_api_cpu_cases():
    """bf16/half host types vs the oracle's rounding, packed coordinates, JSON configuration parsing."""
    _run(["--cpu"])


@pytest.mark.gpu
def test_host_api_gpu_cases():
    """SwiftNetMLP forward/inference/backward, Trainer, L2Loss, grid encoding and every error path, on the GPU."""
    _run([])
