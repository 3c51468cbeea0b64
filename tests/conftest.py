import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tiny-dpcpp-nn_amd"))
sys.path.insert(0, os.path.join(ROOT, "oracle"))  # the checker: oracle_bindings, tolerances
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    """The CPU oracle (oracle/libtnn_oracle.so), built on demand. Test infrastructure only."""
    so = os.path.join(ROOT, "oracle", "libtnn_oracle.so")
    if not os.path.exists(so):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle")])
    import oracle_bindings

    return oracle_bindings.Oracle(so)


@pytest.fixture(scope="session")
def tnn():
    """GPU-side helper around the C ABI; fails loudly when the HIP library is not built."""
    import gpu_harness

    return gpu_harness.Harness()
