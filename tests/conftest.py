import ctypes
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle_c():
    """The C restatement of the reference's native operators (oracle/hades_oracle.c), built on
    demand with the Makefile beside it."""
    odir = os.path.join(ROOT, "oracle")
    so = os.path.join(odir, "libhades_oracle.so")
    src = os.path.join(odir, "hades_oracle.c")
    if not os.path.exists(so) or os.path.getmtime(so) < os.path.getmtime(src):
        subprocess.run(["make", "-C", odir], check=True, capture_output=True)
    return ctypes.CDLL(so)


@pytest.fixture(scope="session")
def cuda_device():
    import torch
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
