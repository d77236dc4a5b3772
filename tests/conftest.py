"""pytest configuration: the ``gpu`` marker, import paths, and a build of the native
libraries when none is present (tests load what is built; they never rebuild it)."""

import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (os.path.join(ROOT, "pplx-kernels_amd"), ROOT):
    if p not in sys.path:
        sys.path.insert(0, p)

LIB = os.path.join(ROOT, "pplx-kernels_amd", "pplx_kernels", "libpplx_kernels.so")
ORACLE_LIB = os.path.join(ROOT, "oracle", "liba2a_oracle.so")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    if not os.path.exists(LIB) or not os.path.exists(os.path.join(ROOT, "pplx-kernels_amd", "bin", "test_a2a")):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "pplx-kernels_amd", "csrc"), "-s"])
    if not os.path.exists(ORACLE_LIB):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "-s"])


@pytest.fixture(scope="session")
def device():
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")
