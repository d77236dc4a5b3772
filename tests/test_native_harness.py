"""Runs the torch-free C++ test binary (``pplx-kernels_amd/csrc/test_a2a.cpp``), the native
counterpart of the reference's ``csrc/all_to_all/test_all_to_all.cpp``: the C ABI used the way a
C++ caller would, all simulated ranks in one process, checked against a host expectation."""

import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "pplx-kernels_amd", "bin", "test_a2a")


@pytest.mark.gpu
def test_cpp_harness_passes():
    assert os.path.exists(BIN), "build it with `make -C pplx-kernels_amd/csrc`"
    proc = subprocess.run([BIN], capture_output=True, text=True, timeout=300)
    print(proc.stdout[-4000:], proc.stderr[-4000:])
    assert proc.returncode == 0, proc.stdout[-2000:] + proc.stderr[-2000:]
    assert "ALL PASSED" in proc.stdout
    assert proc.stdout.count("  pass [") == 19  # 6 geometries x 3 call forms + the division helper


def test_cpp_harness_is_built_and_linked_against_the_library():
    assert os.path.exists(BIN)
    out = subprocess.run(["ldd", BIN], capture_output=True, text=True).stdout
    assert "libpplx_kernels.so" in out and "not found" not in out.split("libpplx_kernels.so")[1].splitlines()[0]


def test_division_helper_of_the_kernels_matches_integer_division():
    """The kernels divide by launch constants (tokens per group, experts per rank ...) with a
    multiply-high and two shifts; the host part of the C++ harness compares that helper with
    the hardware's division on millions of (numerator, divisor) pairs.  Needs no GPU."""
    proc = subprocess.run([BIN, "--host-only"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 0 and "pass [fast_div" in proc.stdout, proc.stdout[-2000:] + proc.stderr[-2000:]
