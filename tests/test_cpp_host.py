"""Runs the C++ host-side mirror's test executable (tests/cpp/test_host.cpp over
adrastea_amd/host/*.hpp and the C ABI).  The CPU leg restates the reference's tensor.rs unit
tests (adrastea_models/src/tensor.rs:583-664) and the lowering of kernels.rs:821-890; the GPU leg
launches through C++ GpuKernels and compares with an integer triple loop."""
import os
import subprocess

import pytest

from adrastea_amd import build


def _binary(allow_build):
    if os.path.exists(build.HOST_TEST_BIN) and not allow_build:
        return build.HOST_TEST_BIN
    return build.build_host_test()


def test_cpp_host_cpu():
    r = subprocess.run([_binary(True)], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout + r.stderr


@pytest.mark.gpu
def test_cpp_host_gpu():
    assert os.path.exists(build.HOST_TEST_BIN), "build the host test first: python -m adrastea_amd.build"
    r = subprocess.run([build.HOST_TEST_BIN, "gpu"], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.strip().endswith("OK"), r.stdout + r.stderr
