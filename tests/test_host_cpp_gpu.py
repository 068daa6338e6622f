"""Runs the C++20 host-layer parity executable (tests/cpp/test_host_ops.cpp) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu


def test_host_ops_executable():
    from brodiffusion_amd import build
    assert os.path.exists(build.HOST_TEST), "build the host layer first (python -m brodiffusion_amd.build)"
    r = subprocess.run([build.HOST_TEST], capture_output=True, text=True, timeout=110)
    print(r.stdout)
    assert r.returncode == 0 and "test_host_ops: OK" in r.stdout, r.stdout + r.stderr
