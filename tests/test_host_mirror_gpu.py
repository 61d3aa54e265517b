"""Runs the C++ host mirror's test program (tests/cpp/test_host_mirror.cpp, built by
floneum_amd/build.py) on the GPU: the reference's own attention / mask / KV-cache tests, written
against include/fusor_hip.hpp."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_host_mirror():
    exe = os.path.join(ROOT, "tests", "cpp", "test_host_mirror")
    assert os.path.exists(exe), "tests/cpp/test_host_mirror is missing: run floneum_amd/build.py"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
