"""Runs the prebuilt C++ facade check (tests/cpp/facade_check.cpp) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cpp_facade_runs():
    exe = os.path.join(ROOT, "tests", "cpp", "facade_check")
    assert os.path.exists(exe), "build it with __graft_entry__.build()"
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0 and "OK" in r.stdout
