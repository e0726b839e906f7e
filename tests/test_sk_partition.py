"""Work partition of the balanced attention launch (lvar_amd/csrc/sk_partition.h): the integer arithmetic is
shared by the kernel and by a host program that walks the ranges as the kernel does, on random weight tables."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_partition_invariants(tmp_path):
    cxx = shutil.which("g++")
    if cxx is None:
        pytest.skip("g++ not available")
    exe = str(tmp_path / "sk_partition_check")
    subprocess.run([cxx, "-O2", "-std=c++17", os.path.join(ROOT, "tests", "host", "sk_partition_check.cpp"), "-o", exe],
                   check=True, timeout=300)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0 and out.stdout.startswith("ok "), out.stdout + out.stderr
