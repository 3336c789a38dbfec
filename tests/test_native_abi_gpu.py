"""GPU: the C ABI driven from a plain C++ program (tests/native/unit_test_abi.cpp, built by
tests/native/build_native.py), over the shape grid of the reference's native test (test/unit_test.cpp:322-323)."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BINARY = os.path.join(os.path.dirname(os.path.abspath(__file__)), "native", "unit_test_abi")


def test_native_unit_test(cuda_device):
    assert os.path.exists(BINARY), "build first: python tests/native/build_native.py"
    proc = subprocess.run([BINARY], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=110)
    print(proc.stdout, flush=True)
    assert proc.returncode == 0, proc.stdout
    lines = [l for l in proc.stdout.splitlines() if "validation:" in l]
    assert len(lines) == 18 and all(l.endswith("validation:1") for l in lines)
    assert "all:1" in proc.stdout
