"""Runs the torch-free C++ harness (tests/abi_harness): the C ABI driven from
plain HIP host code, checked against the C oracle."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

HERE = os.path.dirname(os.path.abspath(__file__))
BINARY = os.path.join(HERE, "abi_harness", "abi_harness")


def test_c_abi_from_plain_hip_host_code():
    if not os.path.exists(BINARY):
        pytest.skip("tests/abi_harness/abi_harness is not built (make -C tests/abi_harness)")
    out = subprocess.run([BINARY], capture_output=True, text=True, timeout=120)
    print(out.stdout)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count(" ok") == 5 and "FAIL" not in out.stdout
