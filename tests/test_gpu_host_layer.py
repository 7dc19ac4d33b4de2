"""Runs the C++ host-layer harness (DeviceArena / StreamPool / Gate / QuantLinear /
DecodeAttention over the C ABI) and requires every one of its checks to pass."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

BIN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "host", "test_host")


def test_cpp_host_harness():
    assert os.path.exists(BIN), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "[FAIL]" not in r.stdout and "ALL PASSED" in r.stdout
