"""The C++ host side (include/ssd_hip.hpp) on the GPU: tests/cpp/host_check drives the forward, the streaming
continuation and the error paths through the wrapper and checks them against the plain-C oracle; this test runs
the prebuilt binary and reads its verdict."""
import subprocess

import pytest

from tests.cpp.build_host_check import BINARY

pytestmark = pytest.mark.gpu


def test_cpp_host_side_matches_the_oracle():
    assert BINARY.exists(), "tests/cpp/host_check is not built (run __graft_entry__.build())"
    proc = subprocess.run([str(BINARY)], capture_output=True, text=True, timeout=300)
    print(proc.stdout)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "host_check OK" in proc.stdout and "FAIL" not in proc.stdout
