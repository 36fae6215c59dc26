"""Runs the C++ host-mirror test (tests/host_cpp/test_host.cpp) on the GPU."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "host_cpp", "test_host")


def test_cpp_host_mirror_matches_oracle():
    print("[gpu-case] C++ host mirror: QLinear / Q8 / Int8Linear", flush=True)
    if not os.path.exists(BIN):
        import __graft_entry__
        __graft_entry__.build_host_cpp_test()
    out = subprocess.run([BIN], capture_output=True, text=True, timeout=300)
    print(out.stdout)
    print(out.stderr)
    assert out.returncode == 0, out.stdout[-2000:]
    assert "all passed" in out.stdout
