"""Runs the C++ host-mirror test program (tests/cpp/host_mirror_test.cpp): the operator surface of
include/ascq_ascendc.hpp over the C ABI, every result compared bit-for-bit with the oracle inside the program."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "host_mirror_test")


@pytest.mark.gpu
def test_cpp_host_mirror_program():
    assert os.path.exists(BIN), "tests/cpp/host_mirror_test is not built: run __graft_entry__.build()"
    print("[case] C++ host mirror program", flush=True)
    r = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "ALL PASSED" in r.stdout
    assert "FAIL" not in r.stdout.replace("FAILED", "")
