"""Runs the C++ host-mirror test program (tests/cpp/host_mirror_test.cpp): the operator surface of
include/ascq_ascendc.hpp over the C ABI, every result compared bit-for-bit with the oracle inside the program."""
import os
import re
import subprocess

import numpy as np
import pytest

from splitmix64 import SplitMix64, fnv1a64

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cpp", "host_mirror_test")


def first_case_inputs():
    """The inputs of the C++ program's first case, drawn with the Python restatement of its generator."""
    r = SplitMix64(1)
    m, n = 64, 256
    x = r.uniform(-6.0, 6.0, m * n).astype(np.float16)
    s = r.uniform(5.0, 40.0, n).astype(np.float16)
    o = r.uniform(-3.0, 3.0, n).astype(np.float16)
    return m, n, x, s, o


def sums(line):
    return {k: int(v, 16) for k, v in re.findall(r"(\w+)=([0-9a-f]{16})", line)}


def test_cpp_and_python_hosts_draw_identical_inputs():
    """No GPU: the C++ program prints checksums of the inputs it generates; the Python generator gives the same bytes."""
    assert os.path.exists(BIN), "tests/cpp/host_mirror_test is not built: run __graft_entry__.build()"
    r = subprocess.run([BIN, "--inputs"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr
    line = [l for l in r.stdout.splitlines() if l.startswith("[inputs] quant_per_channel")][0]
    _, _, x, s, o = first_case_inputs()
    assert sums(line) == {"x": fnv1a64(x), "s": fnv1a64(s), "o": fnv1a64(o)}
    # the generator itself: the widely published first outputs of SplitMix64 for seed 1234567
    assert [int(v) for v in SplitMix64(1234567).next(3)] == [6457827717110365317, 3203168211198807973, 9817491932198370423]


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
    # the same operator on the same seeded inputs through the Python mirror gives the same bytes
    import torch
    from ascq import ops
    from gpu_util import DEV, to_dev
    m, n, x, s, o = first_case_inputs()
    q = torch.zeros((m, n), dtype=torch.int8, device=DEV)
    ops.ascend_quant(q, to_dev(x.reshape(m, n)), to_dev(s), to_dev(o))
    line = [l for l in r.stdout.splitlines() if l.startswith("[output] quant_per_channel")][0]
    assert sums(line) == {"q": fnv1a64(q.cpu().numpy())}
