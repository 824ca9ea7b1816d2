"""Runs the stand-alone C++ consumer of the C ABI (tests/cabi/consumer.cpp, built
by __graft_entry__.build()): no Python, no torch between the caller and the
library."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
BIN = os.path.join(HERE, "cabi", "build", "consumer")


@pytest.mark.gpu
def test_cpp_consumer_runs_clean():
    if not os.path.exists(BIN):
        pytest.fail("tests/cabi/build/consumer is missing: run python -m tspipe_amd.build")
    res = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "c-abi consumer: ok" in res.stdout
