"""Runs the native (C++) caller harness: the mirror of anode's src/ops_gpu.rs on
top of the C ABI, linked against the static archive, re-running the reference's
own GPU tests for this path and the batch-norm recipe against the oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
HARNESS = os.path.join(HERE, "native", "host_ops_harness")


def test_harness_is_built():
    assert os.path.exists(HARNESS), "run __graft_entry__.build() first"


@pytest.mark.gpu
def test_native_caller_harness_passes():
    r = subprocess.run([HARNESS], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "ALL PASS" in r.stdout
