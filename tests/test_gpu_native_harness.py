"""Runs the native (C++) caller harness: the mirror of anode's src/ops_gpu.rs on
top of the C ABI, linked against the static archive, re-running the reference's
own GPU tests for this path and the batch-norm recipe against the oracle."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
HARNESS = os.path.join(HERE, "native", "host_ops_harness")
STAGING = os.path.join(HERE, "native", "io_staging_harness")


def test_harness_is_built():
    assert os.path.exists(HARNESS), "run __graft_entry__.build() first"
    assert os.path.exists(STAGING), "run __graft_entry__.build() first"


@pytest.mark.gpu
def test_native_caller_harness_passes():
    r = subprocess.run([HARNESS], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "ALL PASS" in r.stdout


@pytest.mark.gpu
def test_native_staging_harness_passes():
    """anode_amd/host/io_gpu.hpp: the pinned, double-buffered image pipeline and the device arg-max reader against
    the oracle (bit-exact), and the reference's synchronous copies; also prints host-buffer-inclusive rates."""
    r = subprocess.run([STAGING], capture_output=True, text=True, timeout=300)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-2000:]
    assert "ALL PASS" in r.stdout
