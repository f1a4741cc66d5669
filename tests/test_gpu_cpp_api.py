"""Runs the C++ thread-per-rank test of the MegRay API (tests/cpp/test_vrank_opr.cpp): the reference's
TestOpr cases (test/test_opr.cpp) through get_communicator / HipContext / Communicator virtuals, one
std::thread per rank, linked against libmegray_vrank.so.  One child process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_vrank_opr")


def test_cpp_api_thread_per_rank():
    if not os.path.exists(BIN):
        from megray_amd import build
        build.build_cpp_test()
    proc = subprocess.run([BIN], capture_output=True, text=True, timeout=100)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "all passed" in proc.stdout
    for case in ("Init", "SendRecv", "Scatter", "Gather", "AllToAll", "AllGather", "AllReduce op=0",
                 "AllReduce op=1", "AllReduce op=2", "ReduceScatter op=0", "Broadcast", "Reduce op=0", "Errors"):
        assert f"ok   {case}" in proc.stdout
