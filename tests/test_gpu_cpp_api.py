"""Runs the C++ thread-per-rank test of the MegRay API (tests/cpp/test_vrank_opr.cpp): the reference's
TestOpr cases (test/test_opr.cpp) through get_communicator / HipContext / Communicator virtuals, one
std::thread per rank, linked against libmegray_vrank.so.  One child process."""
import os
import subprocess

import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "cpp", "test_vrank_opr")


@pytest.mark.parametrize("edges", ["default", "events"])
def test_cpp_api_thread_per_rank(edges):
    """`edges`: how the ranks' streams are ordered against each other - one-wavefront arrive / wait / notify
    kernels on counters in device memory (default), or events (MEGRAY_VRANK_EDGES=events, also the fallback
    when the counters cannot be allocated)."""
    if not os.path.exists(BIN):
        from megray_amd import build
        build.build_cpp_test()
    env = dict(os.environ)
    if edges == "events":
        env["MEGRAY_VRANK_EDGES"] = "events"
    proc = subprocess.run([BIN], capture_output=True, text=True, timeout=100, env=env)
    print(proc.stdout)
    print(proc.stderr)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    assert "all passed" in proc.stdout
    for case in ("Init", "InitCallback", "SendRecv", "Scatter", "Gather", "AllToAll", "AllGather", "AllReduce op=0",
                 "AllReduce op=1", "AllReduce op=2", "ReduceScatter op=0", "Broadcast", "Reduce op=0", "Errors"):
        assert f"ok   {case}" in proc.stdout
