"""The thread-per-rank communicator on simulated streams under the thread sanitizer (no GPU).

tests/cpp/stream_sim.cpp compiles the backend's host side as it is (rendezvous of the rank threads, plan cache,
cross-stream ordering by arrive / wait / notify kernels or by events, point-to-point matching) against streams
that are queues worked off in a random order, and checks in every round that no kernel ran before every rank's
input was there, that no rank's stream went on before the result was there, and that no input was overwritten
before it was read - with a stream per rank, shared streams and mixtures, launches that carry the ordering
themselves and launches between wait and notify kernels, the allocation-free entry point, calls that one rank
rejects, and rings of send / recv.  The thread sanitizer watches the host threads meanwhile."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "megray_amd", "csrc")
SOURCES = ["vrank_communicator.cpp", "megray_communicator.cpp", "megray_core.cpp", "vrank_engine.cpp", "vrank_plan.cpp",
           "bootstrap_client.cpp", "bootstrap_server.cpp"]


@pytest.fixture(scope="module")
def simulator(tmp_path_factory):
    gxx = shutil.which("g++")
    rocm_include = os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "include")
    if not gxx or not os.path.exists(os.path.join(rocm_include, "hip", "hip_runtime_api.h")):
        pytest.skip("needs g++ and the HIP runtime API headers")
    exe = str(tmp_path_factory.mktemp("sim") / "stream_sim")
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=thread", "-pthread", "-D__HIP_PLATFORM_AMD__=1",
           f"-I{ROOT}/include", f"-I{CSRC}", f"-I{rocm_include}", os.path.join(ROOT, "tests", "cpp", "stream_sim.cpp")]
    cmd += [os.path.join(CSRC, s) for s in SOURCES] + ["-o", exe]
    build = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    assert build.returncode == 0, build.stderr[-4000:]
    return exe


@pytest.mark.parametrize("seed,mode", [(1, "counters"), (2, "counters"), (3, "counters"), (5, "counters"),
                                       (9, "events"), (10, "events"), (4, "fixed"), (7, "fixed")])
def test_stream_ordering_holds_on_simulated_streams(simulator, seed, mode):
    # "fixed": every round is the allocation-free all_reduce, and the simulator fails if the communicator called
    # hipMalloc, hipHostMalloc or hipEventCreate at all
    args = [simulator, "1200", str(seed)] + ([mode] if mode in ("events", "fixed") else [])
    run = subprocess.run(args, capture_output=True, text=True, timeout=300)
    assert "ThreadSanitizer" not in run.stderr, run.stderr[-4000:]
    assert run.returncode == 0 and run.stdout.strip().startswith("ok "), run.stdout[-2000:] + run.stderr[-2000:]
