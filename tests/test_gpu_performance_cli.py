"""The `performance`-compatible command line tool (megray_amd/apps/megray_performance), run as a child
process with the reference's options (test/performance.cpp:443-496) and checked against the reference's
table (test/performance.cpp:342-362: bufsize / time(us) / speed(GB/s) / iters, speed = bufsize / avg_us /
1000) and against an event timing of the same collective through the flat C ABI."""
import json
import os
import subprocess

import pytest

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from megray_amd import synth  # noqa: E402

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "megray_amd", "apps", "megray_performance")
REFERENCE_SIZES = [8, 1024, 512 * 1024, 1024 * 1024, 10 * 1024 * 1024]  # test/performance.cpp:58-59


def run_cli(*args):
    if not os.path.exists(EXE):
        from megray_amd import build
        build.build_performance()
    proc = subprocess.run([EXE, *args], capture_output=True, text=True, timeout=200)
    assert proc.returncode == 0, proc.stdout + proc.stderr
    return proc.stdout


def parse_tables(text):
    """{function name: (column names, [row of floats])} from the tool's output."""
    tables, name = {}, None
    for line in text.splitlines():
        if line.startswith("Testing "):
            name = line.split()[1]
            tables[name] = (None, [])
        elif name and line.split()[:1] == ["bufsize"]:
            tables[name] = (line.split(), [])
        elif name and line.strip() and tables[name][0]:
            tables[name][1].append([float(x) for x in line.split()])
    return tables


def test_reference_options_and_table():
    # -d devices, -f function, -w warm-up, -i iterations; sizes left at the reference's defaults
    out = run_cli("-d", "4", "-f", "all_reduce", "-w", "10", "-i", "50")
    tables = parse_tables(out)
    assert list(tables) == ["all_reduce_sum"]
    cols, rows = tables["all_reduce_sum"]
    assert cols[:4] == ["bufsize", "time(us)", "speed(GB/s)", "iters"]  # the reference's four columns, in its order
    assert [int(r[0]) for r in rows] == REFERENCE_SIZES
    for r in rows:
        bufsize, avg_us, speed, iters = r[:4]
        assert iters == 50 and avg_us > 0
        assert speed == pytest.approx(bufsize / avg_us / 1000, rel=2e-3)  # printed with six significant digits
    # -s picks one size, -e the backend, -n / -r one node only, like the reference's multi-node options
    out = run_cli("-d", "2", "-f", "all_gather", "-s", "4096", "-w", "5", "-i", "20", "-e", "VRANK", "-n", "1", "-r", "0")
    cols, rows = parse_tables(out)["all_gather"]
    assert len(rows) == 1 and int(rows[0][0]) == 4096 and rows[0][3] == 20
    # every function of the reference's table runs (test/performance.cpp:365-441)
    out = run_cli("-d", "3", "-s", "65536", "-w", "3", "-i", "10")
    assert list(parse_tables(out)) == ["send_recv", "all_reduce_sum", "scatter", "gather", "all_to_all", "all_gather",
                                       "reduce_scatter_sum", "broadcast", "reduce_sum"]
    bad = subprocess.run([EXE, "-n", "2"], capture_output=True, text=True, timeout=60)
    assert bad.returncode != 0  # more than one node: refused


def test_ten_mib_row_agrees_with_an_event_timing(tmp_path):
    """8 ranks x 10 MiB fp32 all_reduce: the tool's HBM column (2 * N * bufsize per collective over its wall
    time per call) against HIP events around the same collective launched through the flat C ABI."""
    nranks, nbytes = 8, 10 * 1024 * 1024
    n = nbytes // 4
    ins = [synth.fill_torch(torch.float32, n, r) for r in range(nranks)]
    outs = [torch.empty_like(t) for t in ins]
    st = torch.cuda.current_stream()
    plan = mr.CollectivePlan(mr.Collective.ALL_REDUCE, ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM)
    for _ in range(50):
        plan.launch(st.cuda_stream)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record(st)
    for _ in range(500):
        plan.launch(st.cuda_stream)
    e1.record(st)
    torch.cuda.synchronize()
    plan.close()
    event_gbps = 2 * nranks * nbytes / (e0.elapsed_time(e1) / 500 * 1e-3) / 1e9

    log = tmp_path / "perf.jsonl"
    # all ranks on one stream (-S): the collectives follow each other on that stream like the event timing's
    out = run_cli("-d", str(nranks), "-f", "all_reduce", "-s", str(nbytes), "-w", "100", "-i", "500", "-S", "-J", str(log))
    cols, rows = parse_tables(out)["all_reduce_sum"]
    assert cols[4:6] == ["hbm(GB/s)", "hbm(%peak)"]
    bufsize, avg_us, speed, iters, hbm, pct = rows[0]
    assert hbm == pytest.approx(2 * nranks * bufsize / avg_us / 1000, rel=2e-3)
    assert pct == pytest.approx(hbm / 80.0, rel=2e-3)
    record = json.loads(log.read_text().splitlines()[0])
    assert record["bufsize"] == nbytes and record["streams"] == "shared"
    assert record["avg_us"] == pytest.approx(avg_us, rel=1e-3)
    print(f"performance tool, one stream: {hbm:.0f} GB/s, event timing {event_gbps:.0f} GB/s")
    # 160 MiB in all: the buffers fit the last-level cache, and how well depends on where each process's allocations lie
    assert hbm == pytest.approx(event_gbps, rel=0.15)
    # every rank on a stream of its own (the reference's harness): each collective waits for all streams and
    # all streams wait for it, a chain of dependent launches that adds a few microseconds per call
    out = run_cli("-d", str(nranks), "-f", "all_reduce", "-s", str(nbytes), "-w", "100", "-i", "500")
    own = parse_tables(out)["all_reduce_sum"][1][0]
    print(f"performance tool, a stream per rank: {own[4]:.0f} GB/s ({own[1]:.1f} us per call)")
    assert own[4] > 0.6 * event_gbps


def test_random_fill_own_buffers_and_the_spread_record(tmp_path):
    """-R fills the inputs from the counter generator, -M lets every rank hipMalloc its own buffers (what the reference's
    harness does, test/performance.cpp:108-110); the table keeps the reference's columns either way, and -J records
    how the per-call times spread, how far the device was behind at the end and how often a rank went to sleep."""
    log = tmp_path / "spread.jsonl"
    out = run_cli("-d", "8", "-f", "all_reduce", "-s", "65536,4194304", "-w", "50", "-i", "300", "-R", "-M", "-J", str(log))
    cols, rows = parse_tables(out)["all_reduce_sum"]
    assert cols[:4] == ["bufsize", "time(us)", "speed(GB/s)", "iters"] and [int(r[0]) for r in rows] == [65536, 4194304]
    records = [json.loads(line) for line in log.read_text().splitlines()]
    assert [r["bufsize"] for r in records] == [65536, 4194304]
    for r in records:
        assert r["fill"] == "random" and r["buffers"] == "own" and r["streams"] == "own" and r["iters"] == 300
        assert 0 < r["median_us"] <= r["p90_us"] <= r["p99_us"] <= r["p999_us"] <= r["max_us"]
        assert r["host_us"] <= r["avg_us"] and r["drain_us"] >= 0
        assert r["avg_us"] * 300 == pytest.approx(r["host_us"] * 300 + r["drain_us"], rel=1e-4)  # six printed digits
        assert r["plans_built"] == 1  # 350 collectives on the same buffers: planned once
    zeros = tmp_path / "zeros.jsonl"
    run_cli("-d", "2", "-f", "all_reduce", "-s", "4096", "-w", "5", "-i", "20", "-J", str(zeros))
    r = json.loads(zeros.read_text().splitlines()[0])
    assert r["fill"] == "zeros" and r["buffers"] == "placed"
