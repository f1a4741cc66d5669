#!/usr/bin/env python3
"""Headline benchmark: 8 virtual ranks x 2^28 fp32 SUM all_reduce on one MI355X.

A "step" is one whole all_reduce (every rank's 1 GiB buffer read, every rank's result written)
with all buffers already resident in HBM.  Prints ONE JSON line:

  value      achieved HBM GB/s of the collective = B_min / t, B_min = 2 * N * n * 4 bytes (each
             input read once, each output written once; the fused schedule executes exactly that)
  roofline   the fold kernel against the 8 TB/s HBM peak, timed with HIP events on the launch stream
  cpu_baseline  the reference tests' expected-value loop (test/test_opr.cpp:321-330) re-stated in the
             CPU oracle, timed on this host on a bounded sample of the same workload
  comm_api_us   the same all_reduce at 4 KiB .. 1 MiB per rank through MegRay::Communicator::all_reduce,
             one thread per rank (the reference's test/performance.cpp:103-137 harness shape), every
             rank on a stream of its own and all ranks on one stream: microseconds per collective
  comm_api_large  the headline shape through the same API and harness on random inputs: 8 ranks x 10 MiB / 128 MiB /
             1 GiB, buffers each rank allocates itself or placed by the library, a stream per rank or one shared
  small_msg_us  the same sizes through the flat C ABI (one caller, one stream)
  other_configs the other benchmark configurations (reduce_scatter / all_gather fp16, MAX int32,
             MIN int64, all_to_all uint8, SUM int8), each timed with HIP events
  other_layout  the headline launches again on buffers placed the other way (--layout), timed like the headline, in this
             process after the headline; beside it (processes_of_their_own) the same in three fresh processes

Usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--log2n 28] [--no-cpu] [--no-small] [--no-comm]
                       [--no-others] [--layout placed|separate]
"""
import argparse
import hashlib
import json
import os
import subprocess
import sys
import tempfile
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0

# HBM bytes per launch measured offline (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by the same
# counters on a plain copy of known size) are kept in a tracked file together with a hash of the kernel
# sources they were measured on; a figure whose hash is not that of the sources in this tree is stale
# and is not reported.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
KERNEL_SOURCES = ("vrank_fold_impl.hpp", "vrank_types.h", "vrank_kernels.hip")


def kernel_source_hash():
    h = hashlib.sha256()
    for name in KERNEL_SOURCES:
        with open(os.path.join(ROOT, "megray_amd", "csrc", name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def measured_traffic(key):
    """HBM bytes per launch of workload `key` from the tracked profile summary, or None if there is no
    figure for the kernels as they are now."""
    try:
        with open(TRAFFIC_FILE) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None
    entry = table.get("workloads", {}).get(key)
    if not entry or table.get("kernel_source_hash") != kernel_source_hash():
        return None
    return entry.get("hbm_bytes_per_launch")


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--log2n", type=int, default=28, help="elements per rank = 2^log2n")
    ap.add_argument("--ranks", type=int, default=8)
    ap.add_argument("--schedule", default="fused", choices=["fused", "two_phase", "ring"])
    ap.add_argument("--workload", default="all_reduce",
                    choices=["all_reduce", "copy", "c2_reduce_scatter", "c2_all_gather", "c3_max_int32",
                             "c3_min_int64", "c5_all_to_all", "c5_sum_int8"],
                    help="all_reduce = the headline; copy = 1 GiB plain copy (counter calibration); "
                         "c2/c3/c5 = the other benchmark configurations")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-small", action="store_true", help="skip the small-message sweep")
    ap.add_argument("--no-check", action="store_true", help="skip the correctness checks")
    ap.add_argument("--no-comm", action="store_true", help="skip the thread-per-rank Communicator API leg")
    ap.add_argument("--no-others", action="store_true", help="skip the other benchmark configurations")
    ap.add_argument("--layout", choices=("placed", "separate"), default="placed",
                    help="where the ranks' buffers lie in HBM: placed = one allocation laid out by the library "
                         "(mrv_rank_buffers_layout), separate = one torch allocation per buffer")
    return ap.parse_args()


LAYOUT_TEXT = {
    "placed": "one allocation, buffers an odd multiple of 128 MiB apart (mrv_rank_buffers_layout)",
    "separate": "one torch allocation per buffer",
}


def alloc_buffers(torch, mr, specs, layout, collective=None, written=None):
    """Tensors for (numel, dtype) pairs in HBM.  "placed": views into one allocation at the distances the
    library recommends for buffers that a collective walks through in step (`collective` and `written` tell it
    what the buffers are for); "separate": one torch allocation each, wherever the caching allocator puts them."""
    if layout == "placed":
        return mr.place_tensors(torch, specs, "cuda:0", collective, written)
    return [torch.empty(numel, dtype=dtype, device="cuda:0") for numel, dtype in specs]


def make_buffers(torch, mr, nranks, n, layout):
    """Inputs and outputs of the headline workload.  Inputs: uniform[-1, 1) fp32 from the counter-based generator,
    element i of rank r depends only on (seed, r, i)."""
    from megray_amd import synth
    bufs = alloc_buffers(torch, mr, [(n, torch.float32)] * (2 * nranks), layout)
    ins, outs = bufs[:nranks], bufs[nranks:]
    for r, t in enumerate(ins):
        synth.fill_torch(torch.float32, n, r, out=t)
    return ins, outs


def make_inputs(torch, nranks, n):
    """The same inputs as separate tensors (small sizes)."""
    from megray_amd import synth
    return [synth.fill_torch(torch.float32, n, r) for r in range(nranks)]


def check_small(torch, mr, orc, np):
    """Full bit compare against the oracle's literal ring replay at a size the CPU finishes fast."""
    nranks, n = 8, (1 << 20) + 5
    ins = make_inputs(torch, nranks, n)
    outs = [torch.empty_like(t) for t in ins]
    mr.all_reduce(ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    from megray_amd import synth
    host = [synth.fill_np(np.float32, n, r) for r in range(nranks)]  # regenerated, not copied back
    want = orc.ucx_all_reduce(host, orc.FLOAT32, orc.SUM)
    for r in range(nranks):
        got = outs[r].cpu().numpy()
        if not np.array_equal(got.view(np.uint32), want[r].view(np.uint32)):
            raise SystemExit("bench: all_reduce differs from the oracle at n=2^20+5")


def check_full(torch, mr, ins, outs, n):
    """Size-independent checks at the full size: every rank holds the same bits, and the fused
    result equals the 2(N-1)-step ring replay of the reference schedule run on the device."""
    for r in range(1, len(outs)):
        if not torch.equal(outs[0].view(torch.int32), outs[r].view(torch.int32)):
            raise SystemExit(f"bench: rank {r} differs from rank 0")
    ref = outs[0].clone()
    mr.all_reduce(ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, schedule=mr.Schedule.RING,
                  stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    if not torch.equal(ref.view(torch.int32), outs[len(outs) // 2].view(torch.int32)):
        raise SystemExit("bench: fused schedule differs from the ring replay")


def small_message_sweep(torch, mr):
    """all_reduce SUM fp32, 8 ranks, 4 KiB .. 1 MiB per rank: microseconds per collective.

    stream_us        planned once (mrv_plan_create), launched back to back on one stream: the rate at
                     which collectives retire (one kernel launch each)
    unplanned_us     the same through mrv_all_reduce, which plans on every call
    sync_median/p99  one planned collective at a time, launch to host-visible completion
    """
    out = {}
    st = torch.cuda.current_stream()
    for nbytes in (4096, 4096, 16384, 65536, 262144, 1048576):  # the first pass only warms the path up
        n = nbytes // 4
        ins = make_inputs(torch, 8, n)
        outs = [torch.empty_like(t) for t in ins]
        plan = mr.CollectivePlan(mr.Collective.ALL_REDUCE, ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM)
        raw = st.cuda_stream

        def timed(fn, iters):
            for _ in range(100):
                fn()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(st)
            for _ in range(iters):
                fn()
            e1.record(st)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1000.0 / iters

        stream_us = timed(lambda: plan.launch(raw), 2000)
        unplanned_us = timed(lambda: mr.all_reduce(ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream=raw), 1000)
        lat = []
        for _ in range(1000):
            t0 = time.perf_counter()
            plan.launch(raw)
            torch.cuda.synchronize()
            lat.append((time.perf_counter() - t0) * 1e6)
        lat.sort()
        out[str(nbytes)] = {"stream_us": round(stream_us, 2), "unplanned_us": round(unplanned_us, 2),
                            "sync_median_us": round(lat[len(lat) // 2], 2),
                            "sync_p99_us": round(lat[int(len(lat) * 0.99)], 2)}
        plan.close()
    return out


def comm_api_sweep():
    """all_reduce SUM fp32, 8 ranks, 4 KiB .. 1 MiB per rank through MegRay::Communicator::all_reduce, driven like
    the reference's benchmark (test/performance.cpp:103-137): one thread per rank, 200 warm-up and 2000 timed
    calls back to back, one stream sync at the end.  Runs the performance CLI as a child process (its threads
    are C++ threads; this process has not touched the GPU yet).

    avg_us     wall time of the 2000 calls including the final sync, per call (the reference's "time(us)")
    median_us / p99_us   of the time from one call's return to the next call's return on rank 0
    """
    exe = os.path.join(ROOT, "megray_amd", "apps", "megray_performance")
    if not os.path.exists(exe):
        raise SystemExit("bench: megray_amd/apps/megray_performance is not built (python -m megray_amd.build)")
    sizes = "4096,16384,65536,262144,1048576"
    out = {}
    for mode, flag in (("own_streams", []), ("shared_stream", ["-S"])):
        with tempfile.NamedTemporaryFile("r", suffix=".jsonl") as tmp:
            cmd = [exe, "-d", "8", "-f", "all_reduce", "-s", sizes, "-w", "200", "-i", "2000", "-J", tmp.name] + flag
            proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
            if proc.returncode != 0:
                raise SystemExit(f"bench: {' '.join(cmd)} failed:\n{proc.stdout}\n{proc.stderr}")
            rows = [json.loads(line) for line in tmp.read().splitlines() if line.strip()]
        keys = ("avg_us", "host_us", "median_us", "p90_us", "p99_us", "p999_us", "max_us")
        out[mode] = {str(r["bufsize"]): dict({k: round(r[k], 2) for k in keys},
                                             drain_ms=round(r["drain_us"] / 1e3, 2), sleeps=r["sleeps"]) for r in rows}
    out["harness"] = "megray_performance -d 8 -f all_reduce -w 200 -i 2000 (thread per rank, MegRay::Communicator API)"
    out["columns"] = ("avg_us: wall time of the 2000 calls including the final stream sync, per call; host_us: the same "
                      "without the final sync (what a call costs the calling thread); median / p90 / p99 / p999 / max: of "
                      "the time between consecutive call returns on rank 0; drain_ms: the final sync (how far the device "
                      "was behind); sleeps: times a rank slept on the condition variable while waiting for the others")
    return out


def comm_api_large():
    """The headline shape through the drop-in boundary itself: MegRay::Communicator::all_reduce, one thread per rank
    (the reference's harness, test/performance.cpp:85-137), inputs from the counter generator (-R), 8 ranks x
    {10 MiB, 128 MiB, 1 GiB} fp32 SUM.  Four set-ups: buffers each rank allocates itself with hipMalloc (-M, what
    test/performance.cpp:108-110 does) or laid out by the library in one allocation, and a stream per rank (as in
    the reference) or one shared stream (-S).  Per size: microseconds per collective (wall clock of all timed calls
    including the final sync), GB/s on the collective's minimum bytes 2 * N * bufsize, and that over the HBM peak.
    Runs as child processes before this process touches the GPU."""
    exe = os.path.join(ROOT, "megray_amd", "apps", "megray_performance")
    if not os.path.exists(exe):
        raise SystemExit("bench: megray_amd/apps/megray_performance is not built (python -m megray_amd.build)")
    out = {}
    for buffers, bflag in (("own_hipMalloc", ["-M"]), ("placed", [])):
        for streams, sflag in (("own_streams", []), ("shared_stream", ["-S"])):
            rows = []
            for sizes, warm, iters in (("10485760", 100, 500), ("134217728,1073741824", 10, 30)):
                with tempfile.NamedTemporaryFile("r", suffix=".jsonl") as tmp:
                    cmd = [exe, "-d", "8", "-f", "all_reduce", "-s", sizes, "-w", str(warm), "-i", str(iters), "-R",
                           "-J", tmp.name] + bflag + sflag
                    proc = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
                    if proc.returncode != 0:
                        raise SystemExit(f"bench: {' '.join(cmd)} failed:\n{proc.stdout}\n{proc.stderr}")
                    rows += [json.loads(line) for line in tmp.read().splitlines() if line.strip()]
            entry = {}
            for r in rows:
                gbps = 2 * 8 * r["bufsize"] / r["avg_us"] / 1e3
                entry[str(r["bufsize"])] = {"avg_us": round(r["avg_us"], 2), "iters": r["iters"], "gbps": round(gbps, 1),
                                            "frac": round(gbps / HBM_PEAK_GBPS, 4)}
            out[f"{buffers}/{streams}"] = entry
    out["harness"] = ("megray_performance -d 8 -f all_reduce -R [-M] [-S]: thread per rank through "
                      "MegRay::Communicator::all_reduce, random inputs, 100 + 500 calls at 10 MiB, 10 + 30 at 128 MiB and 1 GiB")
    return out


def side_leg(leg, *leg_args):
    """Runs one of the legs that report beside the headline in child processes.  A leg that fails (a child that
    exits with an error, or does not come back in time) is reported as {"error": ...} in its place and on stderr:
    the headline measurement does not depend on it."""
    try:
        return leg(*leg_args)
    except (SystemExit, subprocess.SubprocessError, OSError, ValueError, KeyError, IndexError) as failure:
        text = " ".join(str(failure).split())[:600]
        print(f"bench.py: {leg.__name__} failed: {text}", file=sys.stderr)
        return {"error": text}


def other_layout_fresh(args):
    """The headline launches on buffers laid out the OTHER way, in three processes of their own (started before this
    one touches the GPU), beside the measurement this process makes itself after the headline (other_layout's own
    figures, defined as in earlier rounds).  Where the driver puts separately allocated buffers physically is not
    visible to the library and differs from allocation to allocation - one process that allocated, measured and freed
    the same sixteen buffers five times got the same virtual addresses and between 79.5 and 83.3 % of the peak - so
    the record shows the spread: all three in the order they ran, and their median."""
    other = "separate" if args.layout == "placed" else "placed"
    cmd = [sys.executable, os.path.abspath(__file__), "--layout", other, "--steps", str(args.steps), "--warmup", str(args.warmup),
           "--log2n", str(args.log2n), "--ranks", str(args.ranks), "--schedule", args.schedule,
           "--no-cpu", "--no-small", "--no-check", "--no-comm", "--no-others"]
    runs = []
    for _ in range(3):
        proc = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
        if proc.returncode != 0:
            raise SystemExit(f"bench: {' '.join(cmd)} failed:\n{proc.stdout}\n{proc.stderr}")
        child = json.loads([line for line in proc.stdout.splitlines() if line.startswith("{")][-1])
        runs.append((child["roofline"]["frac"], child["roofline"]["kernel_ms"]))
    in_order = [round(100.0 * f, 2) for f, _ in runs]
    runs.sort()
    frac, ms = runs[1]
    return {"median_pct_of_peak": round(100.0 * frac, 2), "median_ms_per_step": ms, "pct_of_peak_in_the_order_they_ran": in_order,
            "process": "three processes of their own, each allocates its sixteen buffers first thing"}


def copy_yardstick(torch, mr):
    """What this particular GPU sustains on the simplest streaming job, for context: a 1 GiB device copy
    through this library's copy kernel and through torch (GB/s, read + write)."""
    from megray_amd import synth
    n = 1 << 30
    src, dst = alloc_buffers(torch, mr, [(n, torch.uint8)] * 2, "placed")
    synth.fill_torch(torch.uint8, n, 0, out=src)  # random bytes: the rate depends on the data (zeros copy faster)
    st = torch.cuda.current_stream()

    def timed(fn):
        for _ in range(3):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(st)
        for _ in range(20):
            fn()
        e1.record(st)
        torch.cuda.synchronize()
        return 2 * n / (e0.elapsed_time(e1) / 20 * 1e-3) / 1e9

    lib = timed(lambda: mr.broadcast(src, [dst], n, mr.DType.UINT8, 0, stream=st))
    tch = timed(lambda: dst.copy_(src))
    return {"library_copy_gbps": round(lib, 1), "torch_copy_gbps": round(tch, 1)}


def cpu_baseline(orc, np, nranks):
    """The reference tests' expected-value loop on the host: single thread (as the reference runs
    it) on a 2^26-element-per-rank sample of the headline workload (the first quarter of every rank's
    buffer), plus the same loop split over all host cores for scale, plus the reference's own ring
    schedule replayed on the host.  About ten seconds of CPU work."""
    from megray_amd import synth
    n = 1 << 26
    ins = [synth.fill_np(np.float32, n, r) for r in range(nranks)]  # the first 2^26 elements of the GPU's buffers
    bmin = 2 * nranks * n * 4

    def timed(threads, reps):
        orc.test_all_reduce_f32(ins, orc.SUM, nthreads=threads)  # warm-up, touches the outputs
        times = []
        for _ in range(reps):
            t0 = time.perf_counter()
            orc.test_all_reduce_f32(ins, orc.SUM, nthreads=threads)
            times.append(time.perf_counter() - t0)
        times.sort()
        return times[len(times) // 2]

    t1 = timed(0, 7)
    cores = min(os.cpu_count() or 1, 16)
    tn = timed(cores, 7)
    # the reference's own schedule on the host: 2(N-1) ring steps of the two-input reduce loop
    # (src/ucx/all_reduce.cpp:53-101 over src/ucx/kernel.cu:16-22), single thread, 2^25 elements per rank
    m = 1 << 25
    part = [a[:m] for a in ins]
    orc.ucx_all_reduce(part, orc.FLOAT32, orc.SUM)
    t0 = time.perf_counter()
    orc.ucx_all_reduce(part, orc.FLOAT32, orc.SUM)
    tr = time.perf_counter() - t0
    return {
        "value": round(bmin / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": f"all_reduce SUM fp32, {nranks} ranks x 2^26 elements, test/test_opr.cpp:321-330 loop, "
                  f"median of 7, {t1 * 1e3:.1f} ms per pass",
        "all_cores": {"value": round(bmin / tn / 1e9, 3), "cores": cores, "ms": round(tn * 1e3, 1)},
        "ring_replay": {"value": round(2 * nranks * m * 4 / tr / 1e9, 3), "cores": 1, "ms": round(tr * 1e3, 1),
                        "sample": f"literal 2(N-1)-step ring replay, {nranks} ranks x 2^25 elements, B_min / t"},
    }


def time_workload(w, torch, mr, steps, warmup, layout="placed"):
    """One of the non-headline workloads: builds its inputs in HBM, times `steps` collectives with HIP
    events on the launch stream and returns the figures."""
    dev = "cuda:0"
    st = torch.cuda.current_stream()
    n8 = 8

    def buffers(n_in, n_out, dtype, count_in=n8, count_out=n8, collective=None):
        """count_in inputs of n_in elements (filled) and count_out outputs of n_out elements."""
        from megray_amd import synth
        bufs = alloc_buffers(torch, mr, [(n_in, dtype)] * count_in + [(n_out, dtype)] * count_out, layout, collective,
                             [0] * count_in + [1] * count_out)
        for rank, t in enumerate(bufs[:count_in]):
            synth.fill_torch(dtype, n_in, rank, "normal" if dtype.is_floating_point else "uniform", device=dev, out=t)
        return bufs[:count_in], bufs[count_in:]

    if w == "copy":
        n = 1 << 30
        src, dst = buffers(n, n, torch.uint8, 1, 1)
        step = lambda: mr.broadcast(src[0], dst, n, mr.DType.UINT8, 0, stream=st)  # noqa: E731
        desc = (mr.Collective.BROADCAST, src, dst, n, mr.DType.UINT8)
        text, dt = "plain copy of 2^30 bytes (one rank, broadcast to itself)", "u8"
    elif w == "c2_reduce_scatter":
        recvlen = 1 << 23
        src, dst = buffers(n8 * recvlen, recvlen, torch.float16)
        step = lambda: mr.reduce_scatter(src, dst, recvlen, mr.DType.FLOAT16, mr.ReduceOp.SUM, stream=st)  # noqa: E731
        desc = (mr.Collective.REDUCE_SCATTER, src, dst, recvlen, mr.DType.FLOAT16)
        text, dt = "reduce_scatter SUM fp16 (fp32 accumulate), 8 ranks x 2^26 elements in, 2^23 out", "f16"
    elif w == "c2_all_gather":
        sendlen = 1 << 23
        src, dst = buffers(sendlen, n8 * sendlen, torch.float16, collective=mr.Collective.ALL_GATHER)
        step = lambda: mr.all_gather(src, dst, sendlen, mr.DType.FLOAT16, stream=st)  # noqa: E731
        desc = (mr.Collective.ALL_GATHER, src, dst, sendlen, mr.DType.FLOAT16)
        text, dt = "all_gather fp16, 8 ranks x 2^23 elements in, 2^26 out", "f16"
    elif w in ("c3_max_int32", "c3_min_int64"):
        tdt, mdt, op = ((torch.int32, mr.DType.INT32, mr.ReduceOp.MAX) if w == "c3_max_int32"
                        else (torch.int64, mr.DType.INT64, mr.ReduceOp.MIN))
        n = 1 << 28
        src, dst = buffers(n, n, tdt)
        step = lambda: mr.all_reduce(src, dst, n, mdt, op, stream=st)  # noqa: E731
        desc = (mr.Collective.ALL_REDUCE, src, dst, n, mdt)
        text, dt = f"all_reduce {op.name} {mdt.name.lower()}, 8 ranks x 2^28 elements", mdt.name.lower()
    elif w == "c5_all_to_all":
        blk = 1 << 24
        src, dst = buffers(n8 * blk, n8 * blk, torch.uint8)
        step = lambda: mr.all_to_all(src, dst, blk, mr.DType.UINT8, stream=st)  # noqa: E731
        desc = (mr.Collective.ALL_TO_ALL, src, dst, blk, mr.DType.UINT8)
        text, dt = "all_to_all uint8, 8 ranks x 8 blocks of 16 MiB", "u8"
    elif w == "c5_sum_int8":
        n = 1 << 27
        src, dst = buffers(n, n, torch.int8)
        step = lambda: mr.all_reduce(src, dst, n, mr.DType.INT8, mr.ReduceOp.SUM, stream=st)  # noqa: E731
        desc = (mr.Collective.ALL_REDUCE, src, dst, n, mr.DType.INT8)
        text, dt = "all_reduce SUM int8 (wrap-around), 8 ranks x 2^27 elements", "i8"
    else:
        raise SystemExit(f"bench: unknown workload {w}")

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(st)
    for _ in range(steps):
        step()
    e1.record(st)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    runs, bytes_read, bytes_written = mr.describe(desc[0], desc[1], desc[2], desc[3], desc[4])
    launches = max(1, len({r["step"] for r in runs}))
    executed = bytes_read + bytes_written  # these workloads run in one pass: executed bytes = B_min
    kernel_ms = e0.elapsed_time(e1) / steps / launches
    achieved = executed / launches / (kernel_ms * 1e-3) / 1e9
    del src, dst
    torch.cuda.empty_cache()
    return {"workload": text, "dtype": dt, "launches": launches, "bytes": executed, "wall_s": wall,
            "kernel_ms": kernel_ms, "achieved": achieved, "traffic": measured_traffic(w)}


def run_other_workload(args, torch, mr):
    """A non-headline workload on its own: same timing, one JSON line, no CPU / small-message legs."""
    r = time_workload(args.workload, torch, mr, args.steps, args.warmup, args.layout)
    value = r["bytes"] / (r["wall_s"] / args.steps) / 1e9
    print(json.dumps({
        "metric": "achieved HBM GB/s (% of peak)", "value": round(value, 1), "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(r["wall_s"] * 1e3 / args.steps, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": r["dtype"], "data": "synthetic",
        "config": {"workload": r["workload"], "launches_per_step": r["launches"], "layout": args.layout},
        "pct_of_peak": round(100.0 * value / HBM_PEAK_GBPS, 2), "bytes_executed": r["bytes"],
        "roofline": {"bound": "hbm", "achieved": round(r["achieved"], 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(r["achieved"] / HBM_PEAK_GBPS, 4), "traffic": r["traffic"],
                     "kernel_ms": round(r["kernel_ms"], 4),
                     "algorithmic_bytes_per_launch": r["bytes"] // r["launches"]},
    }))
    return 0


def other_configs(torch, mr, layout):
    """The other benchmark configurations, twenty timed steps each after five warm-up steps (a hundred after fifty for the
    launches of a few hundred microseconds): milliseconds per collective (HIP events),
    GB/s on the collective's minimum bytes (which is what each of them executes) and that as a fraction of
    the HBM peak."""
    out = {}
    for w in ("c2_reduce_scatter", "c2_all_gather", "c3_max_int32", "c3_min_int64", "c5_all_to_all", "c5_sum_int8"):
        # launches of a few hundred microseconds get more steps: twenty of them are over before the clocks have settled
        steps, warmup = (20, 5) if w.startswith("c3") else (100, 50)
        r = time_workload(w, torch, mr, steps, warmup, layout)
        out[w] = {"workload": r["workload"], "ms": round(r["kernel_ms"] * r["launches"], 4),
                  "gbps": round(r["achieved"], 1), "frac": round(r["achieved"] / HBM_PEAK_GBPS, 4),
                  "bytes_min": r["bytes"], "traffic": r["traffic"]}
    return out


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU; the N ranks are virtual ranks inside it "
              "(use --gpus 1, rank count is --ranks)", file=sys.stderr)
        return 2
    headline = args.workload == "all_reduce"
    # the thread-per-rank legs and the other layout's processes run as children, before this process touches the GPU
    comm_api = side_leg(comm_api_sweep) if headline and not args.no_comm else None
    comm_large = side_leg(comm_api_large) if headline and not args.no_comm and args.log2n == 28 else None
    other_fresh = side_leg(other_layout_fresh, args) if headline and not args.no_others else None

    import numpy as np
    import torch

    import megray_amd as mr
    from megray_amd import _lib

    _lib.load()  # fails loudly when the HIP library is not built
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    if args.workload != "all_reduce":
        return run_other_workload(args, torch, mr)
    nranks, n = args.ranks, 1 << args.log2n
    sched = {"fused": mr.Schedule.FUSED, "two_phase": mr.Schedule.TWO_PHASE, "ring": mr.Schedule.RING}[args.schedule]

    if not args.no_check:
        import oracle as orc
        check_small(torch, mr, orc, np)

    st = torch.cuda.current_stream()

    def timed(ins, outs, steps, warmup):
        """-> (wall seconds, HIP-event milliseconds) of `steps` collectives after `warmup` untimed ones."""
        def step():
            mr.all_reduce(ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, order=mr.FoldOrder.UCX, schedule=sched,
                          stream=st)

        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(st)
        for _ in range(steps):
            step()
        e1.record(st)
        torch.cuda.synchronize()
        return time.perf_counter() - t0, e0.elapsed_time(e1)

    ins, outs = make_buffers(torch, mr, nranks, n, args.layout)
    wall, event_ms = timed(ins, outs, args.steps, args.warmup)

    if not args.no_check:
        check_full(torch, mr, ins, outs, n)

    ms_per_step = wall * 1e3 / args.steps
    bmin = 2 * nranks * n * 4
    runs, bytes_read, bytes_written = mr.describe(mr.Collective.ALL_REDUCE, ins, outs, n, mr.DType.FLOAT32,
                                                  mr.FoldOrder.UCX, sched)
    launches = len({r["step"] for r in runs})
    executed = bytes_read + bytes_written
    value = bmin / (wall / args.steps) / 1e9
    kernel_ms = event_ms / args.steps / launches  # average launch duration over the timed region
    achieved = (executed / launches) / (kernel_ms * 1e-3) / 1e9
    key = f"all_reduce_f32_n{nranks}_2p{args.log2n}_{args.schedule}"
    result = {
        "metric": f"achieved HBM GB/s (% of peak) for {nranks}-rank fp32 SUM all_reduce; small-msg µs",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic: uniform[-1,1) fp32, counter-based splitmix64 of (0x4D656752 + rank) xor golden*index",
        "config": {
            "workload": f"all_reduce SUM fp32, {nranks} virtual ranks x 2^{args.log2n} elements, ucx ring order, "
                        f"{args.schedule} schedule, buffers resident in HBM",
            "layout": LAYOUT_TEXT[args.layout],
            "ranks": nranks, "elements_per_rank": n, "order": "ucx", "schedule": args.schedule,
            "launches_per_step": launches,
        },
        "pct_of_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "bytes_min": bmin,
        "bytes_executed": executed,
        "roofline": {
            "bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": measured_traffic(key),
            "kernel": "fold_group_kernel<float, SUM, K=8>" if args.schedule == "fused" else "fold kernels (several)",
            "kernel_ms": round(kernel_ms, 4), "algorithmic_bytes_per_launch": executed // launches,
        },
    }
    del ins, outs
    torch.cuda.empty_cache()
    if not args.no_others:  # the same launches on buffers placed the other way, for the record
        other = "separate" if args.layout == "placed" else "placed"
        ins, outs = make_buffers(torch, mr, nranks, n, other)
        _, other_ms = timed(ins, outs, args.steps, args.warmup)  # timed like the headline
        same = {"ms_per_step": round(other_ms / args.steps, 4),
                "pct_of_peak": round(100.0 * bmin / (other_ms / args.steps * 1e-3) / 1e9 / HBM_PEAK_GBPS, 2),
                "process": "this one, after the headline's buffers were allocated and freed"}
        result["other_layout"] = dict(same, layout=LAYOUT_TEXT[other], steps=args.steps, warmup=args.warmup)
        if other_fresh:
            result["other_layout"]["processes_of_their_own"] = other_fresh
        del ins, outs
        torch.cuda.empty_cache()
    props = torch.cuda.get_device_properties(0)
    result["device"] = {"name": props.name, "compute_units": props.multi_processor_count,
                        "hbm_gib": round(props.total_memory / 2 ** 30, 1)}
    result["copy_yardstick"] = copy_yardstick(torch, mr)
    if not args.no_small:
        result["small_msg_us"] = small_message_sweep(torch, mr)
    if comm_api is not None:
        result["comm_api_us"] = comm_api
    if comm_large is not None:
        result["comm_api_large"] = comm_large
    if not args.no_others:
        result["other_configs"] = other_configs(torch, mr, args.layout)
    if not args.no_cpu:
        import oracle as orc
        result["cpu_baseline"] = cpu_baseline(orc, np, nranks)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
