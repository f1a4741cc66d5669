"""The allocation-free all_reduce of the thread-per-rank API (mrv_comm_all_reduce_no_alloc) against
mrv_comm_all_reduce: same inputs, bit-identical outputs, on two calls in a row (the second with a
smaller input), every rank on a stream of its own so that the counters in the library's static
device array carry all the ordering.  Also: the group takes a counter block only once, and the 33rd
group alive at the same time is turned away with a clear message."""
import threading

import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import empty_device, to_device, to_host  # noqa: E402


def make_group(nranks):
    port = mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r, mr.Backend.VRANK) for r in range(nranks)]
    threads = [threading.Thread(target=comms[r].init, args=("localhost", port), daemon=True) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
        assert not t.is_alive(), "init hung"
    return comms


def run_ranks(nranks, body):
    errors = []

    def main(rank):
        try:
            torch.cuda.set_device(0)
            body(rank)
        except BaseException as exc:  # noqa: BLE001
            errors.append((rank, repr(exc)))

    threads = [threading.Thread(target=main, args=(r,), daemon=True) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
        assert not t.is_alive(), "a rank hung"
    assert not errors, errors


def test_no_alloc_all_reduce_matches_all_reduce_two_calls_in_a_row():
    nranks = 8
    comms = make_group(nranks)
    rng = np.random.default_rng(20240607)
    # first a launch of many tiles (separate wait / notify kernels), then a short one (ordering inside the fold kernel)
    lengths = [(1 << 20) + 77, 12345]
    inputs = [[rng.uniform(-1, 1, n).astype(np.float32) for _ in range(nranks)] for n in lengths]
    results = {"plain": [[None] * nranks for _ in lengths], "fixed": [[None] * nranks for _ in lengths]}

    def body(rank):
        comm = comms[rank]
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            for which in ("fixed", "plain"):
                call = comm.all_reduce_no_alloc if which == "fixed" else comm.all_reduce
                outs = []
                for i, n in enumerate(lengths):  # two calls in a row, no synchronisation in between
                    src = to_device(inputs[i][rank])
                    dst = empty_device(n * 4)
                    call(src, dst, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                    outs.append((src, dst))
                stream.synchronize()
                for i, (_, dst) in enumerate(outs):
                    results[which][i][rank] = to_host(dst, np.float32)

    run_ranks(nranks, body)
    for i, n in enumerate(lengths):
        want = orc.ucx_all_reduce(inputs[i], orc.FLOAT32, orc.SUM)
        for r in range(nranks):
            fixed, plain = results["fixed"][i][r], results["plain"][i][r]
            assert np.array_equal(fixed.view(np.uint32), plain.view(np.uint32)), f"call {i} rank {r}: differs from all_reduce"
            assert np.array_equal(fixed.view(np.uint32), want[r].view(np.uint32)), f"call {i} rank {r}: differs from the oracle"
    for c in comms:
        c.close()


def test_no_alloc_leaves_the_device_memory_as_it_finds_it():
    """What the entry point is for: between a group's first call through it and its last, the free device memory
    does not change (no hipMalloc, no hipFree).  Buffers are allocated and the kernels loaded (by another group)
    beforehand; the calls take the short launch and the one between wait and notify kernels, a stream per rank.
    (Host-side allocations the free-memory figure cannot see - pinned memory, events - are counted on the simulated
    streams of tests/test_stream_sim.py, mode "fixed".)"""
    nranks = 4
    lengths = [777, (1 << 19) + 5]
    rng = np.random.default_rng(99)
    inputs = [[rng.integers(-1000, 1000, n).astype(np.int32) for _ in range(nranks)] for n in lengths]
    warm, comms = make_group(nranks), make_group(nranks)
    bufs = [[(to_device(inputs[i][r]), empty_device(n * 4)) for i, n in enumerate(lengths)] for r in range(nranks)]
    streams = [torch.cuda.Stream() for _ in range(nranks)]
    free = {}

    def run(group, rank, rounds):
        for _ in range(rounds):
            for i, n in enumerate(lengths):
                src, dst = bufs[rank][i]
                group[rank].all_reduce_no_alloc(src, dst, n, mr.DType.INT32, mr.ReduceOp.SUM, streams[rank])
        streams[rank].synchronize()

    run_ranks(nranks, lambda rank: run(warm, rank, 1))
    torch.cuda.synchronize()
    free["before"] = torch.cuda.mem_get_info()[0]
    run_ranks(nranks, lambda rank: run(comms, rank, 3))
    torch.cuda.synchronize()
    free["after"] = torch.cuda.mem_get_info()[0]
    assert free["after"] == free["before"], free
    for i, n in enumerate(lengths):
        want = sum(x.astype(np.int64) for x in inputs[i]).astype(np.int32)
        for r in range(nranks):
            assert np.array_equal(to_host(bufs[r][i][1], np.int32), want)
    for c in warm + comms:
        c.close()


def test_no_alloc_rejects_a_mixed_collective_and_runs_out_of_blocks_cleanly():
    nranks = 2
    groups = [make_group(nranks) for _ in range(33)]
    data = [np.arange(64, dtype=np.int32) * (r + 1) for r in range(nranks)]

    def use(index):
        comms = groups[index]
        outs = [None] * nranks
        errs = [None] * nranks

        def body(rank):
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                src, dst = to_device(data[rank]), empty_device(64 * 4)
                try:
                    comms[rank].all_reduce_no_alloc(src, dst, 64, mr.DType.INT32, mr.ReduceOp.SUM, stream)
                    stream.synchronize()
                    outs[rank] = to_host(dst, np.int32)
                except mr.MegRayError as exc:
                    errs[rank] = str(exc)

        run_ranks(nranks, body)
        return outs, errs

    for g in range(32):  # 32 groups hold the 32 blocks
        outs, errs = use(g)
        assert errs == [None, None], errs
        for r in range(nranks):
            assert np.array_equal(outs[r], data[0] + data[1])
    outs, errs = use(32)  # the 33rd is turned away, on every rank, with the reason
    assert all(e is not None for e in errs), (outs, errs)
    for c in groups[0]:
        c.close()
    groups[0] = None
    # a block has come free: a group that has not tried yet gets it (and finds it cleared)
    fresh = make_group(nranks)
    groups.append(fresh)
    outs, errs = use(33)
    assert errs == [None, None], errs
    for r in range(nranks):
        assert np.array_equal(outs[r], data[0] + data[1])
    # one rank through this entry point, the other through all_reduce: a mismatch like any other
    mixed = groups[1]
    errs = [None] * nranks

    def body(rank):
        stream = torch.cuda.Stream()
        with torch.cuda.stream(stream):
            src, dst = to_device(data[rank]), empty_device(64 * 4)
            call = mixed[rank].all_reduce_no_alloc if rank == 0 else mixed[rank].all_reduce
            try:
                call(src, dst, 64, mr.DType.INT32, mr.ReduceOp.SUM, stream)
            except mr.MegRayError as exc:
                errs[rank] = str(exc)
            stream.synchronize()

    run_ranks(nranks, body)
    assert all(e and "different collectives" in e for e in errs), errs
    assert errs[0] == errs[1]  # every rank is told the same
    for comms in groups:
        if comms:
            for c in comms:
                c.close()
