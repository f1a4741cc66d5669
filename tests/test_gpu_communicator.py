"""The MegRay::Communicator API on the GPU, driven the way the reference drives it
(test/test_base.h:26-62): create_server on a free port, N communicators in one process, one thread
per rank doing init -> alloc -> copy in -> collective -> sync -> copy out, then compare.  Inputs and
expectations are the closed forms of test/test_opr.cpp (cited per test), plus seeded random data
against the oracle."""
import threading

import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import bits_equal, empty_device, rand_array, to_device, to_host  # noqa: E402


def run_test(nranks, inputs, expected, main_func, own_streams=True, configure=None):
    """Mirror of run_test<T> (test/test_base.h:26-62)."""
    port = mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r, mr.Backend.VRANK) for r in range(nranks)]
    outputs = [None] * nranks
    errors = []

    def rank_main(rank):
        try:
            torch.cuda.set_device(0)  # every virtual rank lives on the one GPU
            comm = comms[rank]
            comm.init("localhost", port)
            if configure:
                comm.configure(*configure)
            stream = torch.cuda.Stream() if own_streams else torch.cuda.current_stream()
            outputs[rank] = main_func(comm, rank, inputs[rank], stream)
        except BaseException as exc:  # noqa: BLE001
            errors.append((rank, repr(exc)))

    threads = [threading.Thread(target=rank_main, args=(r,), daemon=True) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
        assert not t.is_alive(), "a rank hung"
    assert not errors, errors
    for r in range(nranks):
        if expected[r] is not None:
            assert bits_equal(outputs[r], expected[r]), f"rank {r}: {outputs[r]} != {expected[r]}"
    for c in comms:
        c.close()


def f32(values):
    return np.array(values, dtype=np.float32)


def test_send_recv():
    # test/test_opr.cpp:63-99: rank 0 sends "test_message" as CHAR to rank 1
    msg = np.frombuffer(b"test_message", dtype=np.uint8).copy()

    def main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            if rank == 0:
                buf = to_device(inp)
                comm.send(buf, msg.size, mr.DType.CHAR, 1, stream)
                stream.synchronize()
                return None
            buf = empty_device(msg.size)
            comm.recv(buf, msg.size, mr.DType.CHAR, 0, stream)
            stream.synchronize()
            return to_host(buf, np.uint8)

    run_test(2, [msg, None], [None, msg], main)


def test_grouped_exchange_does_not_deadlock():
    # both ranks send first, then receive: only works inside group_start / group_end
    n = 1000
    data = [np.arange(n, dtype=np.int32) * (r + 1) for r in range(2)]

    def main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src, dst = to_device(inp), empty_device(n * 4)
            comm.group_start()
            comm.send(src, n, mr.DType.INT32, 1 - rank, stream)
            comm.recv(dst, n, mr.DType.INT32, 1 - rank, stream)
            comm.group_end()
            stream.synchronize()
            return to_host(dst, np.int32)

    run_test(2, data, [data[1], data[0]], main)


def test_scatter_gather():
    nranks, length, root = 3, 10, 1
    # test/test_opr.cpp:101-146
    root_in = f32([(i + 1) * (j + 2) for i in range(nranks) for j in range(length)])
    parts = [f32([(i + 1) * (j + 2) for j in range(length)]) for i in range(nranks)]

    def scatter_main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            out = empty_device(length * 4)
            src = to_device(inp) if rank == root else None  # non-root passes nullptr (:133-135)
            comm.scatter(src, out, length, mr.DType.FLOAT32, root, stream)
            stream.synchronize()
            return to_host(out, np.float32)

    run_test(nranks, [root_in if r == root else None for r in range(nranks)], parts, scatter_main)

    # test/test_opr.cpp:148-196
    def gather_main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src = to_device(inp)
            out = empty_device(nranks * length * 4) if rank == root else None
            comm.gather(src, out, length, mr.DType.FLOAT32, root, stream)
            stream.synchronize()
            return to_host(out, np.float32) if rank == root else None

    run_test(nranks, parts, [root_in if r == root else None for r in range(nranks)], gather_main)


def test_all_to_all_and_all_gather():
    nranks, length = 3, 6
    # test/test_opr.cpp:198-241
    ins = [f32([(i + 1) * (j + 2) * (k + 3) for j in range(nranks) for k in range(length)]) for i in range(nranks)]
    outs = [f32([(i + 1) * (j + 2) * (k + 3) for i in range(nranks) for k in range(length)]) for j in range(nranks)]

    def a2a_main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src, dst = to_device(inp), empty_device(nranks * length * 4)
            comm.all_to_all(src, dst, length, mr.DType.FLOAT32, stream)
            stream.synchronize()
            return to_host(dst, np.float32)

    run_test(nranks, ins, outs, a2a_main)

    # test/test_opr.cpp:243-284
    sendlen = 10
    ins = [f32([(i + 1) * (j + 1) for j in range(sendlen)]) for i in range(nranks)]
    want = np.concatenate(ins)

    def ag_main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src, dst = to_device(inp), empty_device(nranks * sendlen * 4)
            comm.all_gather(src, dst, sendlen, mr.DType.FLOAT32, stream)
            stream.synchronize()
            return to_host(dst, np.float32)

    run_test(nranks, ins, [want] * nranks, ag_main)


@pytest.mark.parametrize("own_streams", [True, False])
def test_all_reduce_closed_forms(own_streams):
    # test/test_opr.cpp:286-359
    nranks, length = 3, 10
    ins = [f32([(i + 1) * (j + 1) for j in range(length)]) for i in range(nranks)]
    j1 = np.arange(1, length + 1, dtype=np.float32)
    for op, want in ((mr.ReduceOp.SUM, 6 * j1), (mr.ReduceOp.MAX, 3 * j1), (mr.ReduceOp.MIN, j1)):
        def main(comm, rank, inp, stream, op=op):
            with torch.cuda.stream(stream):
                src, dst = to_device(inp), empty_device(length * 4)
                comm.all_reduce(src, dst, length, mr.DType.FLOAT32, op, stream)
                stream.synchronize()
                return to_host(dst, np.float32)

        run_test(nranks, ins, [want] * nranks, main, own_streams=own_streams)


def test_reduce_scatter_closed_forms():
    # test/test_opr.cpp:361-438
    nranks, recvlen = 3, 10
    ins = [f32([(i + 1) * (m + 1) for m in range(nranks * recvlen)]) for i in range(nranks)]
    for op, factor in ((mr.ReduceOp.SUM, 6), (mr.ReduceOp.MAX, 3), (mr.ReduceOp.MIN, 1)):
        want = [f32([factor * (k * recvlen + j + 1) for j in range(recvlen)]) for k in range(nranks)]

        def main(comm, rank, inp, stream, op=op):
            with torch.cuda.stream(stream):
                src, dst = to_device(inp), empty_device(recvlen * 4)
                comm.reduce_scatter(src, dst, recvlen, mr.DType.FLOAT32, op, stream)
                stream.synchronize()
                return to_host(dst, np.float32)

        run_test(nranks, ins, want, main)


def test_broadcast_and_reduce_closed_forms():
    nranks, root, length = 3, 1, 10
    ins = [f32([(i + 1) * (j + 1) for j in range(length)]) for i in range(nranks)]

    # test/test_opr.cpp:440-485
    def bcast_main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src, dst = to_device(inp), empty_device(length * 4)
            comm.broadcast(src, dst, length, mr.DType.FLOAT32, root, stream)
            stream.synchronize()
            return to_host(dst, np.float32)

    run_test(nranks, ins, [ins[root]] * nranks, bcast_main)

    # test/test_opr.cpp:487-551: only the root allocates a receive buffer
    j1 = np.arange(1, length + 1, dtype=np.float32)
    for op, want in ((mr.ReduceOp.SUM, 6 * j1), (mr.ReduceOp.MAX, 3 * j1), (mr.ReduceOp.MIN, j1)):
        def reduce_main(comm, rank, inp, stream, op=op):
            with torch.cuda.stream(stream):
                src = to_device(inp)
                dst = empty_device(length * 4) if rank == root else None
                comm.reduce(src, 0xDEAD0000 if dst is None else dst, length, mr.DType.FLOAT32, op, root, stream)
                stream.synchronize()
                return to_host(dst, np.float32) if rank == root else None

        run_test(nranks, ins, [want if r == root else None for r in range(nranks)], reduce_main)


@pytest.mark.parametrize("nranks", [2, 4, 8, 20])
def test_random_data_orders_and_work_queued_on_rank_streams(nranks):
    """Seeded random fp32 through the thread-per-rank API equals the oracle's literal ucx ring replay;
    with SHM order it equals the shm replay.  Each rank fills its input ON ITS OWN STREAM right before
    the collective and reads the result on it right after, so a missing cross-stream dependency
    would show as stale data."""
    rng = np.random.default_rng(nranks)
    length = 1 << 18
    ins = [rand_array(orc.FLOAT32, length, rng) for _ in range(nranks)]
    for order, want in ((mr.FoldOrder.UCX, orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM)),
                        (mr.FoldOrder.SHM, orc.shm_all_reduce(ins, orc.FLOAT32, orc.SUM))):
        def main(comm, rank, inp, stream):
            with torch.cuda.stream(stream):
                staged = torch.from_numpy(inp.view(np.uint8).copy()).pin_memory()
                src = torch.empty(length * 4, dtype=torch.uint8, device="cuda:0")
                dst = torch.full((length * 4,), 0x5A, dtype=torch.uint8, device="cuda:0")
                host_out = torch.empty(length * 4, dtype=torch.uint8).pin_memory()
                for _ in range(3):  # several rounds back to back, no host sync in between
                    src.copy_(staged, non_blocking=True)
                    comm.all_reduce(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                    host_out.copy_(dst, non_blocking=True)
                stream.synchronize()
                return host_out.numpy().view(np.float32).copy()

        run_test(nranks, ins, want, main, configure=(order, mr.Schedule.FUSED))

    want = orc.ucx_reduce(ins, orc.FLOAT32, orc.SUM, nranks - 1)

    def reduce_main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src, dst = to_device(inp), empty_device(length * 4)
            comm.reduce(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, nranks - 1, stream)
            stream.synchronize()
            return to_host(dst, np.float32)

    run_test(nranks, ins, [want[r] if r == nranks - 1 else None for r in range(nranks)], reduce_main)


def test_ranks_that_share_a_stream_and_ranks_that_stop_sharing_it():
    """Ranks on one stream need no cross-stream edges, and a rank skips marking its stream when everyone
    shared it last time.  First pass: all four ranks on the default stream.  Second pass: ranks 1 and 3 move to
    streams of their own, fill their inputs there right before the collective and read the result there
    right after - the leader has to insert the edges those ranks did not announce.  Third pass: all share
    again."""
    nranks, length = 4, 1 << 16
    rng = np.random.default_rng(99)
    rounds = [[rand_array(orc.FLOAT32, length, rng) for _ in range(nranks)] for _ in range(3)]
    wants = [orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM) for ins in rounds]
    shared = torch.cuda.current_stream()
    gate = threading.Barrier(nranks)

    def main(comm, rank, _inp, _stream):
        outs = []
        own = torch.cuda.Stream()
        for rnd in range(3):
            stream = own if (rnd == 1 and rank in (1, 3)) else shared
            staged = torch.from_numpy(rounds[rnd][rank].view(np.uint8).copy()).pin_memory()
            host_out = torch.empty(length * 4, dtype=torch.uint8).pin_memory()
            with torch.cuda.stream(stream):
                src = torch.empty(length * 4, dtype=torch.uint8, device="cuda:0")
                dst = torch.full((length * 4,), 0x5A, dtype=torch.uint8, device="cuda:0")
                src.copy_(staged, non_blocking=True)
                comm.all_reduce(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                host_out.copy_(dst, non_blocking=True)
            stream.synchronize()
            outs.append(host_out.numpy().view(np.float32).copy())
            gate.wait(60)  # keep the rounds apart: on the shared stream they would order themselves anyway
        return np.concatenate(outs)

    expected = [np.concatenate([wants[rnd][r] for rnd in range(3)]) for r in range(nranks)]
    run_test(nranks, [None] * nranks, expected, main, own_streams=False)


def test_contract_violations_throw_on_the_calling_rank():
    nranks = 2
    port = mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r) for r in range(nranks)]
    threads = [threading.Thread(target=comms[r].init, args=("localhost", port)) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
    buf = empty_device(64)
    with pytest.raises(mr.MegRayError, match="unknown dtype"):      # src/ucx/kernel.cu:95-96
        comms[0].all_reduce(buf, buf, 16, mr.DType.CHAR, mr.ReduceOp.SUM)
    with pytest.raises(mr.MegRayError, match="unknown reduce op"):  # src/ucx/kernel.cu:55-56
        comms[0].all_reduce(buf, buf, 16, mr.DType.FLOAT32, 7)
    with pytest.raises(mr.MegRayError, match="unknown dtype"):      # src/core/common.cpp:35-36
        comms[0].all_gather(buf, buf, 1, 42)
    with pytest.raises(mr.MegRayError):
        comms[0].broadcast(buf, buf, 1, mr.DType.FLOAT32, 5)
    fresh = mr.get_communicator(2, 0)
    with pytest.raises(mr.MegRayError):
        fresh.all_reduce(buf, buf, 16, mr.DType.FLOAT32, mr.ReduceOp.SUM)  # before init()


def test_parked_ranks_are_released_when_another_rank_rejects_its_arguments():
    """Two ranks are already waiting in all_reduce, each on a stream of its own, when the third calls with a
    dtype no reduce exists for: the third throws as the reference does (src/ucx/kernel.cu:95-96), the two get
    MEGRAY_INVALID_USAGE with the same text, and the group goes on to the next collective as if nothing had been."""
    import time
    nranks, n = 3, 1000
    port = mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r, mr.Backend.VRANK) for r in range(nranks)]
    data = [np.arange(n, dtype=np.float32) * (r + 1) for r in range(nranks)]
    results, messages = [None] * nranks, [None] * nranks
    errors = []

    def rank_main(rank):
        try:
            torch.cuda.set_device(0)
            comm = comms[rank]
            comm.init("localhost", port)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                src, dst = to_device(data[rank]), empty_device(n * 4)
                if rank == 2:
                    time.sleep(0.3)  # the others are parked by now
                try:
                    comm.all_reduce(src, dst, n, mr.DType.CHAR if rank == 2 else mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                except mr.MegRayError as exc:
                    messages[rank] = (exc.status, exc.message)
                comm.all_reduce(src, dst, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)  # the group still works
                stream.synchronize()
                results[rank] = to_host(dst, np.float32)
        except BaseException as exc:  # noqa: BLE001
            errors.append((rank, repr(exc)))

    threads = [threading.Thread(target=rank_main, args=(r,), daemon=True) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
        assert not t.is_alive(), "a rank hung"
    assert not errors, errors
    assert messages[2][0] == mr.Status.INVALID_ARGUMENT and "unknown dtype" in messages[2][1]
    assert messages[0] == messages[1]
    assert messages[0][0] == mr.Status.INVALID_USAGE and "rank 2 left the collective: unknown dtype" in messages[0][1]
    want = orc.ucx_all_reduce(data, orc.FLOAT32, orc.SUM)
    for r in range(nranks):
        assert bits_equal(results[r], want[r])
    for c in comms:
        c.close()


def test_a_stream_wait_that_nothing_satisfies_gives_up_at_its_limit():
    """The kernels that make one stream wait for another poll a counter and give up after a time limit, so that a
    lost mark cannot hold a wavefront (and the stream behind it) for ever.  Forced from the host: a wait for a count
    nothing raises, with limits of 200 us and 20 ms; the kernel ends by itself, reports one wait given up, and
    takes about as long as its limit."""
    import time
    stream = torch.cuda.Stream()
    for limit_us in (200, 20000):
        t0 = time.perf_counter()
        gave_up = mr.probe_bounded_wait(limit_us, stream)
        elapsed_us = (time.perf_counter() - t0) * 1e6
        assert gave_up == 1
        assert elapsed_us >= limit_us * 0.9, (limit_us, elapsed_us)
        assert elapsed_us < limit_us + 500000, (limit_us, elapsed_us)


def test_init_through_the_callers_own_broadcast():
    """Communicator::init(BcastCallback) (include/megray/communicator.h:49, src/core/communicator.cpp:23-25): no
    bootstrap server; the group is formed through a broadcast the caller supplies (here a slot in host memory that
    rank 0 fills and the others wait for), the way the reference's NCCL backend passes its unique id through the
    callback (src/nccl/communicator.cpp:54-64).  Then an all_reduce of seeded data against the oracle."""
    nranks, n = 5, 4099
    rng = np.random.default_rng(606)
    data = [rand_array(orc.FLOAT32, n, rng, wide=False) for _ in range(nranks)]
    want = orc.ucx_all_reduce(data, orc.FLOAT32, orc.SUM)
    comms = [mr.get_communicator(nranks, r, mr.Backend.VRANK) for r in range(nranks)]
    slot, filled = {}, threading.Event()
    results, errors, seen = [None] * nranks, [], [None] * nranks

    def rank_main(rank):
        try:
            torch.cuda.set_device(0)

            def broadcast(mine):
                if rank == 0:
                    slot["id"] = bytes(mine)
                    filled.set()
                else:
                    assert filled.wait(60), "rank 0 never broadcast"
                seen[rank] = slot["id"]
                return slot["id"]

            comms[rank].init_callback(broadcast)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                src, dst = to_device(data[rank]), empty_device(n * 4)
                comms[rank].all_reduce(src, dst, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                stream.synchronize()
                results[rank] = to_host(dst, np.float32)
        except BaseException as exc:  # noqa: BLE001
            errors.append((rank, repr(exc)))

    threads = [threading.Thread(target=rank_main, args=(r,), daemon=True) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(120)
        assert not t.is_alive(), "a rank hung"
    assert not errors, errors
    assert len(seen[0]) == 16 and any(seen[0]) and all(s == seen[0] for s in seen)  # one 128-bit id, rank 0's
    for r in range(nranks):
        assert bits_equal(results[r], want[r])
    for c in comms:
        c.close()


@pytest.mark.parametrize("entry", ["all_reduce", "all_reduce_no_alloc"])
@pytest.mark.parametrize("length", [3000, 1 << 20])
def test_a_stream_wait_that_gives_up_poisons_its_group(entry, length, monkeypatch):
    """A rank whose stream does not get to the collective within the wait limit: forced from the host with a limit of
    250 ms and a rank whose stream is kept busy with well over a second of its own work before the call.  Every kernel ends
    normally.  What must hold: the collective that could not wait long enough stores NOTHING (its inputs were not
    ready), the streams behind it are let go at once rather than each waiting out its own limit, and from then on
    every call of the group fails with MEGRAY_UNEXPECTED_ERR and says why - at the very next call for groups whose
    counters report to pinned host memory, after mrv_comm_check or within one and a half limits for a group that
    only uses the allocation-free entry point.  The lengths take the short launch that waits inside the fold kernel
    and the group launch between wait and notify kernels."""
    import time
    monkeypatch.setenv("MEGRAY_VRANK_WAIT_LIMIT_MS", "250")
    nranks, fill = 2, 0x3C
    rng = np.random.default_rng(length)
    data = [rand_array(orc.FLOAT32, length, rng, wide=False) for _ in range(nranks)]
    want = orc.ucx_all_reduce(data, orc.FLOAT32, orc.SUM)
    port = mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r, mr.Backend.VRANK) for r in range(nranks)]
    ballast = torch.ones(1 << 28, dtype=torch.float32, device="cuda:0")  # 1 GiB: ~0.6 ms per pass over it
    first, late, after, errors = [None] * nranks, [None] * nranks, [[] for _ in range(nranks)], []
    barrier = threading.Barrier(nranks)

    def rank_main(rank):
        try:
            torch.cuda.set_device(0)
            comm = comms[rank]
            comm.init("localhost", port)
            call = getattr(comm, entry)
            stream = torch.cuda.Stream()
            with torch.cuda.stream(stream):
                src = to_device(data[rank])
                dst = empty_device(length * 4, fill=fill)
                stream.synchronize()
                barrier.wait(60)  # both ranks are ready: nobody's stream waits long for the other
                call(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)  # a healthy collective first
                stream.synchronize()
                first[rank] = to_host(dst, np.float32)
                dst.fill_(fill)
                stream.synchronize()
                barrier.wait(60)
                if rank == 1:  # well over a second of work in front of this rank's call
                    for _ in range(3000):
                        ballast.mul_(1.0)
                call(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)  # enqueued all the same: returns OK
                t0 = time.perf_counter()
                stream.synchronize()
                waited = time.perf_counter() - t0
                late[rank] = (to_host(dst, np.uint8).copy(), waited)
                barrier.wait(60)
                if entry == "all_reduce_no_alloc":
                    with pytest.raises(mr.MegRayError) as info:
                        comm.check(stream)
                    after[rank].append((info.value.status, info.value.message))
                for _ in range(2):  # and it stays that way
                    with pytest.raises(mr.MegRayError) as info:
                        call(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                    after[rank].append((info.value.status, info.value.message))
                stream.synchronize()
        except BaseException as exc:  # noqa: BLE001
            errors.append((rank, repr(exc)))
            barrier.abort()

    threads = [threading.Thread(target=rank_main, args=(r,), daemon=True) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(180)
        assert not t.is_alive(), "a rank hung"
    assert not errors, errors
    for r in range(nranks):
        assert bits_equal(first[r], want[r])
        untouched, waited = late[r]
        assert bool((untouched == fill).all()), f"rank {r}: the collective that could not wait stored something"
        assert waited < 8.0, f"rank {r} waited {waited:.1f} s"
        for status, message in after[r]:
            assert status == mr.Status.UNEXPECTED_ERR and "gave up" in message, (status, message)
    for c in comms:
        c.close()


@pytest.mark.parametrize("length", [3000, 30000, 70000, 100000, (1 << 19) + 11])
def test_back_to_back_rounds_with_fresh_data_on_rank_streams(length):
    """Five all_reduces back to back, every round with different inputs that each rank copies into the SAME device
    buffer on its own stream right before the call, and with the result copied out of the SAME device buffer on
    that stream right after, no host synchronisation in between.  A collective that started before some rank's
    copy-in had landed, or a copy-in that overtook the previous collective's reads, or a copy-out that overtook
    the collective's writes, shows as a wrong round.  The lengths run the short kernel that carries the stream
    ordering itself (12 and 118 tiles), the short kernel between separate wait / notify kernels (274 and 391 tiles) and the
    group kernel between them (2049 tiles)."""
    nranks, rounds = 8, 5
    rng = np.random.default_rng(length)
    data = [[rand_array(orc.FLOAT32, length, rng) for _ in range(nranks)] for _ in range(rounds)]
    wants = [orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM) for ins in data]
    outs = [[None] * nranks for _ in range(rounds)]

    def main(comm, rank, _inp, stream):
        with torch.cuda.stream(stream):
            staged = [torch.from_numpy(data[r][rank].view(np.uint8).copy()).pin_memory() for r in range(rounds)]
            host_out = [torch.empty(length * 4, dtype=torch.uint8).pin_memory() for _ in range(rounds)]
            src = torch.empty(length * 4, dtype=torch.uint8, device="cuda:0")
            dst = torch.full((length * 4,), 0x5A, dtype=torch.uint8, device="cuda:0")
            for r in range(rounds):
                src.copy_(staged[r], non_blocking=True)
                comm.all_reduce(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                host_out[r].copy_(dst, non_blocking=True)
            stream.synchronize()
            for r in range(rounds):
                outs[r][rank] = host_out[r].numpy().view(np.float32).copy()
        return None

    run_test(nranks, [None] * nranks, [None] * nranks, main)
    for r in range(rounds):
        for rank in range(nranks):
            assert bits_equal(outs[r][rank], wants[r][rank]), f"round {r} rank {rank}"


@pytest.mark.parametrize("nbytes", [13, 4096 + 3, 3 * 1024 * 1024 + 5])
def test_ring_of_sends_back_to_back_on_rank_streams(nbytes):
    """Four ranks, each on a stream of its own, pass blocks round a ring five times without a host synchronisation:
    every round a rank copies fresh bytes into the SAME send buffer on its stream, sends it to the right neighbour
    and receives from the left one inside group_start / group_end, and copies the SAME receive buffer out on its
    stream.  A copy that started before the sender's copy-in had landed, a copy-in that overtook the previous
    round's transfer, or a copy-out that overtook the transfer shows as a wrong round.  Buffers sit at odd byte
    addresses; the lengths run the edge bytes only, the short copy kernel and the group copy kernel."""
    nranks, rounds = 4, 5
    rng = np.random.default_rng(nbytes)
    data = [[rng.integers(0, 256, nbytes, dtype=np.uint8) for _ in range(nranks)] for _ in range(rounds)]
    outs = [[None] * nranks for _ in range(rounds)]

    def main(comm, rank, _inp, stream):
        right, left = (rank + 1) % nranks, (rank - 1) % nranks
        with torch.cuda.stream(stream):
            staged = [torch.from_numpy(data[r][rank].copy()).pin_memory() for r in range(rounds)]
            host_out = [torch.empty(nbytes, dtype=torch.uint8).pin_memory() for _ in range(rounds)]
            src = torch.empty(nbytes + 64, dtype=torch.uint8, device="cuda:0")[1 + rank:1 + rank + nbytes]
            dst = torch.full((nbytes + 64,), 0x5A, dtype=torch.uint8, device="cuda:0")[7 - rank:7 - rank + nbytes]
            for r in range(rounds):
                src.copy_(staged[r], non_blocking=True)
                comm.group_start()
                comm.send(src, nbytes, mr.DType.UINT8, right, stream)
                comm.recv(dst, nbytes, mr.DType.UINT8, left, stream)
                comm.group_end()
                host_out[r].copy_(dst, non_blocking=True)
            stream.synchronize()
            for r in range(rounds):
                outs[r][rank] = host_out[r].numpy().copy()
        return None

    for own_streams in (True, False):
        run_test(nranks, [None] * nranks, [None] * nranks, main, own_streams=own_streams)
        for r in range(rounds):
            for rank in range(nranks):
                assert bits_equal(outs[r][rank], data[r][(rank - 1) % nranks]), f"round {r} rank {rank}"


@pytest.mark.parametrize("nranks,part", [(8, 3), (5, 1000 + 1), (8, 40 * 256), (3, 700 * 256 + 2)])
def test_back_to_back_rounds_of_every_collective_on_rank_streams(nranks, part):
    """Four rounds of reduce_scatter, all_gather, all_to_all, scatter, gather, broadcast and reduce, one after the
    other on each rank's own stream with no host synchronisation: every round a rank copies fresh data into the SAME
    send buffer on its stream before the first call and copies every result out of the SAME receive buffers on its
    stream after the calls.  The short lengths run single launches of one wavefront per workgroup, which carry the
    stream ordering themselves (copy, segment fold, tree and flat kernels alike); the long ones run between separate
    wait and notify kernels."""
    rounds, root = 4, nranks - 2
    length = part * nranks
    f32, npf = mr.DType.FLOAT32, np.float32
    rng = np.random.default_rng(nranks * 1000003 + part)
    data = [[rand_array(orc.FLOAT32, length, rng, wide=False) for _ in range(nranks)] for _ in range(rounds)]
    names = ("reduce_scatter", "all_gather", "all_to_all", "scatter", "gather", "broadcast", "reduce")
    sizes = {"reduce_scatter": part, "all_gather": length, "all_to_all": length, "scatter": part, "gather": length,
             "broadcast": part, "reduce": part}
    wants = []
    for ins in data:
        heads = [x[:part] for x in ins]
        wants.append({
            "reduce_scatter": orc.ucx_reduce_scatter(ins, orc.FLOAT32, orc.SUM),
            "all_gather": orc.ucx_all_gather(heads, orc.FLOAT32),
            "all_to_all": orc.ucx_all_to_all(ins, orc.FLOAT32),
            "scatter": orc.ucx_scatter(ins, orc.FLOAT32, root),
            "gather": orc.ucx_gather(heads, orc.FLOAT32, root),
            "broadcast": orc.ucx_broadcast(heads, orc.FLOAT32, root),
            "reduce": orc.ucx_reduce(heads, orc.FLOAT32, orc.MAX, root),
        })
    outs = [[None] * nranks for _ in range(rounds)]

    def main(comm, rank, _inp, stream):
        with torch.cuda.stream(stream):
            staged = [torch.from_numpy(data[r][rank].view(np.uint8).copy()).pin_memory() for r in range(rounds)]
            host = [{k: torch.empty(sizes[k] * 4, dtype=torch.uint8).pin_memory() for k in names} for _ in range(rounds)]
            src = torch.empty(length * 4, dtype=torch.uint8, device="cuda:0")
            dev = {k: torch.full((sizes[k] * 4,), 0x5A, dtype=torch.uint8, device="cuda:0") for k in names}
            for r in range(rounds):
                src.copy_(staged[r], non_blocking=True)
                comm.reduce_scatter(src, dev["reduce_scatter"], part, f32, mr.ReduceOp.SUM, stream)
                comm.all_gather(src, dev["all_gather"], part, f32, stream)
                comm.all_to_all(src, dev["all_to_all"], part, f32, stream)
                comm.scatter(src if rank == root else None, dev["scatter"], part, f32, root, stream)
                comm.gather(src, dev["gather"] if rank == root else None, part, f32, root, stream)
                comm.broadcast(src, dev["broadcast"], part, f32, root, stream)
                comm.reduce(src, dev["reduce"] if rank == root else None, part, f32, mr.ReduceOp.MAX, root, stream)
                for k in names:
                    host[r][k].copy_(dev[k], non_blocking=True)
            stream.synchronize()
            for r in range(rounds):
                outs[r][rank] = {k: host[r][k].numpy().view(npf).copy() for k in names}
        return None

    run_test(nranks, [None] * nranks, [None] * nranks, main)
    for r in range(rounds):
        for rank in range(nranks):
            for k in names:
                if k in ("gather", "reduce") and rank != root:
                    continue
                want = wants[r][k][rank]
                assert bits_equal(outs[r][rank][k], want), f"round {r} rank {rank} {k}"


def test_more_distinct_collectives_than_the_plan_cache_holds():
    """A group keeps the plans of its 64 most recently used collectives.  Seventy all_reduces of different lengths,
    gone through twice in the same order (every call of the second pass finds its plan evicted) and then the last
    few once more (found), all give the exact sums."""
    nranks, longest = 4, 70
    rng = np.random.default_rng(70)
    ins = [rng.integers(-2 ** 31, 2 ** 31, longest, dtype=np.int64).astype(np.int32) for _ in range(nranks)]
    total = np.sum(np.stack(ins).astype(np.int64), axis=0).astype(np.int32)  # wraps like the int32 sum
    lengths = list(range(1, longest + 1)) * 2 + list(range(longest - 5, longest + 1))

    def main(comm, rank, inp, stream):
        with torch.cuda.stream(stream):
            src = to_device(inp)
            outs = [empty_device(n * 4) for n in lengths]
            for n, dst in zip(lengths, outs):
                comm.all_reduce(src, dst, n, mr.DType.INT32, mr.ReduceOp.SUM, stream)
            stream.synchronize()
            return np.concatenate([to_host(dst, np.int32) for dst in outs])

    want = np.concatenate([total[:n] for n in lengths])
    run_test(nranks, ins, [want] * nranks, main)


def test_two_groups_at_the_same_time():
    """Two communicator groups of four ranks each, alive and busy at the same time (eight rank threads, eight streams):
    each group keeps its own counters, plans and rendezvous, so their collectives - short ones that carry the stream
    ordering themselves and long ones between wait and notify kernels - do not disturb each other."""
    nranks, rounds = 4, 12
    results = {}

    def group_main(tag, length):
        rng = np.random.default_rng(1000 + tag)
        ins = [rand_array(orc.FLOAT32, length, rng) for _ in range(nranks)]
        want = orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM)

        def main(comm, rank, inp, stream):
            with torch.cuda.stream(stream):
                staged = torch.from_numpy(inp.view(np.uint8).copy()).pin_memory()
                src = torch.empty(length * 4, dtype=torch.uint8, device="cuda:0")
                dst = torch.full((length * 4,), 0x5A, dtype=torch.uint8, device="cuda:0")
                host_out = torch.empty(length * 4, dtype=torch.uint8).pin_memory()
                for _ in range(rounds):
                    src.copy_(staged, non_blocking=True)
                    comm.all_reduce(src, dst, length, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream)
                    host_out.copy_(dst, non_blocking=True)
                stream.synchronize()
                return host_out.numpy().view(np.float32).copy()

        try:
            run_test(nranks, ins, want, main)
            results[tag] = "ok"
        except BaseException as exc:  # noqa: BLE001
            results[tag] = repr(exc)

    threads = [threading.Thread(target=group_main, args=(0, 20000), daemon=True),
               threading.Thread(target=group_main, args=(1, 300000), daemon=True)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(200)
        assert not t.is_alive(), "a group hung"
    assert results == {0: "ok", 1: "ok"}, results
