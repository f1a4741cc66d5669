"""The bootstrap service (create_server / Client), CPU only.  Scenarios follow the reference's
test/test_server_client.cpp:20-216: connect, barrier under skewed arrival, broadcast, allgather and
a mixed request sequence, N ranks as N threads over TCP on localhost."""
import threading
import time

import pytest

import megray_amd as mr


def run_ranks(nranks, fn):
    errors = []

    def wrap(rank):
        try:
            fn(rank)
        except BaseException as exc:  # noqa: BLE001
            errors.append((rank, exc))

    threads = [threading.Thread(target=wrap, args=(r,)) for r in range(nranks)]
    for t in threads:
        t.start()
    for t in threads:
        t.join(60)
        assert not t.is_alive(), "a rank hung"
    assert not errors, errors


def test_get_free_port():
    assert mr.get_free_port() > 0  # test/test_server_client.cpp:28-31


def test_connect():
    nranks, port = 3, mr.get_free_port()
    mr.create_server(nranks, port)

    def rank_main(rank):
        client = mr.Client(nranks, rank)
        client.connect("localhost", port)  # the reference's tests say "localhost" too
        client.close()

    run_ranks(nranks, rank_main)


def test_barrier_holds_back_early_ranks():
    # test/test_server_client.cpp:55-92: rank i sleeps i*100 ms before the barrier; nobody passes early
    nranks, port = 3, mr.get_free_port()
    mr.create_server(nranks, port)
    counter = {"n": 0}
    lock = threading.Lock()

    def rank_main(rank):
        client = mr.Client(nranks, rank)
        client.connect("127.0.0.1", port)
        time.sleep(0.1 * rank)
        with lock:
            counter["n"] += 1
        client.barrier()
        assert counter["n"] == nranks
        client.barrier()
        client.close()

    run_ranks(nranks, rank_main)


@pytest.mark.parametrize("root", [0, 1, 2])
def test_broadcast(root):
    nranks, port = 3, mr.get_free_port()
    mr.create_server(nranks, port)
    payload = bytes(range(256)) * 17

    def rank_main(rank):
        client = mr.Client(nranks, rank)
        client.connect("127.0.0.1", port)
        got = client.broadcast(payload if rank == root else bytes(len(payload)), root, rank == root)
        assert got == payload
        client.close()

    run_ranks(nranks, rank_main)


def test_allgather_and_sequence():
    nranks, port = 4, mr.get_free_port()
    mr.create_server(nranks, port)

    def rank_main(rank):
        client = mr.Client(nranks, rank)
        client.connect("127.0.0.1", port)
        for round_ in range(5):  # barrier / broadcast / allgather interleaved
            got = client.allgather(bytes([rank, round_]) * 100)
            assert got == b"".join(bytes([r, round_]) * 100 for r in range(nranks))
            client.barrier()
            msg = bytes([round_]) * 33
            assert client.broadcast(msg, round_ % nranks, rank == round_ % nranks) == msg
        client.close()

    run_ranks(nranks, rank_main)


def test_invalid_usage():
    # src/core/client.cpp:31-34,69-72: MEGRAY_INVALID_USAGE
    client = mr.Client(1, 0)
    with pytest.raises(mr.MegRayError) as err:
        client.barrier()
    assert err.value.status == mr.Status.INVALID_USAGE
    port = mr.get_free_port()
    mr.create_server(1, port)
    client.connect("127.0.0.1", port)
    with pytest.raises(mr.MegRayError) as err:
        client.connect("127.0.0.1", port)
    assert err.value.status == mr.Status.INVALID_USAGE
    client.barrier()
    client.close()


def test_unknown_backend_throws():
    # src/megray.cpp:56-57
    for backend in (mr.Backend.NCCL, mr.Backend.UCX, mr.Backend.RCCL, mr.Backend.SHM, 5, 99):
        with pytest.raises(mr.MegRayError, match="unknown backend"):
            mr.Communicator(2, 0, backend)


def test_group_rendezvous_without_gpu():
    """init() through the bootstrap server forms one group per server; no device call is made."""
    nranks, port = 3, mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r) for r in range(nranks)]

    def rank_main(rank):
        comms[rank].init("localhost", port)

    run_ranks(nranks, rank_main)
    for c in comms:
        c.close()
    with pytest.raises(mr.MegRayError):
        mr.Communicator(33, 0)  # more ranks than the backend takes


def test_a_rank_that_rejects_its_arguments_releases_the_others_without_gpu():
    """A rank whose own arguments fail validation throws on its own thread, as in the reference
    (src/ucx/kernel.cu:95-96), and tells the group: the other ranks' calls come back with
    MEGRAY_INVALID_USAGE and the reason instead of waiting for it.  No device call is made on this path (the
    rank that arrives last and finds everyone else there enqueues nothing on its stream before it looks at
    the group), so the rendezvous logic runs without a GPU."""
    nranks, port = 2, mr.get_free_port()
    mr.create_server(nranks, port)
    comms = [mr.get_communicator(nranks, r) for r in range(nranks)]
    run_ranks(nranks, lambda rank: comms[rank].init("localhost", port))
    fake = 0x10000000  # never dereferenced: nothing is launched
    with pytest.raises(mr.MegRayError, match="unknown dtype"):
        comms[0].all_reduce(fake, fake, 16, mr.DType.CHAR, mr.ReduceOp.SUM)
    # a second rejected call on the same rank does not wait for the first one's collective to end
    with pytest.raises(mr.MegRayError, match="unknown reduce op"):
        comms[0].all_reduce(fake, fake, 16, mr.DType.FLOAT32, 9)
    with pytest.raises(mr.MegRayError) as info:
        comms[1].all_reduce(fake + 4096, fake + 4096, 16, mr.DType.FLOAT32, mr.ReduceOp.SUM)
    assert info.value.status == mr.Status.INVALID_USAGE
    assert "rank 0 left the collective" in info.value.message and "unknown dtype" in info.value.message
    for c in comms:
        c.close()
