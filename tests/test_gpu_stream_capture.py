"""The flat entry points inside a caller's stream capture.

Every collective of the flat C ABI is a handful of kernel launches on the stream it is given: no
allocation, no memset, no event, no host synchronisation.  A caller may therefore record them into a
HIP graph of its own by stream capture (mrv_plan_create builds graphs of its own; this is the other
way round).  The captured graph is replayed several times, on fresh inputs and with the program's own
eager work and host synchronisations between the replays, and every replay is compared with the oracle.
"""
import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import bits_equal, empty_device, first_mismatch, rand_array, to_device, to_host  # noqa: E402


def assert_same(got, want, what):
    if not bits_equal(got, want):
        raise AssertionError(f"{what}: first mismatch (index, got, want, count) = {first_mismatch(got, want)}")


def refill(dev, arr):
    dev.copy_(torch.from_numpy(np.ascontiguousarray(arr).view(np.uint8).reshape(-1).copy()))


# lengths: one that runs the short kernels (one wavefront per tile), one that runs the group kernels, and one whose
# chunks lie on cache-line boundaries, so that the one-output folds run at the reduced occupancy (LDS reserved at launch)
@pytest.mark.parametrize("length", [8 * 1000 + 8, 8 * 3000 * 256 + 8 * 5, 8 * 3000 * 256 + 8 * 32])
def test_captured_collectives_replay_on_fresh_data(length):
    rng = np.random.default_rng(length)
    nranks = 8
    part = length // nranks
    f32, u8 = mr.DType.FLOAT32, mr.DType.UINT8
    d_in = [to_device(rand_array(orc.FLOAT32, length, rng)) for _ in range(nranks)]
    d_fused = [empty_device(length * 4) for _ in range(nranks)]
    d_two = [empty_device(length * 4) for _ in range(nranks)]
    d_ring = [empty_device(length * 4) for _ in range(nranks)]
    d_part = [empty_device(part * 4) for _ in range(nranks)]
    d_gath = [empty_device(length * 4) for _ in range(nranks)]
    d_swap = [empty_device(length * 4) for _ in range(nranks)]
    d_root = empty_device(length * 4)

    def enqueue(st):
        mr.all_reduce(d_in, d_fused, length, f32, mr.ReduceOp.SUM, stream=st)
        mr.all_reduce(d_in, d_two, length, f32, mr.ReduceOp.SUM, schedule=mr.Schedule.TWO_PHASE, stream=st)
        mr.all_reduce(d_in, d_ring, length, f32, mr.ReduceOp.SUM, schedule=mr.Schedule.RING, stream=st)
        mr.reduce_scatter(d_in, d_part, part, f32, mr.ReduceOp.SUM, stream=st)
        # reads what the reduce_scatter before it on the same stream wrote
        mr.all_gather(d_part, d_gath, part, f32, stream=st)
        mr.all_to_all(d_in, d_swap, part * 4, u8, stream=st)
        mr.reduce_to_root(d_in, d_root, length, f32, mr.ReduceOp.MAX, 3, stream=st)

    side = torch.cuda.Stream()
    enqueue(side)  # once eagerly: the runtime loads a kernel's code at its first launch, which a capture may refuse
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        enqueue(torch.cuda.current_stream())

    for replay in range(3):
        ins = [rand_array(orc.FLOAT32, length, rng) for _ in range(nranks)]
        for d, x in zip(d_in, ins):
            refill(d, x)
        for o in d_fused + d_two + d_ring + d_part + d_gath + d_swap + [d_root]:
            o.fill_(replay + 1)  # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        what = f"length={length} replay={replay}"
        want = orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM)
        scattered = orc.ucx_reduce_scatter(ins, orc.FLOAT32, orc.SUM)
        gathered = orc.ucx_all_gather(scattered, orc.FLOAT32)
        swapped = orc.ucx_all_to_all([x.view(np.uint8) for x in ins], orc.UINT8)
        for r in range(nranks):
            assert_same(to_host(d_fused[r], np.float32), want[r], f"{what} fused all_reduce, rank {r}")
            assert_same(to_host(d_two[r], np.float32), want[r], f"{what} two-phase all_reduce, rank {r}")
            assert_same(to_host(d_ring[r], np.float32), want[r], f"{what} ring all_reduce, rank {r}")
            assert_same(to_host(d_part[r], np.float32), scattered[r], f"{what} reduce_scatter, rank {r}")
            assert_same(to_host(d_gath[r], np.float32), gathered[r], f"{what} all_gather, rank {r}")
            assert_same(to_host(d_swap[r], np.uint8), swapped[r], f"{what} all_to_all, rank {r}")
        assert_same(to_host(d_root, np.float32), np.stack(ins).max(axis=0), f"{what} reduce MAX to rank 3")
