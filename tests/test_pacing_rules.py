"""When a planned launch spaces its accesses out (the `paced` field of mrv_describe's runs).

Host arithmetic on the buffers' addresses, checked here without a GPU on made-up addresses; that paced and unpaced
launches give the same results is checked on the GPU (test_gpu_parity.py)."""
import pytest

import megray_amd as mr

MIB = 1 << 20
GIB = 1 << 30
BASE = 0x7F0000000000


def placed(count, size, start=BASE, shift=0):
    """Addresses as mrv_rank_buffers_layout gives them: an odd multiple of 128 MiB (+ shift) apart."""
    units = -(-size // (128 * MIB))
    pitch = (units | 1) * 128 * MIB + shift
    return [start + i * pitch for i in range(count)]


def separate(count, size, start=BASE):
    """Addresses as one allocation per buffer gives them: the size plus a 2 MiB page apart."""
    return [start + i * (size + 2 * MIB) for i in range(count)]


def is_paced(coll, send, recv, count, dtype=mr.DType.FLOAT32, **kw):
    runs, _, _ = mr.describe(coll, send, recv, count, dtype, **kw)
    flags = {r["paced"] for r in runs}
    assert len(flags) == 1, "every run of a plan is paced or none is"
    return flags.pop() == 1


@pytest.fixture(autouse=True)
def no_override(monkeypatch):
    monkeypatch.delenv("MEGRAY_VRANK_PACE", raising=False)


def all_reduce_paced(nranks, elems, layout):
    size = 4 * elems
    bufs = layout(2 * nranks, size)
    return is_paced(mr.Collective.ALL_REDUCE, bufs[:nranks], bufs[nranks:], elems)


def test_all_reduce_on_buffers_the_library_did_not_place_paces_from_three_gib():
    assert all_reduce_paced(8, 1 << 28, separate)       # 16 GiB moved
    assert all_reduce_paced(8, 1 << 26, separate)       # 4 GiB
    assert not all_reduce_paced(8, 1 << 25, separate)   # 2 GiB
    assert all_reduce_paced(4, 1 << 27, separate)       # 4 GiB on four ranks
    assert not all_reduce_paced(2, 1 << 20, separate)


def test_all_reduce_on_placed_buffers_never_paces():
    assert not all_reduce_paced(8, 1 << 28, placed)     # the headline: 16 GiB
    assert not all_reduce_paced(8, 1 << 27, placed)
    assert not all_reduce_paced(4, 1 << 29, placed)
    assert not all_reduce_paced(5, 1 << 28, placed)     # the general kernel, every rank an output


def test_the_environment_overrides_the_rule(monkeypatch):
    monkeypatch.setenv("MEGRAY_VRANK_PACE", "never")
    assert not all_reduce_paced(8, 1 << 28, separate)
    monkeypatch.setenv("MEGRAY_VRANK_PACE", "always")
    assert all_reduce_paced(8, 1 << 22, placed)


def all_gather_paced(nranks, block, out_layout):
    ins = placed(nranks, block)
    outs = out_layout(nranks, block * nranks, BASE + (1 << 40))
    return is_paced(mr.Collective.ALL_GATHER, ins, outs, block, mr.DType.UINT8)


def gather_layout(count, size, start):
    return placed(count, size, start, shift=32 * MIB)   # what the all_gather hint of the placement gives written buffers


def test_all_gather_paces_its_stores_by_rank_count_and_bytes_written_wherever_the_outputs_lie():
    for layout in (separate, placed, gather_layout):
        assert all_gather_paced(8, 16 * MIB, layout)            # 1 GiB written
        assert all_gather_paced(8, 6 * MIB, layout)             # 384 MiB
        assert all_gather_paced(6, 11 * MIB, layout)            # 396 MiB
        assert not all_gather_paced(8, 5 * MIB, layout)         # 320 MiB
        assert not all_gather_paced(6, 10 * MIB, layout)        # 360 MiB
        assert all_gather_paced(4, 128 * MIB, layout)           # 2 GiB
        assert not all_gather_paced(5, 64 * MIB, layout)        # 1.6 GiB on fewer than six ranks
        assert not all_gather_paced(3, 512 * MIB, layout)       # fewer than four ranks: never
        for nranks in (12, 16, 32):
            assert all_gather_paced(nranks, 1 * MIB, layout)
    runs, _, _ = mr.describe(mr.Collective.ALL_GATHER, placed(12, 4096), placed(12, 12 * 4096, BASE + (1 << 40)), 4096, mr.DType.UINT8)
    assert all(r["waves"] == 1 and r["paced"] == 0 for r in runs)   # short blocks: one wavefront per tile, nothing to pace


def broadcast_paced(nranks, block):
    outs = placed(nranks, block, BASE + (1 << 40))
    return is_paced(mr.Collective.BROADCAST, [BASE] + [0] * (nranks - 1), outs, block, mr.DType.UINT8, root=0, nranks=nranks)


def test_broadcast_paces_its_stores_by_rank_count_and_block_size():
    assert broadcast_paced(9, 16 * MIB) and broadcast_paced(16, 64 * MIB) and not broadcast_paced(16, 8 * MIB)
    assert broadcast_paced(8, 256 * MIB) and broadcast_paced(5, 256 * MIB) and not broadcast_paced(8, 128 * MIB)
    assert broadcast_paced(4, 512 * MIB) and not broadcast_paced(4, 256 * MIB)
    assert not broadcast_paced(3, 1024 * MIB) and not broadcast_paced(2, 1024 * MIB)


def test_a_fold_into_one_output_off_the_tile_grid_paces_from_a_gib_wherever_the_buffers_lie():
    """reduce_scatter of a rank count that leaves the blocks off the 1 KiB grid runs the general group kernel."""
    for layout in (placed, separate):
        for nranks, recv_elems, want in ((5, (128 * MIB // 4) // 5, True), (7, (128 * MIB // 4) // 7, True),
                                         (12, (256 * MIB // 4) // 12, True), (5, (32 * MIB // 4) // 5, False)):
            size = 4 * recv_elems * nranks
            bufs = layout(2 * nranks, size)
            assert is_paced(mr.Collective.REDUCE_SCATTER, bufs[:nranks], bufs[nranks:], recv_elems) == want, (nranks, recv_elems)
    # eight ranks, blocks on the grid: the flat kernel, which paces all_reduce shapes only
    bufs = placed(16, 512 * MIB)
    assert not is_paced(mr.Collective.REDUCE_SCATTER, bufs[:8], bufs[8:], (512 * MIB // 4) // 8)


def test_the_other_pack_collectives_never_pace():
    n, block = 16, 16 * MIB
    ins, outs = placed(n, n * block), placed(n, n * block, BASE + (1 << 40))
    assert not is_paced(mr.Collective.ALL_TO_ALL, ins, outs, block, mr.DType.UINT8)
    assert not is_paced(mr.Collective.SCATTER, [ins[0]] + [0] * (n - 1), outs, block, mr.DType.UINT8, root=0, nranks=n)
    assert not is_paced(mr.Collective.GATHER, ins, [outs[0]] + [0] * (n - 1), block, mr.DType.UINT8, root=0, nranks=n)


def keeps(coll, send, recv, count, dtype=mr.DType.FLOAT32, **kw):
    runs, _, written = mr.describe(coll, send, recv, count, dtype, **kw)
    flags = {r["keep"] for r in runs}
    assert len(flags) == 1, "one store policy per plan"
    return flags.pop() == 1, written


def test_results_of_128_mib_and_less_stay_in_the_last_level_cache(monkeypatch):
    """The stores of a collective that writes up to 128 MiB in all leave their data in the cache; longer ones stream."""
    monkeypatch.delenv("MEGRAY_VRANK_KEEP", raising=False)
    for elems, want in ((1 << 10, True), (1 << 22, True), ((1 << 22) + 256, False), (1 << 28, False)):   # 8 x 16 MiB is the border
        bufs = placed(16, 4 * elems)
        got, written = keeps(mr.Collective.ALL_REDUCE, bufs[:8], bufs[8:], elems)
        assert got == want and written == 8 * 4 * elems
    # every launch of a multi-launch plan follows the plan's total
    bufs = placed(16, 1 << 26)
    for sched in (mr.Schedule.TWO_PHASE, mr.Schedule.RING):
        assert keeps(mr.Collective.ALL_REDUCE, bufs[:8], bufs[8:], 1 << 20, schedule=sched)[0]
        assert not keeps(mr.Collective.ALL_REDUCE, bufs[:8], bufs[8:], 1 << 24, schedule=sched)[0]
    # a reduce_scatter writes one block per rank, an all_gather N blocks per rank
    assert keeps(mr.Collective.REDUCE_SCATTER, bufs[:8], bufs[8:], 1 << 21)[0]          # 8 x 8 MiB written of 8 x 64 MiB read
    ins, outs = placed(8, 16 * MIB), placed(8, 128 * MIB, BASE + (1 << 40))
    assert keeps(mr.Collective.ALL_GATHER, ins, outs, 2 * MIB, mr.DType.UINT8)[0]        # 128 MiB written
    assert not keeps(mr.Collective.ALL_GATHER, ins, outs, 2 * MIB + 16, mr.DType.UINT8)[0]
    assert keeps(mr.Collective.BROADCAST, [BASE] + [0] * 7, outs, 16 * MIB, mr.DType.UINT8, root=0, nranks=8)[0]
    assert not keeps(mr.Collective.BROADCAST, [BASE] + [0] * 7, outs, 17 * MIB, mr.DType.UINT8, root=0, nranks=8)[0]
    assert keeps(mr.Collective.REDUCE, bufs[:5], [0, 0, bufs[8], 0, 0], 1 << 24, root=2, nranks=5)[0]   # the tree kernel: 64 MiB
    monkeypatch.setenv("MEGRAY_VRANK_KEEP", "never")
    assert not keeps(mr.Collective.ALL_REDUCE, bufs[:8], bufs[8:], 1 << 10)[0]
    monkeypatch.setenv("MEGRAY_VRANK_KEEP", "always")
    assert keeps(mr.Collective.ALL_REDUCE, bufs[:8], bufs[8:], 1 << 24)[0]
