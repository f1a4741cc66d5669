"""Placement of the ranks' buffers in one allocation (mrv_rank_buffers_layout / _alloc / _free).

The layout is host arithmetic and is checked here without a GPU; the allocation and a collective over placed
buffers run on the GPU against the oracle's literal ring replay."""
import ctypes

import numpy as np
import pytest

import megray_amd as mr
from megray_amd import _lib

MIB = 1 << 20
UNIT = 128 * MIB


def test_large_buffers_lie_an_odd_multiple_of_128_mib_apart():
    for size in (8 * MIB, 16 * MIB, 100 * MIB, 128 * MIB, 128 * MIB + 1, 256 * MIB, 1 << 30, (1 << 30) + 5, 3 << 30):
        offsets, total = mr.rank_buffers_layout([size] * 16)
        pitch = offsets[1] - offsets[0]
        assert pitch >= size and pitch % UNIT == 0 and (pitch // UNIT) % 2 == 1, (size, pitch)
        assert pitch - size < 2 * UNIT  # never more than two units of slack
        assert offsets == [i * pitch for i in range(16)]
        # the sixteen starts differ in the address bits from 128 MiB up to 4 GiB
        assert len({(o // UNIT) % 32 for o in offsets}) == 16
        assert offsets[-1] + size <= total < offsets[-1] + size + 4096


def test_buffers_an_all_gather_writes_lie_32_mib_off_the_128_mib_grid():
    """all_gather stores every rank's block into every rank's buffer: the written buffers go a multiple of
    128 MiB plus 32 MiB apart (what eight write streams against one read stream are served best at), the buffers
    that are read keep the odd multiple of 128 MiB; every other collective is laid out as without the hint."""
    shift = 32 * MIB
    for coll in (mr.Collective.ALL_GATHER,):
        for small, large in ((16 * MIB, 128 * MIB), (64 * MIB, 512 * MIB), (9 * MIB, 72 * MIB + 4096)):
            sizes, written = [small] * 8 + [large] * 8, [0] * 8 + [1] * 8
            offsets, total = mr.rank_buffers_layout(sizes, coll, written)
            read_pitch, write_pitch = offsets[1] - offsets[0], offsets[9] - offsets[8]
            assert read_pitch % UNIT == 0 and (read_pitch // UNIT) % 2 == 1
            assert write_pitch % UNIT == shift and large <= write_pitch - shift < large + UNIT, (large, write_pitch)
            assert offsets[8:] == [offsets[8] + i * write_pitch for i in range(8)]
            spans = sorted(zip(offsets, sizes))
            assert all(a + n <= b for (a, n), (b, _) in zip(spans, spans[1:])) and spans[-1][0] + spans[-1][1] <= total
        # small written buffers live in the caches and stay close together
        assert mr.rank_buffers_layout([4096] * 4, coll, [1] * 4) == mr.rank_buffers_layout([4096] * 4)
    sizes = [1 << 27] * 16
    for coll in (mr.Collective.ALL_REDUCE, mr.Collective.REDUCE_SCATTER, mr.Collective.ALL_TO_ALL, mr.Collective.SCATTER,
                 mr.Collective.GATHER, mr.Collective.BROADCAST, mr.Collective.REDUCE, mr.Collective.REDUCE2):
        assert mr.rank_buffers_layout(sizes, coll, [0] * 8 + [1] * 8) == mr.rank_buffers_layout(sizes)
    assert mr.rank_buffers_layout(sizes, mr.Collective.ALL_GATHER, None) == mr.rank_buffers_layout(sizes)  # nothing marked
    with pytest.raises(mr.MegRayError, match="unknown collective"):
        mr.rank_buffers_layout(sizes, 99, [0] * 16)
    with pytest.raises(mr.MegRayError, match="written flags"):
        mr.rank_buffers_layout(sizes, mr.Collective.ALL_GATHER, [1] * 3)


def test_small_buffers_stay_close_together():
    offsets, total = mr.rank_buffers_layout([4096] * 16)
    assert offsets == [i * 4096 for i in range(16)] and total == 16 * 4096
    offsets, total = mr.rank_buffers_layout([100, 5000, 0, 3 * MIB, 3 * MIB + 1])
    assert offsets == [0, 4096, 3 * 4096, 2 * MIB, 6 * MIB]
    assert total == 6 * MIB + 3 * MIB + 4096


def test_mixed_sizes_do_not_overlap_and_keep_their_alignment():
    sizes = [1 << 27] * 8 + [1 << 24] * 8 + [12345, 7 * MIB]
    offsets, total = mr.rank_buffers_layout(sizes)
    spans = sorted(zip(offsets, sizes))
    for (a, n), (b, _) in zip(spans, spans[1:]):
        assert a + n <= b
    assert spans[-1][0] + spans[-1][1] <= total
    for off, size in zip(offsets, sizes):
        assert off % (2 * MIB if size >= 2 * MIB else 4096) == 0


def test_layout_argument_errors():
    assert mr.rank_buffers_layout([]) == ([], 0)
    with pytest.raises(mr.MegRayError, match="address space"):
        mr.rank_buffers_layout([2 ** 63] * 3)
    L = _lib.load()
    total = ctypes.c_size_t(0)
    assert L.mrv_rank_buffers_layout(-1, None, None, ctypes.byref(total)) == int(mr.Status.INVALID_ARGUMENT)
    assert b"negative" in L.mrv_last_error()
    assert L.mrv_rank_buffers_layout(2, None, None, ctypes.byref(total)) == int(mr.Status.INVALID_ARGUMENT)
    assert L.mrv_rank_buffers_layout(0, None, None, None) == int(mr.Status.INVALID_ARGUMENT)
    base = ctypes.c_void_p()
    assert L.mrv_rank_buffers_alloc(0, None, None, ctypes.byref(base)) == int(mr.Status.INVALID_ARGUMENT)
    assert L.mrv_rank_buffers_free(None) == 0


@pytest.mark.gpu
def test_all_reduce_on_placed_buffers_equals_the_ring_replay():
    import torch

    import oracle as orc
    from megray_amd import synth

    nranks, n = 4, (9 * MIB) // 4 + 3  # above the 8 MiB threshold: the buffers are spread
    with mr.RankBuffers([n * 4] * (2 * nranks)) as bufs:
        assert all(b - a == UNIT for a, b in zip(bufs.ptrs, bufs.ptrs[1:]))
        ins, outs = bufs.ptrs[:nranks], bufs.ptrs[nranks:]
        host = [synth.fill_np(np.float32, n, r) for r in range(nranks)]
        staged = [torch.from_numpy(h).cuda() for h in host]
        got = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(nranks)]
        st = torch.cuda.current_stream()
        raw = ctypes.CDLL("libamdhip64.so")
        raw.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
        for r in range(nranks):
            assert raw.hipMemcpy(ins[r], staged[r].data_ptr(), n * 4, 3) == 0  # device to device
        mr.all_reduce(ins, outs, n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream=st)
        torch.cuda.synchronize()
        for r in range(nranks):
            assert raw.hipMemcpy(got[r].data_ptr(), outs[r], n * 4, 3) == 0
        torch.cuda.synchronize()
    want = orc.ucx_all_reduce(host, orc.FLOAT32, orc.SUM)
    for r in range(nranks):
        assert np.array_equal(got[r].cpu().numpy().view(np.uint32), want[r].view(np.uint32))


@pytest.mark.gpu
def test_place_tensors_views_are_placed_and_usable():
    import torch

    n = 1 << 22  # 16 MiB of fp32: spread
    ts = mr.place_tensors(torch, [(n, torch.float32)] * 4 + [(100, torch.int8)])
    ptrs = [t.data_ptr() for t in ts]
    assert all(b - a == UNIT for a, b in zip(ptrs[:4], ptrs[1:4]))
    assert ptrs[0] % (2 * MIB) == 0 and ts[4].numel() == 100 and ts[4].dtype == torch.int8
    for i, t in enumerate(ts[:2]):
        t.fill_(float(i + 1))
    mr.all_reduce(ts[:2], ts[2:4], n, mr.DType.FLOAT32, mr.ReduceOp.SUM, stream=torch.cuda.current_stream())
    torch.cuda.synchronize()
    assert torch.all(ts[2] == 3.0) and torch.all(ts[3] == 3.0)
