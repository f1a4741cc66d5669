"""GPU parity: the HIP path, called through the C ABI, against the CPU oracle on the same seeded
inputs.  Bar: bit-exact for every dtype, including fp32/fp64 SUM under the reference's rank order
and FLOAT16 (fp32 accumulation, one rounding; the stated tolerance is 1 ulp, the check is exact).
"""
import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import (bits_equal, empty_device, first_mismatch, rand_array, to_device,  # noqa: E402
                      to_host)

REDUCE_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.UINT64, orc.FLOAT16,
                orc.FLOAT32, orc.FLOAT64]
OPS = [orc.SUM, orc.MAX, orc.MIN]
# the types cpu_reduce() has a loop for (src/shm/utils.cpp:39-69); the shm replays throw for the others
SHM_REDUCE_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.FLOAT32]
ORDERS = [orc.ORDER_UCX, orc.ORDER_SHM, orc.ORDER_RANK0]


def assert_same(got, want, what):
    if not bits_equal(got, want):
        raise AssertionError(f"{what}: first mismatch (index, got, want, count) = {first_mismatch(got, want)}")


def run_all_reduce(ins, dtype, op, order, sched, offsets=None, inplace=False):
    n = len(ins)
    size = orc.dtype_size(dtype)
    offsets = offsets or [0] * n
    d_in = [to_device(x, offsets[r]) for r, x in enumerate(ins)]
    d_out = d_in if inplace else [empty_device(ins[0].size * size, offsets[r]) for r in range(n)]
    mr.all_reduce(d_in, d_out, ins[0].size, dtype, op, order, sched)
    torch.cuda.synchronize()
    return [to_host(o, ins[0].dtype) for o in d_out]


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
@pytest.mark.parametrize("nranks", [1, 2, 3, 4, 5, 8, 16])
def test_all_reduce_fused_all_orders(dtype, nranks):
    rng = np.random.default_rng(1000 * dtype + nranks)
    for length in (0, 1, nranks + 1, 1027, 8 * 4096 + 3, 70001):
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        for op in OPS:
            for order in ORDERS:
                want = orc.fold_all_reduce(ins, dtype, op, order)
                got = run_all_reduce(ins, dtype, op, order, mr.Schedule.FUSED)
                for r in range(nranks):
                    assert_same(got[r], want[r], f"all_reduce dtype={dtype} N={nranks} len={length} op={op} "
                                                 f"order={order} rank={r}")


@pytest.mark.parametrize("nranks", [17, 24, 32])
def test_more_than_sixteen_ranks(nranks):
    """The reference's get_communicator takes any rank count (include/megray.h:33-34); this backend takes up to 32
    virtual ranks.  Every collective at 17, 24 and 32 ranks against the oracle's literal replays: the folds in all three
    orders (more chunks than one launch descriptor holds segments for: several launches), reduce towards a root in the
    tree order, and the block copies; short and long (group form) lengths."""
    rng = np.random.default_rng(3200 + nranks)
    for dtype, length in ((orc.FLOAT32, 5 * nranks + 3), (orc.INT8, 40001), (orc.FLOAT32, 300 * 1024 + 7), (orc.FLOAT16, 2 * 1024 * 1024 + 11)):
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MAX, orc.ORDER_SHM), (orc.MIN, orc.ORDER_RANK0)):
            want = orc.fold_all_reduce(ins, dtype, op, order)
            got = run_all_reduce(ins, dtype, op, order, mr.Schedule.FUSED)
            for r in range(nranks):
                assert_same(got[r], want[r], f"all_reduce N={nranks} dtype={dtype} len={length} op={op} order={order} rank={r}")
        if dtype != orc.FLOAT16:
            root = nranks - 2
            out = empty_device(length * orc.dtype_size(dtype))
            mr.reduce_to_root([to_device(x) for x in ins], out, length, dtype, orc.SUM, root)
            torch.cuda.synchronize()
            assert_same(to_host(out, ins[0].dtype), orc.ucx_reduce(ins, dtype, orc.SUM, root)[root], f"reduce N={nranks} dtype={dtype}")
    recvlen = 1000 + nranks
    ins = [rand_array(orc.FLOAT32, recvlen * nranks, rng) for _ in range(nranks)]
    d_out = [empty_device(recvlen * 4) for _ in range(nranks)]
    mr.reduce_scatter([to_device(x) for x in ins], d_out, recvlen, orc.FLOAT32, orc.SUM)
    torch.cuda.synchronize()
    want = orc.ucx_reduce_scatter(ins, orc.FLOAT32, orc.SUM)
    for r in range(nranks):
        assert_same(to_host(d_out[r], np.float32), want[r], f"reduce_scatter N={nranks} rank={r}")
    for length in (77, 140 * 1024 + 5):
        check_pack_collectives(orc.UINT8, nranks, length, 0, rng)


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_all_reduce_group_form(dtype):
    """Long launches take the group form of the flat kernel (four wavefronts per workgroup, four tiles 32 tiles
    apart; the fewer the ranks, the later: from 15360 / 10752 / 6400 / 2560 tiles per buffer for 2 / 3 / 4 / 8 ranks):
    ragged lengths, so that chunk borders fall inside tiles and the last group of tiles is incomplete; out of place
    and in place."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(77 + dtype)
    for nranks, tiles in ((2, 15400), (3, 10800), (4, 6401), (8, 5051)):
        length = (tiles * 1024 + 1024 - 16 * (nranks - 1)) // size - 3
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        d_in = [to_device(x) for x in ins]
        runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, d_in, [empty_device(length * size) for _ in range(nranks)],
                                 length, dtype)
        assert runs and all(r["waves"] == 4 for r in runs), "the group form is not what runs here"
        for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MAX, orc.ORDER_SHM), (orc.MIN, orc.ORDER_RANK0),
                          (orc.SUM, orc.ORDER_SHM)):
            want = orc.fold_all_reduce(ins, dtype, op, order)
            for inplace in (False, True):
                got = run_all_reduce(ins, dtype, op, order, mr.Schedule.FUSED, inplace=inplace)
                for r in range(nranks):
                    assert_same(got[r], want[r], f"group form dtype={dtype} N={nranks} len={length} op={op} "
                                                 f"order={order} inplace={inplace} rank={r}")


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_all_reduce_group_form_with_paced_accesses(dtype, monkeypatch):
    """Long group launches keep two loads and two stores per wavefront in flight instead of all of them (the planner
    switches it on from a few GiB; MEGRAY_VRANK_PACE=always forces it here at sizes the oracle handles): same results,
    bit for bit, ragged lengths, every order, out of place and in place."""
    monkeypatch.setenv("MEGRAY_VRANK_PACE", "always")
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(1077 + dtype)
    for nranks, tiles in ((3, 10800), (4, 6401), (8, 5051)):
        length = (tiles * 1024 + 1024 - 16 * (nranks - 1)) // size - 3
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MAX, orc.ORDER_SHM), (orc.MIN, orc.ORDER_RANK0)):
            want = orc.fold_all_reduce(ins, dtype, op, order)
            for inplace in (False, True):
                got = run_all_reduce(ins, dtype, op, order, mr.Schedule.FUSED, inplace=inplace)
                for r in range(nranks):
                    assert_same(got[r], want[r], f"paced group form dtype={dtype} N={nranks} len={length} op={op} "
                                                 f"order={order} inplace={inplace} rank={r}")
    # the general group kernel paces the same way: five ranks (inputs staged four at a time), and three ranks whose
    # buffers share an offset from a 16-byte boundary
    for nranks, offset in ((5, 0), (3, max(size, 4))):
        length = 4300 * 1024 // size + 7
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        want = orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX)
        got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, mr.Schedule.FUSED, offsets=[offset] * nranks)
        for r in range(nranks):
            assert_same(got[r], want[r], f"paced segment group form dtype={dtype} N={nranks} offset={offset} rank={r}")
    monkeypatch.setenv("MEGRAY_VRANK_PACE", "never")
    nranks, length = 8, 5051 * 1024 // size + 5
    ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
    got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, mr.Schedule.FUSED)
    want = orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX)
    for r in range(nranks):
        assert_same(got[r], want[r], f"unpaced group form dtype={dtype} rank={r}")


@pytest.mark.parametrize("keep", ["never", "always"])
def test_either_store_policy_gives_the_same_results(keep, monkeypatch):
    """A collective that writes 128 MiB or less leaves its results in the last-level cache, longer ones stream past it:
    two store instructions, chosen per launch.  Every test at a size the oracle handles runs the first; here
    MEGRAY_VRANK_KEEP forces the streaming stores (and, for completeness, the keeping ones) through every kernel form:
    flat (one wavefront per tile, and the group form), general (one wavefront, group form), tree, pack (both forms)."""
    monkeypatch.setenv("MEGRAY_VRANK_KEEP", keep)
    rng = np.random.default_rng(4100)
    for dtype in (orc.FLOAT32, orc.UINT8, orc.FLOAT16):
        size = orc.dtype_size(dtype)
        for nranks, length, offsets in ((8, 40000 // size, None), (8, 5051 * 1024 // size + 5, None), (5, 9000 // size + 3, None),
                                        (5, 4300 * 1024 // size + 7, None), (3, 4300 * 1024 // size + 7, [max(size, 4)] * 3)):
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            want = orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX)
            got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, mr.Schedule.FUSED, offsets=offsets)
            for r in range(nranks):
                assert_same(got[r], want[r], f"keep={keep} all_reduce dtype={dtype} N={nranks} len={length} rank={r}")
        for length in (3000 // size, 4300 * 1024 // size + 7) if dtype != orc.FLOAT16 else ():   # the binomial tree towards a root
            nranks, root = 5, 3
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            want = orc.ucx_reduce(ins, dtype, orc.MAX, root)[root]
            d_in = [to_device(x) for x in ins]
            d_out = empty_device(length * size)
            mr.reduce_to_root(d_in, d_out, length, dtype, orc.MAX, root)
            torch.cuda.synchronize()
            assert_same(to_host(d_out, ins[0].dtype), want, f"keep={keep} tree reduce dtype={dtype} len={length}")
    for length in (1000, 1030 * 1024 + 48):
        check_pack_collectives(orc.UINT8, 8, length, 0, rng)


@pytest.mark.parametrize("dtype", [orc.INT8, orc.FLOAT16, orc.FLOAT32, orc.INT64])
def test_general_folds_of_a_few_mib_keep_one_wavefront_per_group_of_vectors(dtype):
    """Folds through the general kernel whose buffers are vectors throughout keep one wavefront per group of 64
    vectors up to 8 MiB per buffer (3 MiB for twelve and more ranks with several destinations; one-byte elements: 2 MiB, and 1 MiB from twelve ranks on): rank counts without a
    flat kernel, and eight ranks at a common offset from a 16-byte boundary."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(377 + dtype)
    for nranks, offset, kib in ((5, 0, 7900), (7, 0, 1500), (8, max(size, 4), 4100)):
        kib = min(kib, 1900) if size == 1 else kib
        length = kib * 1024 // size + 5
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        d_in = [to_device(x, offset) for x in ins]
        d_out = [empty_device(length * size, offset) for _ in range(nranks)]
        runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, d_in, d_out, length, dtype)
        assert runs and all(r["waves"] == 1 for r in runs), "not the form this test is about"
        for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MIN, orc.ORDER_SHM)):
            want = orc.fold_all_reduce(ins, dtype, op, order)
            got = run_all_reduce(ins, dtype, op, order, mr.Schedule.FUSED, offsets=[offset] * nranks)
            for r in range(nranks):
                assert_same(got[r], want[r], f"all_reduce dtype={dtype} N={nranks} offset={offset} op={op} rank={r}")
    for nranks, kib in ((6, 1900 if size == 1 else 7900), (12, 900 if size == 1 else 3000)):
        recvlen = kib * 1024 // size // nranks // 16 * 16 + 16
        ins = [rand_array(dtype, recvlen * nranks, rng) for _ in range(nranks)]
        d_in = [to_device(x) for x in ins]
        parts = [empty_device(recvlen * size) for _ in range(nranks)]
        runs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, d_in, parts, recvlen, dtype)
        assert runs and all(r["waves"] == 1 for r in runs), "not the form this test is about"
        want = orc.fold_reduce_scatter(ins, dtype, orc.SUM, orc.ORDER_UCX)
        mr.reduce_scatter(d_in, parts, recvlen, dtype, orc.SUM, orc.ORDER_UCX)
        torch.cuda.synchronize()
        for r in range(nranks):
            assert_same(to_host(parts[r], ins[0].dtype), want[r], f"reduce_scatter dtype={dtype} N={nranks} rank={r}")


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_segment_group_form(dtype):
    """The general fold kernel with long vector bodies (beyond 8 MiB per buffer; 512 groups of 64 vectors and more
    for copies and for buffers with element tiles) runs in its group form: rank counts without a flat kernel (5 and 16: the fold count is read from the launch and
    the inputs pass through LDS four at a time), buffers that share an offset from a 16-byte boundary,
    and the ring replay's two-input steps and copies."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(277 + dtype)
    cases = ((5, 0, mr.Schedule.FUSED, orc.SUM, orc.ORDER_UCX), (16, 0, mr.Schedule.FUSED, orc.MAX, orc.ORDER_SHM),
             (8, max(size, 4), mr.Schedule.FUSED, orc.SUM, orc.ORDER_UCX), (3, 0, mr.Schedule.RING, orc.MIN, orc.ORDER_UCX),
             (4, 0, mr.Schedule.RING, orc.SUM, orc.ORDER_UCX))
    for nranks, offset, sched, op, order in cases:
        if sched == mr.Schedule.RING and dtype == orc.FLOAT16:
            continue  # the ring replay would round at every hop and is refused for FLOAT16
        per_chunk = 8300 if sched == mr.Schedule.RING else 0  # ring steps work on one chunk per rank
        tiles = max(8300, per_chunk * nranks)
        length = tiles * 1024 // size + 7
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        d_in = [to_device(x, offset) for x in ins]
        d_out = [empty_device(length * size, offset) for _ in range(nranks)]
        runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, d_in, d_out, length, dtype, order, sched)
        assert any(r["waves"] == 4 and r["vector"] == 1 for r in runs), "the segment group form is not what runs here"
        want = orc.fold_all_reduce(ins, dtype, op, order)
        got = run_all_reduce(ins, dtype, op, order, sched, offsets=[offset] * nranks)
        for r in range(nranks):
            assert_same(got[r], want[r], f"segment group form dtype={dtype} N={nranks} offset={offset} sched={sched} "
                                         f"op={op} rank={r}")
        if sched == mr.Schedule.FUSED:
            got = run_all_reduce(ins, dtype, op, order, sched, offsets=[offset] * nranks, inplace=True)
            for r in range(nranks):
                assert_same(got[r], want[r], f"in-place segment group form dtype={dtype} N={nranks} rank={r}")
    # a long copy with a common offset: broadcast through the general kernel's copy
    nranks, offset = 5, max(size, 4)
    length = 4200 * 1024 // size + 3
    src = rand_array(dtype, length, rng)
    d_src = to_device(src, offset)
    d_out = [empty_device(length * size, offset) for _ in range(nranks)]
    mr.broadcast(d_src, d_out, length, dtype, 2)
    torch.cuda.synchronize()
    for r in range(nranks):
        assert_same(to_host(d_out[r], src.dtype), src, f"long unaligned broadcast dtype={dtype} rank={r}")


def tree_expectation(ins, dtype, op, root):
    """reduce towards `root`: the oracle's literal replay of the binomial tree; FLOAT16 (which the
    reference cannot reduce) as the same tree in fp32 with one rounding."""
    nranks = len(ins)
    if dtype != orc.FLOAT16:
        return orc.ucx_reduce(ins, dtype, op, root)[root]
    a = [ins[(root + v) % nranks].astype(np.float32) for v in range(nranks)]
    bit = 1
    while bit < nranks:
        for v in range(0, nranks - bit, 2 * bit):
            x, y = a[v], a[v + bit]
            with np.errstate(over="ignore"):
                a[v] = {orc.SUM: x + y, orc.MAX: np.where(y > x, y, x), orc.MIN: np.where(y < x, y, x)}[op]
        bit *= 2
    with np.errstate(over="ignore"):
        return a[0].astype(np.float16)


@pytest.mark.parametrize("dtype", [orc.FLOAT32, orc.FLOAT16, orc.UINT8, orc.INT64])
def test_tree_reduce_for_every_batch_shape(dtype, monkeypatch):
    """reduce towards a root in the reference's binomial-tree order (src/ucx/reduce.cpp:56-80) for rank counts without a
    flat kernel.  The kernel takes the tree eight leaves at a time - whole and partial batches, one to four of them -
    or walks it leaf by leaf (twelve and more ranks between 2 and 8 MiB per buffer; up to nine ranks of 4- and 8-byte
    elements where the stores stream, forced here through the store policy): every rank count's tree against the
    oracle's literal replay, ragged lengths, every root position class."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(4100 + dtype)
    for nranks in (5, 6, 7, 9, 10, 11, 13, 15, 16, 17, 23, 25, 31):
        for policy, length in (("", 70001), ("never", 33003), ("", (3000 * 1024) // size + 5 if nranks in (13, 25) else 0)):
            if not length:
                continue
            if policy:
                monkeypatch.setenv("MEGRAY_VRANK_KEEP", policy)
            else:
                monkeypatch.delenv("MEGRAY_VRANK_KEEP", raising=False)
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            d_in = [to_device(x) for x in ins]
            for op, root in ((orc.SUM, nranks - 1), (orc.MAX, nranks // 2)):
                out = empty_device(length * size)
                mr.reduce_to_root(d_in, out, length, dtype, op, root)
                torch.cuda.synchronize()
                assert_same(to_host(out, ins[0].dtype), tree_expectation(ins, dtype, op, root),
                            f"tree reduce dtype={dtype} N={nranks} len={length} policy={policy!r} op={op} root={root}")
    monkeypatch.delenv("MEGRAY_VRANK_KEEP", raising=False)


@pytest.mark.parametrize("dtype", [orc.FLOAT32, orc.FLOAT16, orc.INT8, orc.INT64])
def test_large_folds_into_one_output_at_reduced_occupancy(dtype):
    """reduce_scatter, reduce towards a root and the two-phase all_reduce from 8192 tiles per buffer on (four ranks:
    from 65536 on), tiles on cache-line boundaries, three or more ranks: one wavefront per tile, launched with LDS
    reserved per workgroup so that the number of wavefronts sharing a CU is the one that serves the shape best -
    eagerly, as a planned HIP graph (the reservation is part of the kernel node), with four ranks on either side of
    their threshold and with two ranks (which stay in the group form)."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(991 + dtype)
    for nranks, tiles, waves in ((8, 8200, 1), (3, 8200, 1), (2, 15400, 4), (4, 8200, 4), (4, 65600, 1)):
        recvlen = (tiles * 1024 // size + nranks - 1) // nranks // 128 * 128 + 128  # chunks on 128-byte boundaries
        length = recvlen * nranks
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        d_in = [to_device(x) for x in ins]
        parts = [empty_device(recvlen * size) for _ in range(nranks)]
        runs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, d_in, parts, recvlen, dtype)
        assert runs and all(r["waves"] == waves for r in runs), "not the kernel form this test is about"
        for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MIN, orc.ORDER_SHM)):
            want = orc.fold_reduce_scatter(ins, dtype, op, order)
            mr.reduce_scatter(d_in, parts, recvlen, dtype, op, order)
            torch.cuda.synchronize()
            for r in range(nranks):
                assert_same(to_host(parts[r], ins[0].dtype), want[r], f"reduce_scatter dtype={dtype} N={nranks} op={op} rank={r}")
            plan = mr.CollectivePlan(mr.Collective.REDUCE_SCATTER, d_in, parts, recvlen, dtype, op, order=order, graph=True)
            for replay in range(2):
                for o in parts:
                    o.fill_(replay)
                torch.cuda.synchronize()
                plan.launch()
                torch.cuda.synchronize()
                for r in range(nranks):
                    assert_same(to_host(parts[r], ins[0].dtype), want[r], f"planned reduce_scatter dtype={dtype} N={nranks} replay={replay}")
            plan.close()
        root = nranks - 1
        out = empty_device(length * size)
        mr.reduce_to_root(d_in, out, length, dtype, orc.MAX, root)
        torch.cuda.synchronize()
        assert_same(to_host(out, ins[0].dtype), tree_expectation(ins, dtype, orc.MAX, root), f"tree reduce dtype={dtype} N={nranks}")
        mr.reduce_to_root(d_in, out, length, dtype, orc.SUM, root, orc.ORDER_RANK0)
        torch.cuda.synchronize()
        assert_same(to_host(out, ins[0].dtype), orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_RANK0)[0],
                    f"left-fold reduce dtype={dtype} N={nranks}")
        got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, mr.Schedule.TWO_PHASE)
        want = orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX)
        for r in range(nranks):
            assert_same(got[r], want[r], f"two-phase all_reduce dtype={dtype} N={nranks} rank={r}")


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_group_form_with_one_output(dtype):
    """reduce_scatter, reduce towards a root and the two-phase all_reduce on long buffers: the
    group form in which every wavefront stores the tile it folded (shifted outputs, one destination)."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(177 + dtype)
    for nranks, tiles in ((4, 6500), (8, 4999)):
        recvlen = (tiles * 1024 // size) // nranks // 16 * 16 + 16  # keeps chunk r of rank r on a 16-byte boundary
        length = recvlen * nranks
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        d_in = [to_device(x) for x in ins]
        parts = [empty_device(recvlen * size) for _ in range(nranks)]
        runs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, d_in, parts, recvlen, dtype)
        assert runs and all(r["waves"] == 4 for r in runs), "the group form is not what runs here"
        for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MAX, orc.ORDER_UCX), (orc.MIN, orc.ORDER_SHM)):
            want = orc.fold_reduce_scatter(ins, dtype, op, order)
            mr.reduce_scatter(d_in, parts, recvlen, dtype, op, order)
            torch.cuda.synchronize()
            for r in range(nranks):
                assert_same(to_host(parts[r], ins[0].dtype), want[r],
                            f"reduce_scatter group form dtype={dtype} N={nranks} op={op} order={order} rank={r}")
            # in place: rank r's result lands on its own chunk r
            d_io = [to_device(x) for x in ins]
            mr.reduce_scatter(d_io, [d_io[r][r * recvlen * size:(r + 1) * recvlen * size] for r in range(nranks)],
                              recvlen, dtype, op, order)
            torch.cuda.synchronize()
            for r in range(nranks):
                got = to_host(d_io[r], ins[0].dtype)[r * recvlen:(r + 1) * recvlen]
                assert_same(got, want[r], f"in-place reduce_scatter group form dtype={dtype} N={nranks} rank={r}")
        for op in (orc.SUM, orc.MAX):
            root = nranks - 2
            out = empty_device(length * size)
            mr.reduce_to_root(d_in, out, length, dtype, op, root)
            torch.cuda.synchronize()
            assert_same(to_host(out, ins[0].dtype), tree_expectation(ins, dtype, op, root),
                        f"tree reduce group form dtype={dtype} N={nranks} op={op}")
            mr.reduce_to_root(d_in, out, length, dtype, op, root, orc.ORDER_RANK0)
            torch.cuda.synchronize()
            assert_same(to_host(out, ins[0].dtype), orc.fold_all_reduce(ins, dtype, op, orc.ORDER_RANK0)[0],
                        f"left-fold reduce group form dtype={dtype} N={nranks} op={op}")
        want = orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX)
        got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, mr.Schedule.TWO_PHASE)
        for r in range(nranks):
            assert_same(got[r], want[r], f"two-phase group form dtype={dtype} N={nranks} rank={r}")


@pytest.mark.parametrize("dtype", [orc.INT8, orc.INT32, orc.FLOAT32, orc.FLOAT64, orc.UINT64])
def test_all_reduce_equals_literal_ring_replay(dtype):
    """Against the oracle's literal replay of src/ucx/all_reduce.cpp, not only its fold form."""
    rng = np.random.default_rng(dtype)
    for nranks in (2, 3, 4, 8):
        for length in (nranks * 1000 + 7, 13):
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            for op in OPS:
                want = orc.ucx_all_reduce(ins, dtype, op)
                for sched in (mr.Schedule.FUSED, mr.Schedule.TWO_PHASE, mr.Schedule.RING):
                    got = run_all_reduce(ins, dtype, op, orc.ORDER_UCX, sched)
                    for r in range(nranks):
                        assert_same(got[r], want[r], f"dtype={dtype} N={nranks} len={length} op={op} sched={sched}")
                if dtype in (orc.INT8, orc.INT32, orc.FLOAT32):
                    want = orc.shm_all_reduce(ins, dtype, op)
                    for sched in (mr.Schedule.FUSED, mr.Schedule.TWO_PHASE):
                        got = run_all_reduce(ins, dtype, op, orc.ORDER_SHM, sched)
                        for r in range(nranks):
                            assert_same(got[r], want[r], f"shm dtype={dtype} N={nranks} op={op} sched={sched}")


def test_all_reduce_in_place_and_misaligned():
    rng = np.random.default_rng(77)
    for dtype in (orc.FLOAT32, orc.INT8, orc.FLOAT16, orc.INT64):
        size = orc.dtype_size(dtype)
        for nranks in (3, 8):
            ins = [rand_array(dtype, 5000 + nranks, rng) for _ in range(nranks)]
            want = orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX)
            scheds = [mr.Schedule.FUSED, mr.Schedule.TWO_PHASE]
            if dtype == orc.FLOAT16:  # a ring hop would round to fp16 every time
                with pytest.raises(mr.MegRayError, match="ring schedule"):
                    run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, mr.Schedule.RING)
            else:
                scheds.append(mr.Schedule.RING)
            for sched in scheds:
                got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, sched, inplace=True)
                for r in range(nranks):
                    assert_same(got[r], want[r], f"in-place dtype={dtype} sched={sched}")
                # every rank buffer off 16-byte alignment by a different element count
                offs = [size * (1 + r % 3) for r in range(nranks)]
                got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, sched, offsets=offs)
                for r in range(nranks):
                    assert_same(got[r], want[r], f"misaligned dtype={dtype} sched={sched}")
                # all buffers off by the same element count: vector body behind a longer scalar head
                got = run_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX, sched, offsets=[size * 3] * nranks)
                for r in range(nranks):
                    assert_same(got[r], want[r], f"common offset dtype={dtype} sched={sched}")


def test_float_special_values_and_tie_conventions():
    """+-0, NaN, inf and denormals through MAX/MIN/SUM: compare + select must follow the reference's
    ?: (src/ucx/kernel.cu:24-38), not the hardware's max/min."""
    n = 4
    base = np.array([0.0, -0.0, np.nan, 1.0, -1.0, np.inf, -np.inf, 1e-45, -1e-45, 3e38, -3e38, 2.5],
                    dtype=np.float64)
    rng = np.random.default_rng(3)
    for dtype in (orc.FLOAT32, orc.FLOAT64, orc.FLOAT16):
        npdt = orc.NP_DTYPE[dtype]
        with np.errstate(over="ignore", under="ignore"):
            vals = base.astype(npdt)
        ins = [rng.choice(vals, size=4096 + 5).astype(npdt) for _ in range(n)]
        # the same through the group kernels: 2600 tiles per buffer
        long_ins = [rng.choice(vals, size=2600 * 1024 // orc.dtype_size(dtype) + 5).astype(npdt) for _ in range(n)]
        for op in OPS:
            for order in ORDERS:
                for data in (ins, long_ins):
                    want = orc.fold_all_reduce(data, dtype, op, order)[0]
                    got = run_all_reduce(data, dtype, op, order, mr.Schedule.FUSED)[0]
                    nan = np.isnan(want)
                    assert np.array_equal(np.isnan(got), nan), f"NaN placement dtype={dtype} op={op} order={order}"
                    assert_same(got[~nan], want[~nan], f"specials dtype={dtype} op={op} order={order} len={data[0].size}")
            rs_in = [x[:4096] for x in ins]
            want = orc.fold_reduce_scatter(rs_in, dtype, op, orc.ORDER_UCX)
            d_in = [to_device(x) for x in rs_in]
            d_out = [empty_device(1024 * orc.dtype_size(dtype)) for _ in range(n)]
            mr.reduce_scatter(d_in, d_out, 1024, dtype, op)
            torch.cuda.synchronize()
            for r in range(n):
                got = to_host(d_out[r], npdt)
                nan = np.isnan(want[r])
                assert np.array_equal(np.isnan(got), nan)
                assert_same(got[~nan], want[r][~nan], f"reduce_scatter specials dtype={dtype} op={op}")


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_reduce_scatter(dtype):
    rng = np.random.default_rng(50 + dtype)
    size = orc.dtype_size(dtype)
    for nranks in (1, 2, 3, 8):
        for recvlen in (0, 1, 5, 144, 1024, 4099):  # 144: aligned chunks whose borders fall inside tiles
            ins = [rand_array(dtype, nranks * recvlen, rng) for _ in range(nranks)]
            for op in OPS:
                for order in ORDERS:
                    want = orc.fold_reduce_scatter(ins, dtype, op, order)
                    d_in = [to_device(x) for x in ins]
                    d_out = [empty_device(recvlen * size) for _ in range(nranks)]
                    mr.reduce_scatter(d_in, d_out, recvlen, dtype, op, order)
                    torch.cuda.synchronize()
                    for r in range(nranks):
                        assert_same(to_host(d_out[r], ins[0].dtype), want[r],
                                    f"reduce_scatter dtype={dtype} N={nranks} recvlen={recvlen} op={op} order={order}")
            if dtype in (orc.INT32, orc.FLOAT32, orc.FLOAT64) and recvlen:
                want = orc.ucx_reduce_scatter(ins, dtype, orc.SUM)  # the literal replay
                d_in = [to_device(x) for x in ins]
                d_out = [empty_device(recvlen * size) for _ in range(nranks)]
                mr.reduce_scatter(d_in, d_out, recvlen, dtype, orc.SUM)
                torch.cuda.synchronize()
                for r in range(nranks):
                    assert_same(to_host(d_out[r], ins[0].dtype), want[r], "reduce_scatter vs literal replay")


COPY_TYPES = [orc.UINT8, orc.FLOAT16, orc.FLOAT32, orc.INT64, orc.CHAR]


@pytest.mark.parametrize("dtype", COPY_TYPES)
def test_pack_collectives(dtype):
    rng = np.random.default_rng(90 + dtype)
    size = orc.dtype_size(dtype)
    for nranks in (1, 2, 3, 8, 16):
        for length in (0, 1, 6, 1000, 4096 + 3):
            for misalign in (0, size):
                check_pack_collectives(dtype, nranks, length, misalign, rng)


@pytest.mark.parametrize("dtype", [orc.UINT8, orc.FLOAT16, orc.INT64])
def test_pack_collectives_group_form(dtype):
    """Long blocks go through the group form of the pack kernel (four wavefronts, four tiles per workgroup; an
    all_gather of three ranks from 8192 tiles per block on, of eight from 2048, a broadcast from 2048, the others from
    128); the block ends in a partial tile."""
    rng = np.random.default_rng(190 + dtype)
    size = orc.dtype_size(dtype)
    for nranks, tiles in ((3, 8200), (8, 2060)):
        length = (tiles * 1024 + 48) // size
        runs, _, _ = mr.describe(mr.Collective.ALL_GATHER, [(1 << 40) + (r << 30) for r in range(nranks)],
                                 [(2 << 40) + (r << 34) for r in range(nranks)], length, dtype)
        assert runs and all(r["waves"] == 4 and r["vector"] == 16 for r in runs), "the group form is not what runs here"
        check_pack_collectives(dtype, nranks, length, 0, rng)
    # just below those sizes an all_gather and a broadcast keep one wavefront per tile, the others are in the group form
    for nranks, tiles in ((3, 8100), (8, 2000)):
        length = (tiles * 1024 + 48) // size
        runs, _, _ = mr.describe(mr.Collective.ALL_GATHER, [(1 << 40) + (r << 30) for r in range(nranks)],
                                 [(2 << 40) + (r << 34) for r in range(nranks)], length, dtype)
        assert runs and all(r["waves"] == 1 and r["vector"] == 16 for r in runs), "one wavefront per tile is not what runs here"
        check_pack_collectives(dtype, nranks, length, 0, rng)


@pytest.mark.parametrize("pace", ["always", "never"])
def test_pack_collectives_group_form_with_paced_stores(pace, monkeypatch):
    """A long all_gather or broadcast in the group form issues a wavefront's stores one at a time (the planner decides
    by rank count and size); MEGRAY_VRANK_PACE forces that on (and off) here at a size the oracle handles.  Same
    permutations either way."""
    monkeypatch.setenv("MEGRAY_VRANK_PACE", pace)
    rng = np.random.default_rng(290)
    for dtype in (orc.UINT8, orc.FLOAT32):
        for nranks, tiles in ((3, 8200), (8, 2060)):  # long enough for the group form of every pack collective
            check_pack_collectives(dtype, nranks, (tiles * 1024 + 48) // orc.dtype_size(dtype), 0, rng)


def test_many_rank_gathers_and_broadcasts_pace_their_stores_by_themselves():
    """From twelve ranks on an all_gather in the group form issues a wavefront's stores one at a time whatever the
    buffers' addresses, and so does a broadcast of 16 MiB and more to nine ranks and more: the same permutations."""
    rng = np.random.default_rng(291)
    length = 1030 * 1024 + 48
    for nranks in (12, 16):
        runs, _, _ = mr.describe(mr.Collective.ALL_GATHER, [(1 << 40) + (r << 30) for r in range(nranks)],
                                 [(2 << 40) + (r << 34) for r in range(nranks)], length, orc.UINT8)
        assert runs and all(r["waves"] == 4 and r["paced"] == 1 for r in runs)
        check_pack_collectives(orc.UINT8, nranks, length, 0, rng)
    nranks, length, root = 9, (16 << 20) + 48, 4
    runs, _, _ = mr.describe(mr.Collective.BROADCAST, [1 << 40] * nranks, [(2 << 40) + (r << 34) for r in range(nranks)],
                             length, orc.UINT8, root=root)
    assert runs and all(r["waves"] == 4 and r["paced"] == 1 for r in runs)
    block = rand_array(orc.UINT8, length, rng)
    d_root = to_device(block)
    d_out = [empty_device(length) for _ in range(nranks)]
    mr.broadcast(d_root, d_out, length, orc.UINT8, root)
    torch.cuda.synchronize()
    for r in range(nranks):
        assert_same(to_host(d_out[r], block.dtype), block, f"paced broadcast rank={r}")


def check_pack_collectives(dtype, nranks, length, misalign, rng):
    size = orc.dtype_size(dtype)
    gen = orc.UINT8 if dtype == orc.CHAR else dtype
    ins = [rand_array(gen, nranks * length, rng) for _ in range(nranks)]
    npdt = ins[0].dtype
    # all_to_all
    want = orc.ucx_all_to_all(ins, dtype)
    d_in = [to_device(x, misalign) for x in ins]
    d_out = [empty_device(nranks * length * size, misalign) for _ in range(nranks)]
    mr.all_to_all(d_in, d_out, length, dtype)
    torch.cuda.synchronize()
    for r in range(nranks):
        assert_same(to_host(d_out[r], npdt), want[r], f"all_to_all dtype={dtype} N={nranks} len={length}")
    # all_gather
    parts = [x[:length] for x in ins]
    want = orc.ucx_all_gather(parts, dtype)
    d_in = [to_device(x, misalign) for x in parts]
    d_out = [empty_device(nranks * length * size, misalign) for _ in range(nranks)]
    mr.all_gather(d_in, d_out, length, dtype)
    torch.cuda.synchronize()
    for r in range(nranks):
        assert_same(to_host(d_out[r], npdt), want[r], f"all_gather dtype={dtype} N={nranks} len={length}")
    root = nranks // 2
    # scatter: only the root has a send buffer
    want = orc.ucx_scatter([ins[root] if r == root else None for r in range(nranks)], dtype, root)
    d_root = to_device(ins[root], misalign)
    d_out = [empty_device(length * size, misalign) for _ in range(nranks)]
    mr.scatter(d_root, d_out, length, dtype, root)
    torch.cuda.synchronize()
    for r in range(nranks):
        assert_same(to_host(d_out[r], npdt), want[r], f"scatter dtype={dtype} N={nranks} len={length}")
    # gather: only the root has a receive buffer
    want = orc.ucx_gather(parts, dtype, root)[root]
    d_in = [to_device(x, misalign) for x in parts]
    d_root = empty_device(nranks * length * size, misalign)
    mr.gather(d_in, d_root, length, dtype, root)
    torch.cuda.synchronize()
    assert_same(to_host(d_root, npdt), want, f"gather dtype={dtype} N={nranks} len={length}")
    # broadcast (the ucx tree of src/ucx/broadcast.cpp:21-76 and the shm arena of src/shm/broadcast.cpp:19-51 agree)
    want = orc.ucx_broadcast(parts, dtype, root)
    want_shm = orc.shm_broadcast(parts, dtype, root)
    for r in range(nranks):
        assert_same(want_shm[r], want[r], "the two broadcast replays")
    d_root = to_device(parts[root], misalign)
    d_out = [empty_device(length * size, misalign) for _ in range(nranks)]
    mr.broadcast(d_root, d_out, length, dtype, root)
    torch.cuda.synchronize()
    for r in range(nranks):
        assert_same(to_host(d_out[r], npdt), want[r], f"broadcast dtype={dtype} N={nranks} len={length}")


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_two_input_reduce(dtype):
    """mrv_reduce against the oracle's restatement of MegRay::reduce (src/ucx/kernel.cu:60-98)."""
    rng = np.random.default_rng(dtype)
    size = orc.dtype_size(dtype)
    for length in (0, 1, 255, 4096, 100003):
        a, b = rand_array(dtype, length, rng), rand_array(dtype, length, rng)
        for op in OPS:
            if dtype == orc.FLOAT16:  # the reference has no FLOAT16 reduce: fp32 arithmetic, one rounding
                with np.errstate(over="ignore"):
                    a32, b32 = a.astype(np.float32), b.astype(np.float32)
                    want = {orc.SUM: (a32 + b32), orc.MAX: np.where(a32 > b32, a32, b32),
                            orc.MIN: np.where(a32 < b32, a32, b32)}[op].astype(np.float16)
            else:
                want = orc.reduce_ucx(a, b, dtype, op)
            d_a, d_b = to_device(a), to_device(b)
            d_o = empty_device(length * size)
            mr.reduce(d_a, d_b, d_o, length, dtype, op)
            torch.cuda.synchronize()
            assert_same(to_host(d_o, a.dtype), want, f"reduce dtype={dtype} len={length} op={op}")
            # in place on the first operand, as every reference caller uses it
            mr.reduce(d_a, d_b, d_a, length, dtype, op)
            torch.cuda.synchronize()
            assert_same(to_host(d_a, a.dtype), want, f"reduce in place dtype={dtype} len={length} op={op}")


def test_reference_closed_forms_on_gpu():
    """The reference's own test vectors (test/test_opr.cpp:286-359, 361-438, 198-257)."""
    n, length = 3, 10
    ins = [np.array([(i + 1) * (j + 1) for j in range(length)], dtype=np.float32) for i in range(n)]
    j1 = np.arange(1, length + 1, dtype=np.float32)
    for op, want in ((orc.SUM, 6 * j1), (orc.MAX, 3 * j1), (orc.MIN, j1)):
        for order in ORDERS:
            for r, got in enumerate(run_all_reduce(ins, orc.FLOAT32, op, order, mr.Schedule.FUSED)):
                assert np.array_equal(got, want)
    recvlen = 10
    ins = [np.array([(i + 1) * (m + 1) for m in range(n * recvlen)], dtype=np.float32) for i in range(n)]
    for op, factor in ((orc.SUM, 6), (orc.MAX, 3), (orc.MIN, 1)):
        d_in = [to_device(x) for x in ins]
        d_out = [empty_device(recvlen * 4) for _ in range(n)]
        mr.reduce_scatter(d_in, d_out, recvlen, orc.FLOAT32, op)
        torch.cuda.synchronize()
        for k in range(n):
            want = np.array([factor * (k * recvlen + j + 1) for j in range(recvlen)], dtype=np.float32)
            assert np.array_equal(to_host(d_out[k], np.float32), want)
    length = 6
    ins = [np.array([(i + 1) * (j + 2) * (k + 3) for j in range(n) for k in range(length)], dtype=np.float32)
           for i in range(n)]
    d_in = [to_device(x) for x in ins]
    d_out = [empty_device(n * length * 4) for _ in range(n)]
    mr.all_to_all(d_in, d_out, length, orc.FLOAT32)
    torch.cuda.synchronize()
    for j in range(n):
        want = np.array([(i + 1) * (j + 2) * (k + 3) for i in range(n) for k in range(length)], dtype=np.float32)
        assert np.array_equal(to_host(d_out[j], np.float32), want)


def test_errors_follow_the_reference():
    d = to_device(np.zeros(64, dtype=np.float32))
    o = empty_device(256)
    with pytest.raises(mr.MegRayError, match="unknown dtype"):      # src/ucx/kernel.cu:95-96
        mr.reduce(d, d, o, 64, mr.DType.CHAR, mr.ReduceOp.SUM)
    with pytest.raises(mr.MegRayError, match="unknown dtype"):
        mr.all_reduce([d], [o], 64, 17, mr.ReduceOp.SUM)
    with pytest.raises(mr.MegRayError, match="unknown reduce op"):  # src/ucx/kernel.cu:55-56
        mr.all_reduce([d], [o], 64, mr.DType.FLOAT32, 3)
    with pytest.raises(mr.MegRayError, match="overlap"):
        mr.all_reduce([d, d], [o, o], 64, mr.DType.FLOAT32, mr.ReduceOp.SUM)
    with pytest.raises(mr.MegRayError, match="nranks"):
        mr.all_reduce([d] * 33, [o] * 33, 1, mr.DType.FLOAT32, mr.ReduceOp.SUM)
    torch.cuda.synchronize()


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
def test_reduce_to_root(dtype):
    """ucx order = the binomial tree of src/ucx/reduce.cpp:56-80, against the oracle's literal replay
    (FLOAT16: the same tree in fp32 with one rounding)."""
    rng = np.random.default_rng(300 + dtype)
    size = orc.dtype_size(dtype)
    for nranks in (1, 2, 3, 4, 5, 8, 11):
        for length in (0, 1, 777, 4096 * 4 + 5):
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            for root in sorted({0, nranks - 1}):
                for op in OPS:
                    for misalign in (0, size):
                        d_in = [to_device(x, misalign) for x in ins]
                        d_out = empty_device(length * size, misalign)
                        mr.reduce_to_root(d_in, d_out, length, dtype, op, root)
                        torch.cuda.synchronize()
                        got = to_host(d_out, ins[0].dtype)
                        want = tree_expectation(ins, dtype, op, root)
                        assert_same(got, want, f"reduce dtype={dtype} N={nranks} len={length} root={root} op={op}")
                    for order in (orc.ORDER_SHM, orc.ORDER_RANK0):
                        d_in = [to_device(x) for x in ins]
                        d_out = empty_device(length * size)
                        mr.reduce_to_root(d_in, d_out, length, dtype, op, root, order)
                        torch.cuda.synchronize()
                        got = to_host(d_out, ins[0].dtype)
                        assert_same(got, orc.fold_all_reduce(ins, dtype, op, order)[0], f"reduce order={order}")
                        if order == orc.ORDER_SHM and dtype in SHM_REDUCE_TYPES:
                            # the literal replay of src/shm/reduce.cpp:21-100, mutexes and all
                            assert_same(got, orc.shm_reduce(ins, dtype, op, root)[root], "reduce vs shm replay")


def test_planned_collectives_and_graph_replay():
    """mrv_plan_*: a plan launched repeatedly, eagerly and as a HIP graph of kernel nodes, gives the
    eager result on every replay, with other work and host syncs between the replays."""
    rng = np.random.default_rng(11)
    nranks = 8
    # the second length runs the group kernels (workgroups of 256 threads) also as graph nodes
    for sched, length in ((mr.Schedule.FUSED, 40000 + 3), (mr.Schedule.TWO_PHASE, 40000 + 3),
                          (mr.Schedule.RING, 40000 + 3), (mr.Schedule.FUSED, 2700 * 256 + 5),
                          (mr.Schedule.TWO_PHASE, 5000 * 256 + 5)):
        ins = [rand_array(orc.FLOAT32, length, rng) for _ in range(nranks)]
        want = orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM)
        d_in = [to_device(x) for x in ins]
        for graph in (False, True):
            d_out = [empty_device(length * 4) for _ in range(nranks)]
            plan = mr.CollectivePlan(mr.Collective.ALL_REDUCE, d_in, d_out, length, mr.DType.FLOAT32, mr.ReduceOp.SUM,
                                     schedule=sched, graph=graph)
            assert plan.launch_count == {mr.Schedule.FUSED: 1, mr.Schedule.TWO_PHASE: 2,
                                         mr.Schedule.RING: 1 + 2 * (nranks - 1)}[sched]
            for replay in range(4):
                for o in d_out:
                    o.fill_(replay)  # the program's own eager work between replays
                torch.cuda.synchronize()
                plan.launch()
                torch.cuda.synchronize()
                for r in range(nranks):
                    assert_same(to_host(d_out[r], np.float32), want[r], f"sched={sched} graph={graph} replay={replay}")
            plan.close()
    # new data in the same buffers is picked up by a replay (the plan holds addresses, not values)
    ins = [rand_array(orc.INT32, 5000, rng) for _ in range(4)]
    d_in = [to_device(x) for x in ins]
    d_out = [empty_device(5000 * 4) for _ in range(4)]
    plan = mr.CollectivePlan(mr.Collective.ALL_REDUCE, d_in, d_out, 5000, mr.DType.INT32, mr.ReduceOp.MAX,
                             schedule=mr.Schedule.TWO_PHASE, graph=True)
    for _ in range(3):
        ins = [rand_array(orc.INT32, 5000, rng) for _ in range(4)]
        for d, x in zip(d_in, ins):
            d.copy_(torch.from_numpy(x.view(np.uint8).copy()))
        plan.launch()
        torch.cuda.synchronize()
        assert_same(to_host(d_out[2], np.int32), np.stack(ins).max(axis=0), "graph replay on new data")
    with pytest.raises(mr.MegRayError, match="unknown reduce op"):
        mr.CollectivePlan(mr.Collective.ALL_REDUCE, d_in, d_out, 5000, mr.DType.INT32, 9)
    # the other collectives plan and replay the same way (here: blocks long enough for the group kernels)
    nranks, block = 4, 200 * 1024 + 16
    parts = [rand_array(orc.UINT8, block, rng) for _ in range(nranks)]
    d_parts = [to_device(x) for x in parts]
    d_all = [empty_device(nranks * block) for _ in range(nranks)]
    gather_plan = mr.CollectivePlan(mr.Collective.ALL_GATHER, d_parts, d_all, block, mr.DType.UINT8, graph=True)
    want = orc.ucx_all_gather(parts, orc.UINT8)
    for _ in range(2):
        for o in d_all:
            o.zero_()
        gather_plan.launch()
        torch.cuda.synchronize()
        for r in range(nranks):
            assert_same(to_host(d_all[r], np.uint8), want[r], "planned all_gather")
    gather_plan.close()
    ins = [rand_array(orc.INT32, nranks * 150 * 256, rng) for _ in range(nranks)]
    d_in = [to_device(x) for x in ins]
    d_out = [empty_device(150 * 256 * 4) for _ in range(nranks)]
    rs_plan = mr.CollectivePlan(mr.Collective.REDUCE_SCATTER, d_in, d_out, 150 * 256, mr.DType.INT32, mr.ReduceOp.MIN)
    want = orc.fold_reduce_scatter(ins, orc.INT32, orc.MIN, orc.ORDER_UCX)
    for _ in range(2):
        rs_plan.launch()
        torch.cuda.synchronize()
        for r in range(nranks):
            assert_same(to_host(d_out[r], np.int32), want[r], "planned reduce_scatter")
    rs_plan.close()


def test_sixteen_ranks_many_segments():
    """16 ranks with ragged, unaligned pieces: more runs than one launch descriptor holds, so the
    planner splits the collective over several launches."""
    rng = np.random.default_rng(16)
    nranks, recvlen = 16, 1031
    for dtype in (orc.FLOAT32, orc.INT8):
        size = orc.dtype_size(dtype)
        ins = [rand_array(dtype, nranks * recvlen, rng) for _ in range(nranks)]
        for order in ORDERS:
            want = orc.fold_reduce_scatter(ins, dtype, orc.SUM, order)
            d_in = [to_device(x, size * (r % 3)) for r, x in enumerate(ins)]
            d_out = [empty_device(recvlen * size, size * (r % 2)) for r in range(nranks)]
            runs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, d_in, d_out, recvlen, dtype, order)
            mr.reduce_scatter(d_in, d_out, recvlen, dtype, orc.SUM, order)
            torch.cuda.synchronize()
            for r in range(nranks):
                assert_same(to_host(d_out[r], ins[0].dtype), want[r], f"N=16 reduce_scatter dtype={dtype} order={order}")
            if order == orc.ORDER_SHM:
                assert len({run["step"] for run in runs}) == 1 or len(runs) > 96
            want = orc.fold_all_reduce(ins, dtype, orc.MAX, order)
            d_out = [empty_device(nranks * recvlen * size, size * (r % 2)) for r in range(nranks)]
            mr.all_reduce(d_in, d_out, nranks * recvlen, dtype, orc.MAX, order)
            torch.cuda.synchronize()
            for r in (0, 7, 15):
                assert_same(to_host(d_out[r], ins[0].dtype), want[r], f"N=16 all_reduce dtype={dtype} order={order}")
