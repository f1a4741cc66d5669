"""Host planner (no GPU): the launches mrv_describe() reports are interpreted here with numpy, run
by run, and must reproduce the oracle's literal replays bit for bit.  This checks chunking, fold
orders, tie conventions, the head / vector-body / tail split and the multi-launch schedules
independently of the kernels."""
import os

import numpy as np
import pytest

import megray_amd as mr
import oracle as orc

SEND_BASE = 0x100000000000
RECV_BASE = 0x200000000000
STRIDE = 0x001000000000

REDUCE_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.UINT64, orc.FLOAT32, orc.FLOAT64]


def rand_array(dtype, n, rng):
    npdt = orc.NP_DTYPE[dtype]
    if np.issubdtype(npdt, np.integer):
        raw = rng.integers(0, 2 ** 64, size=n, dtype=np.uint64)
        return raw.astype(np.dtype(npdt).str.replace("i", "u")).view(npdt)
    return (rng.standard_normal(n) * np.exp(rng.uniform(-20, 20, n))).astype(npdt)


def fake_ptrs(base, n, offsets, stride=None):
    return [base + r * (stride or STRIDE) + offsets[r] for r in range(n)]


def combine(acc, x, op, new_wins):
    with np.errstate(over="ignore"):
        if op == orc.SUM:
            return acc + x
        if op == orc.MAX:
            return np.where(acc > x, acc, x) if new_wins else np.where(x > acc, x, acc)
        return np.where(acc < x, acc, x) if new_wins else np.where(x < acc, x, acc)


def execute(runs, sends, recvs, nranks, op, elem_size, send_ptrs, recv_ptrs):
    """Interpret plan runs in launch order.  Within one launch all reads happen on the values the
    previous launch left, unless a run reads and writes the very same element (in place)."""
    steps = sorted({r["step"] for r in runs})
    for step in steps:
        snapshot = [x.copy() for x in recvs]
        for run in (r for r in runs if r["step"] == step):
            if run["kind"] == 0:
                src = snapshot if run["reads_recv"] else sends
                lo, cnt = run["in_begin"], run["count"]
                if run["dir"] == 0:
                    # binomial tree towards rank `start` (src/ucx/reduce.cpp:56-80): virtual rank v takes in
                    # v + bit as reduce(incoming, own), own surviving a tie
                    ranks = [(run["start"] + v) % nranks for v in range(nranks)]
                    a = [src[r][lo:lo + cnt].copy() for r in ranks]
                    bit = 1
                    while bit < nranks:
                        for v in range(0, nranks - bit, 2 * bit):
                            a[v] = combine(a[v], a[v + bit], op, False)
                        bit *= 2
                    acc = a[0]
                else:
                    ranks = [(run["start"] + run["dir"] * j) % nranks for j in range(run["nfold"])]
                    acc = src[ranks[0]][lo:lo + cnt].copy()
                    for r in ranks[1:]:
                        acc = combine(acc, src[r][lo:lo + cnt], op, run["new_wins_ties"])
                for m in range(run["nout"]):
                    dst = (run["out_first"] + m) % nranks
                    recvs[dst][run["out_begin"]:run["out_begin"] + cnt] = acc
                if run["vector"]:
                    epv = 16 // elem_size
                    base_in = recv_ptrs if run["reads_recv"] else send_ptrs
                    # 16-byte accesses sit on 16-byte boundaries, except that elements are taken as they lie (gfx950
                    # serves 128-bit accesses at any byte address): buffers whose offsets from such a boundary
                    # differ, and inputs that are shifted against the outputs by a part of a vector (the outputs,
                    # i.e. the stores, then still sit on 16-byte boundaries).  The flat kernels use buffer
                    # instructions throughout, which need 4-byte boundaries.
                    touched = [p for p in list(send_ptrs) + list(recv_ptrs) if p]
                    need_out = 16 if len({p % 16 for p in touched}) == 1 else elem_size
                    need_in = need_out
                    if run["vector"] == 1:
                        assert cnt % epv == 0
                        if (lo - run["out_begin"]) % epv:
                            need_in = elem_size
                    else:
                        assert need_out == 16 or elem_size >= 4
                        if need_out == 16:  # flat launch: bases aligned, outputs shifted by whole vectors
                            assert (lo - run["out_begin"]) % epv == 0
                            lo = 0
                            run = dict(run, out_begin=0)
                    for r in ranks:
                        assert (base_in[r] + lo * elem_size) % need_in == 0
                    for m in range(run["nout"]):
                        dst = (run["out_first"] + m) % nranks
                        assert (recv_ptrs[dst] + run["out_begin"] * elem_size) % need_out == 0
            else:
                s = run["start"]
                a, b, cnt = run["in_begin"], run["out_begin"], run["count"]
                width = run["vector"]
                for m in range(run["nout"]):
                    d = (run["out_first"] + m) % nranks
                    recvs[d].view(np.uint8)[b:b + cnt] = sends[s].view(np.uint8)[a:a + cnt]
                    assert cnt % width == 0 and (send_ptrs[s] + a) % width == 0 and (recv_ptrs[d] + b) % width == 0
    return recvs


def bits_equal(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.mark.parametrize("dtype", REDUCE_TYPES)
@pytest.mark.parametrize("nranks", [1, 2, 3, 4, 7, 8, 16])
def test_all_reduce_plans_reproduce_the_replays(dtype, nranks):
    rng = np.random.default_rng(dtype * 100 + nranks)
    size = orc.dtype_size(dtype)
    for length in (0, 1, nranks - 1, 3 * nranks + 1, 300, 4099, 20011):
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        for misalign in (0, 1, 2):
            # 1: every rank off by a different element count; 2: all buffers off by the same count
            offs = {0: [0] * nranks, 1: [size * (r % 3) for r in range(nranks)], 2: [size] * nranks}[misalign]
            sp, rp = fake_ptrs(SEND_BASE, nranks, offs), fake_ptrs(RECV_BASE, nranks, offs)
            if misalign == 2 and length * size >= 2048 * nranks:  # every chunk outgrows its scalar head
                runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, sp, rp, length, dtype)
                assert any(r["vector"] == 1 for r in runs), "a common offset must keep the vector path"
            for op in (orc.SUM, orc.MAX, orc.MIN):
                cases = [(orc.ORDER_UCX, s) for s in (mr.Schedule.FUSED, mr.Schedule.TWO_PHASE, mr.Schedule.RING)]
                cases += [(orc.ORDER_SHM, s) for s in (mr.Schedule.FUSED, mr.Schedule.TWO_PHASE)]
                cases += [(orc.ORDER_RANK0, mr.Schedule.FUSED)]
                for order, sched in cases:
                    runs, br, bw = mr.describe(mr.Collective.ALL_REDUCE, sp, rp, length, dtype, order, sched)
                    recvs = [np.zeros(length, dtype=ins[0].dtype) for _ in range(nranks)]
                    got = execute(runs, ins, recvs, nranks, op, size, sp, rp)
                    if order == orc.ORDER_UCX:
                        want = orc.ucx_all_reduce(ins, dtype, op)
                    elif order == orc.ORDER_SHM and dtype in (orc.INT8, orc.UINT8, orc.INT32, orc.UINT32,
                                                              orc.INT64, orc.FLOAT32):
                        want = orc.shm_all_reduce(ins, dtype, op)
                    else:
                        want = orc.fold_all_reduce(ins, dtype, op, order)
                    for r in range(nranks):
                        assert bits_equal(got[r], want[r]), (dtype, nranks, length, misalign, op, order, sched)
                    # algorithmic bytes of the schedule
                    ns = length * size
                    if sched == mr.Schedule.FUSED:
                        assert (br, bw) == (nranks * ns, nranks * ns)
                    elif sched == mr.Schedule.TWO_PHASE:
                        assert (br, bw) == (nranks * ns + (ns if nranks > 1 else 0), ns + (nranks - 1) * ns)
                    else:  # N copies in, (N-1) steps of 2 reads + 1 write, (N-1) steps of 1 read + 1 write per chunk
                        assert br + bw == 2 * nranks * ns + 5 * (nranks - 1) * ns


@pytest.mark.parametrize("dtype", [orc.INT8, orc.INT32, orc.FLOAT32, orc.FLOAT64, orc.UINT64])
@pytest.mark.parametrize("nranks", [1, 2, 3, 8, 16])
def test_reduce_scatter_plans(dtype, nranks):
    rng = np.random.default_rng(dtype * 10 + nranks)
    size = orc.dtype_size(dtype)
    for recvlen in (0, 1, 3, 5, 64, 1031):
        ins = [rand_array(dtype, nranks * recvlen, rng) for _ in range(nranks)]
        sp, rp = fake_ptrs(SEND_BASE, nranks, [0] * nranks), fake_ptrs(RECV_BASE, nranks, [0] * nranks)
        for op in (orc.SUM, orc.MAX, orc.MIN):
            for order in (orc.ORDER_UCX, orc.ORDER_SHM, orc.ORDER_RANK0):
                runs, br, bw = mr.describe(mr.Collective.REDUCE_SCATTER, sp, rp, recvlen, dtype, order)
                recvs = [np.zeros(recvlen, dtype=ins[0].dtype) for _ in range(nranks)]
                got = execute(runs, ins, recvs, nranks, op, size, sp, rp)
                if order == orc.ORDER_UCX:
                    want = orc.ucx_reduce_scatter(ins, dtype, op)
                elif order == orc.ORDER_SHM and dtype in (orc.INT8, orc.INT32, orc.FLOAT32):
                    want = orc.shm_reduce_scatter(ins, dtype, op)
                else:
                    want = orc.fold_reduce_scatter(ins, dtype, op, order)
                for r in range(nranks):
                    assert bits_equal(got[r], want[r]), (dtype, nranks, recvlen, op, order)
                assert (br, bw) == (nranks * nranks * recvlen * size, nranks * recvlen * size)


@pytest.mark.parametrize("nranks", [1, 2, 3, 8, 16])
def test_pack_plans(nranks):
    rng = np.random.default_rng(nranks)
    for dtype in (orc.UINT8, orc.FLOAT16, orc.FLOAT32, orc.INT64, orc.CHAR):
        size = orc.dtype_size(dtype)
        gen = orc.UINT8 if dtype == orc.CHAR else dtype
        for length in (0, 1, 6, 100, 1030):
            for misalign in (0, size):
                offs = [misalign] * nranks
                sp, rp = fake_ptrs(SEND_BASE, nranks, offs), fake_ptrs(RECV_BASE, nranks, offs)
                ins = [rand_array(gen, nranks * length, rng) if gen != orc.FLOAT16
                       else rng.standard_normal(nranks * length).astype(np.float16) for _ in range(nranks)]
                npdt = ins[0].dtype

                def run(coll, sends, out_len, count, root=0):
                    runs, _, _ = mr.describe(coll, sp, rp, count, dtype, root=root, nranks=nranks)
                    recvs = [np.zeros(out_len, dtype=npdt) for _ in range(nranks)]
                    return execute(runs, sends, recvs, nranks, orc.SUM, size, sp, rp)

                got = run(mr.Collective.ALL_TO_ALL, ins, nranks * length, length)
                want = orc.ucx_all_to_all(ins, dtype)
                assert all(bits_equal(got[r], want[r]) for r in range(nranks))
                parts = [x[:length].copy() for x in ins]
                got = run(mr.Collective.ALL_GATHER, parts, nranks * length, length)
                want = orc.ucx_all_gather(parts, dtype)
                assert all(bits_equal(got[r], want[r]) for r in range(nranks))
                root = nranks - 1
                got = run(mr.Collective.SCATTER, ins, length, length, root)
                want = orc.ucx_scatter([ins[root] if r == root else None for r in range(nranks)], dtype, root)
                assert all(bits_equal(got[r], want[r]) for r in range(nranks))
                got = run(mr.Collective.GATHER, parts, nranks * length, length, root)
                assert bits_equal(got[root], orc.ucx_gather(parts, dtype, root)[root])
                got = run(mr.Collective.BROADCAST, parts, length, length, root)
                assert all(bits_equal(got[r], parts[root]) for r in range(nranks))


@pytest.mark.parametrize("dtype", [orc.INT8, orc.INT32, orc.FLOAT32, orc.FLOAT64, orc.UINT64])
@pytest.mark.parametrize("nranks", [1, 2, 3, 4, 5, 8, 13, 16])
def test_reduce_plans(dtype, nranks):
    """reduce to a root: the ucx order is the binomial tree of src/ucx/reduce.cpp, checked against the
    oracle's literal replay of it."""
    rng = np.random.default_rng(dtype * 31 + nranks)
    size = orc.dtype_size(dtype)
    for length in (0, 1, 5, 300, 1031):
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        for misalign in (False, True):
            offs = [size * (r % 3) for r in range(nranks)] if misalign else [0] * nranks
            sp, rp = fake_ptrs(SEND_BASE, nranks, offs), fake_ptrs(RECV_BASE, nranks, offs)
            for root in sorted({0, nranks // 2, nranks - 1}):
                for op in (orc.SUM, orc.MAX, orc.MIN):
                    runs, br, bw = mr.describe(mr.Collective.REDUCE, sp, rp, length, dtype, orc.ORDER_UCX, root=root)
                    recvs = [np.zeros(length, dtype=ins[0].dtype) for _ in range(nranks)]
                    got = execute(runs, ins, recvs, nranks, op, size, sp, rp)
                    want = orc.ucx_reduce(ins, dtype, op, root)
                    assert bits_equal(got[root], want[root]), (dtype, nranks, length, root, op)
                    assert (br, bw) == ((nranks * length * size, length * size) if length else (0, 0))
                    for order in (orc.ORDER_SHM, orc.ORDER_RANK0):
                        runs, _, _ = mr.describe(mr.Collective.REDUCE, sp, rp, length, dtype, order, root=root)
                        recvs = [np.zeros(length, dtype=ins[0].dtype) for _ in range(nranks)]
                        got = execute(runs, ins, recvs, nranks, op, size, sp, rp)
                        assert bits_equal(got[root], orc.fold_all_reduce(ins, dtype, op, order)[root])


def test_two_input_reduce_plan_keeps_i1_on_ties():
    # src/ucx/kernel.cu:24-38: (i0 > i1) ? i0 : i1
    a = np.array([0.0, -0.0, np.nan, 1.0, 5.0], dtype=np.float32)
    b = np.array([-0.0, 0.0, 1.0, np.nan, 2.0], dtype=np.float32)
    sp = [SEND_BASE, SEND_BASE + STRIDE]
    rp = [RECV_BASE]
    for op in (orc.MAX, orc.MIN, orc.SUM):
        runs, br, bw = mr.describe(mr.Collective.REDUCE2, sp, rp, a.size, orc.FLOAT32, nranks=2)
        got = execute(runs, [a, b], [np.zeros_like(a), np.zeros_like(a)], 2, op, 4, sp, rp + [0])[0]
        want = orc.reduce_ucx(a, b, orc.FLOAT32, op)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan) and bits_equal(got[~nan], want[~nan])
        assert (br, bw) == (2 * a.size * 4, a.size * 4)


def test_full_size_plan_shapes():
    """The headline shape: 8 ranks x 2^28 fp32 is one launch of 8 vector runs, 65536 x 1 KiB-per-wave
    tiles... and every planned byte is accounted for."""
    n = 1 << 28
    sp, rp = fake_ptrs(SEND_BASE, 8, [0] * 8), fake_ptrs(RECV_BASE, 8, [0] * 8)
    runs, br, bw = mr.describe(mr.Collective.ALL_REDUCE, sp, rp, n, orc.FLOAT32)
    assert len(runs) == 8 and all(r["vector"] == 2 and r["nfold"] == 8 and r["nout"] == 8 for r in runs)
    assert sum(r["tiles"] for r in runs) == n * 4 // 1024
    assert sum(r["count"] for r in runs) == n
    assert br == bw == 8 * n * 4
    assert all(r["waves"] == 4 for r in runs)  # the group form: four wavefronts, four tiles per workgroup
    # so do reduce_scatter and tree launches of 2560 to 8191 tiles per buffer; short launches keep one wavefront per tile
    rs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, sp, rp, 1 << 17, orc.FLOAT32)
    assert rs and all(r["waves"] == 4 and r["vector"] == 2 for r in rs)
    tree, _, _ = mr.describe(mr.Collective.REDUCE, sp, rp, 1 << 20, orc.FLOAT32, root=3)
    assert tree and all(r["waves"] == 4 and r["dir"] == 0 for r in tree)
    # from 8192 tiles on, folds of three or more inputs into ONE output go back to one wavefront per tile (launched
    # at a reduced occupancy); two inputs stay in the group form
    rs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, sp, rp, 1 << 22, orc.FLOAT32)
    assert rs and all(r["waves"] == 1 and r["vector"] == 2 for r in rs)
    tree, _, _ = mr.describe(mr.Collective.REDUCE, sp, rp, 1 << 22, orc.FLOAT32, root=3)
    assert tree and all(r["waves"] == 1 and r["dir"] == 0 for r in tree)
    two_phase, _, _ = mr.describe(mr.Collective.ALL_REDUCE, sp, rp, 1 << 24, orc.FLOAT32, schedule=mr.Schedule.TWO_PHASE)
    assert {r["waves"] for r in two_phase if r["step"] == 0 and r["nfold"] == 8} == {1}
    shifted, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, sp, rp, (1 << 22) - 4, orc.FLOAT32)  # outputs off the lines
    assert shifted and all(r["waves"] == 1 and r["vector"] == 2 for r in shifted)
    off = [p + 16 for p in sp]  # inputs off the lines: the group form, which deals workgroups to XCDs
    moved, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, off, [p + 16 for p in rp], 1 << 22, orc.FLOAT32)
    assert moved and all(r["waves"] == 4 and r["deal"] == 1 for r in moved)
    pair, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, sp[:2], rp[:2], 1 << 24, orc.FLOAT32, nranks=2)
    assert pair and all(r["waves"] == 4 for r in pair)
    # the group form starts the later the fewer the ranks (a tile is 256 fp32 elements)
    for ranks, first in ((8, 2560), (4, 6400), (3, 10752), (2, 15360)):
        for tiles, waves in ((first - 1, 1), (first, 4)):
            ar, _, _ = mr.describe(mr.Collective.ALL_REDUCE, sp[:ranks], rp[:ranks], tiles * 256, orc.FLOAT32, nranks=ranks)
            assert ar and all(r["waves"] == waves for r in ar), (ranks, tiles)
    # four ranks stay in the group form up to 65535 tiles per buffer
    for recvlen, waves in ((1 << 21, 4), ((1 << 22) - 256, 4), (1 << 22, 1), (1 << 24, 1)):
        four, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, sp[:4], rp[:4], recvlen, orc.FLOAT32, nranks=4)
        assert four and all(r["waves"] == waves for r in four), recvlen
    for coll, count in ((mr.Collective.ALL_REDUCE, 1 << 15), (mr.Collective.REDUCE_SCATTER, 1 << 12),
                        (mr.Collective.REDUCE, 1 << 15)):
        small, _, _ = mr.describe(coll, sp, rp, count, orc.FLOAT32)
        assert small and all(r["waves"] == 1 for r in small)
    # a buffer far beyond one launch's grid is split into several launches, nothing lost
    big = 1 << 41
    runs, br, bw = mr.describe(mr.Collective.ALL_REDUCE, [SEND_BASE, SEND_BASE + (1 << 42)],
                               [RECV_BASE, RECV_BASE + (1 << 42)], big, orc.INT8)
    assert sum(r["count"] for r in runs) == big and len({r["step"] for r in runs}) >= 1
    assert all(r["tiles"] <= 0x7fffffff for r in runs)


def test_planner_rejects_what_it_cannot_honour():
    sp, rp = fake_ptrs(SEND_BASE, 4, [0] * 4), fake_ptrs(RECV_BASE, 4, [0] * 4)
    with pytest.raises(mr.MegRayError, match="ring schedule"):
        mr.describe(mr.Collective.ALL_REDUCE, sp, rp, 100, orc.FLOAT32, orc.ORDER_SHM, mr.Schedule.RING)
    with pytest.raises(mr.MegRayError, match="overlap"):
        mr.describe(mr.Collective.ALL_REDUCE, sp, [sp[1], rp[1], rp[2], rp[3]], 100, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="overlap"):
        mr.describe(mr.Collective.ALL_REDUCE, sp, [rp[0], rp[0] + 8, rp[2], rp[3]], 100, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="in place"):
        mr.describe(mr.Collective.ALL_TO_ALL, sp, sp, 100, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="unknown dtype"):
        mr.describe(mr.Collective.ALL_REDUCE, sp, rp, 100, orc.CHAR)
    with pytest.raises(mr.MegRayError, match="root"):
        mr.describe(mr.Collective.SCATTER, sp, rp, 100, orc.FLOAT32, root=4)
    # a null buffer would fault on the device; a zero-length call touches nothing and may pass them
    with pytest.raises(mr.MegRayError, match="send buffer is null"):
        mr.describe(mr.Collective.ALL_REDUCE, [sp[0], 0, sp[2], sp[3]], rp, 100, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="receive buffer is null"):
        mr.describe(mr.Collective.ALL_GATHER, sp, [rp[0], rp[1], 0, rp[3]], 100, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="root's send buffer is null"):
        mr.describe(mr.Collective.BROADCAST, [0, 0, 0, 0], rp, 100, orc.FLOAT32, root=2)
    mr.describe(mr.Collective.ALL_REDUCE, [0] * 4, [0] * 4, 0, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="beyond 2.48 elements"):
        mr.describe(mr.Collective.ALL_REDUCE, sp, rp, 1 << 50, orc.INT8)
    # in place is fine where every element keeps its address
    mr.describe(mr.Collective.ALL_REDUCE, sp, sp, 100, orc.FLOAT32)
    mr.describe(mr.Collective.REDUCE_SCATTER, sp, [sp[r] + r * 400 for r in range(4)], 100, orc.FLOAT32)
    mr.describe(mr.Collective.ALL_GATHER, [rp[r] + r * 400 for r in range(4)], rp, 100, orc.FLOAT32)
    with pytest.raises(mr.MegRayError, match="out of place"):
        mr.describe(mr.Collective.REDUCE_SCATTER, sp, sp, 100, orc.FLOAT32)


def test_group_form_tile_mapping_covers_every_tile_once():
    """The group kernels map workgroup b to the tiles first + k * 32 (k = 0..3), first = (b // 32) * 128 + b % 32,
    over a grid of ceil(tiles / 128) * 32 workgroups (kGroupWaves = 4, kGroupStride = 32 in vrank_types.h).
    Restated here: every tile below the rounded-up count is owned by exactly one (workgroup, wavefront), so
    with the kernels' own "tile inside the buffer" checks nothing is skipped and nothing is touched twice."""
    waves, stride = 4, 32
    for tiles in (1, 31, 32, 127, 128, 129, 512, 1000, 4097, 65536 + 5):
        grid = (tiles + waves * stride - 1) // (waves * stride) * stride
        owned = np.zeros(grid * waves, dtype=np.int32)
        b = np.arange(grid)
        first = (b // stride) * (waves * stride) + b % stride
        for k in range(waves):
            np.add.at(owned, first + k * stride, 1)
        assert owned.size >= tiles and owned.size - tiles < waves * stride
        assert (owned == 1).all(), f"tiles={tiles}"
    # the planner's grid for a described launch agrees: 2^20 tiles -> 2^18 workgroups of 4 wavefronts
    sp, rp = fake_ptrs(SEND_BASE, 8, [0] * 8), fake_ptrs(RECV_BASE, 8, [0] * 8)
    runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, sp, rp, 1 << 28, orc.FLOAT32)
    assert sum(r["tiles"] for r in runs) == 1 << 20 and all(r["waves"] == 4 for r in runs)


def test_blocks_too_long_for_one_grid_are_cut_into_several_pack_launches():
    """A grid holds 2^31 - 1 workgroups.  16 ranks' all_to_all is 256 block copies; a workgroup of the group form
    takes 4 KiB of a block whatever the buffers' alignment, so a block beyond 32 GiB no longer fits one launch and
    is cut into slices, one launch each, that cover every block exactly once.  Pointers are synthetic: describe()
    never dereferences them."""
    nranks = 16
    block = 40 * 2 ** 30 + 3  # bytes; odd, and the buffers sit at odd addresses: width 1
    sp = fake_ptrs(1 << 44, nranks, [1] * nranks, stride=1 << 40)
    rp = fake_ptrs(1 << 46, nranks, [1] * nranks, stride=1 << 40)
    runs, bytes_read, bytes_written = mr.describe(mr.Collective.ALL_TO_ALL, sp, rp, block, mr.DType.UINT8)
    assert bytes_read == bytes_written == nranks * nranks * block
    steps = sorted({r["step"] for r in runs})
    assert len(steps) >= 2, "one launch cannot hold 256 x 40 GiB / 4 KiB workgroups"
    for step in steps:
        launch = [r for r in runs if r["step"] == step]
        assert len(launch) == nranks * nranks
        assert all(r["vector"] == 1 and r["waves"] == 4 for r in launch)
        assert sum(-(-r["tiles"] // 4) for r in launch) <= 2 ** 31 - 1  # a workgroup of four wavefronts takes four tiles
    # per copy (source rank, source block): the slices tile [0, block) in order
    for src in range(nranks):
        for dst in range(nranks):
            mine = sorted((r for r in runs if r["start"] == src and r["out_first"] == dst), key=lambda r: r["in_begin"])
            pos = 0
            for r in mine:
                assert r["in_begin"] == dst * block + pos and r["out_begin"] == src * block + pos
                pos += r["count"]
            assert pos == block
    # the group form (16-byte accesses) is cut on whole groups of workgroups
    sp = fake_ptrs(1 << 44, nranks, [0] * nranks, stride=1 << 40)
    rp = fake_ptrs(1 << 46, nranks, [0] * nranks, stride=1 << 40)
    block = 40 * 2 ** 30  # 40 GiB blocks: 256 copies x 2.6 M workgroups
    runs, _, _ = mr.describe(mr.Collective.ALL_TO_ALL, sp, rp, block, mr.DType.UINT8)
    steps = sorted({r["step"] for r in runs})
    assert len(steps) >= 2 and all(r["waves"] == 4 and r["vector"] == 16 for r in runs)
    first = sorted((r for r in runs if r["start"] == 0 and r["out_first"] == 0), key=lambda r: r["in_begin"])
    assert sum(r["count"] for r in first) == block
    assert all(r["in_begin"] % (128 * 1024) == 0 for r in first)


def test_runs_whose_tiles_share_cache_lines_are_dealt_to_xcds():
    """Consecutive workgroups run on different XCDs, each with an L2 of its own.  Where tiles do not sit on the
    cache lines of every buffer, a line is shared by two tiles, and the planner asks the group kernels to deal runs
    of workgroups to one XCD each; tiles on line boundaries keep the plain order."""
    nranks = 8
    send = fake_ptrs(1 << 44, nranks, [0] * nranks, stride=1 << 40)
    recv = fake_ptrs(1 << 46, nranks, [0] * nranks, stride=1 << 40)
    big = 1 << 24

    def vector_runs(*args, **kw):
        runs, _, _ = mr.describe(*args, **kw)
        return [r for r in runs if r["vector"] and r["waves"] == 4]

    # everything on 256-byte boundaries: plain order, flat and segment kernels
    runs = vector_runs(mr.Collective.ALL_REDUCE, send, recv, big, mr.DType.FLOAT32)
    assert runs and all(r["deal"] == 0 for r in runs)
    runs = vector_runs(mr.Collective.REDUCE_SCATTER, send, recv, (1 << 20) // nranks, mr.DType.FLOAT32)  # 4096 tiles
    assert runs and all(r["deal"] == 0 for r in runs)
    five_s, five_r = send[:5], recv[:5]
    runs = vector_runs(mr.Collective.ALL_REDUCE, five_s, five_r, 5 * (1 << 20), mr.DType.FLOAT32)
    assert runs and all(r["vector"] == 1 and r["deal"] == 0 for r in runs)
    # a receive length off the line grid shifts the outputs against the inputs
    # (the last case is a flat launch, kept below the size from which one-output folds leave the group form)
    for dtype, recvlen in ((mr.DType.FLOAT32, big // nranks - 1), (mr.DType.FLOAT16, big // nranks - 3),
                           (mr.DType.FLOAT32, (1 << 20) // nranks - 4)):
        runs = vector_runs(mr.Collective.REDUCE_SCATTER, send, recv, recvlen, dtype)
        dealt = [r for r in runs if r["out_first"] != 0]  # rank 0's block starts where its output does
        assert dealt and all(r["deal"] == 1 for r in dealt)
    # every input at its own offset: flat launch (4-byte elements) or segments (2-byte elements), dealt
    offs = [4 * (r % 3) for r in range(nranks)]
    runs = vector_runs(mr.Collective.ALL_REDUCE, fake_ptrs(1 << 44, nranks, offs, stride=1 << 40), recv, big, mr.DType.FLOAT32)
    assert runs and all(r["vector"] == 2 and r["deal"] == 1 for r in runs)
    offs = [2 * (r % 5) for r in range(nranks)]
    runs = vector_runs(mr.Collective.ALL_REDUCE, fake_ptrs(1 << 44, nranks, offs, stride=1 << 40), recv, big, mr.DType.FLOAT16)
    assert runs and all(r["vector"] == 1 and r["deal"] == 1 for r in runs)
    # a common offset of 16 bytes: flat tiles start at the buffers' first byte, off the lines
    offs = [16] * nranks
    runs = vector_runs(mr.Collective.ALL_REDUCE, fake_ptrs(1 << 44, nranks, offs, stride=1 << 40),
                       fake_ptrs(1 << 46, nranks, offs, stride=1 << 40), big, mr.DType.FLOAT32)
    assert runs and all(r["deal"] == 1 for r in runs)


def test_random_plans_keep_inside_the_buffers_under_host_sanitizers(tmp_path):
    """tests/cpp/plan_fuzz.cpp: the host planner (pure host code) built with the address and undefined-behaviour
    sanitizers and called with random collectives, rank counts, element sizes, lengths up to 2^33 elements and
    buffer offsets.  Every launch descriptor of every plan must keep the kernels inside the callers' buffers, the
    tile tables must add up, and the one-pass plans must write every output element exactly once."""
    import shutil
    import subprocess

    gxx = shutil.which("g++")
    if not gxx:
        pytest.skip("no host compiler")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    exe = str(tmp_path / "plan_fuzz")
    build = subprocess.run([gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined",
                            f"-I{root}/include", f"-I{root}/megray_amd/csrc", f"{root}/tests/cpp/plan_fuzz.cpp",
                            f"{root}/megray_amd/csrc/vrank_plan.cpp", "-o", exe], capture_output=True, text=True, timeout=300)
    assert build.returncode == 0, build.stderr
    for seed in ("11", "12"):
        run = subprocess.run([exe, "30000", seed], capture_output=True, text=True, timeout=300)
        assert run.returncode == 0 and run.stdout.startswith("ok "), run.stdout + run.stderr
