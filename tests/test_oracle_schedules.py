"""Pins the oracle's ring / tree replays and fold orders (no GPU).

Evidence used: the closed-form inputs and expectations the reference's own tests hold
(test/test_opr.cpp, cited per test), numpy on integers (order independent), a tracing reduce that
reveals the order operands meet in, and an independent numpy left fold for fp32.
"""
import numpy as np
import pytest

import oracle as orc

UCX_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.UINT64, orc.FLOAT32,
             orc.FLOAT64]
SHM_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.FLOAT32]
ALL_REDUCE_TYPES = UCX_TYPES + [orc.FLOAT16]


def rand_array(dtype, n, rng, wide=True):
    npdt = orc.NP_DTYPE[dtype]
    if np.issubdtype(npdt, np.integer):
        raw = rng.integers(0, 2 ** 64, size=n, dtype=np.uint64)
        return raw.astype(np.dtype(npdt).str.replace("i", "u")).view(npdt)
    if dtype == orc.FLOAT16:
        return (rng.standard_normal(n) * np.exp(rng.uniform(-6, 6, n))).astype(npdt)
    scale = np.exp(rng.uniform(-20, 20, n)) if wide else 1.0
    return (rng.standard_normal(n) * scale).astype(npdt)


# ----------------------------------------------------------------------------- reference KATs

def test_kat_all_reduce_n3_len10():
    # test/test_opr.cpp:286-359: in[i][j] = (i+1)(j+1), N=3, len=10
    n, length = 3, 10
    ins = [np.array([(i + 1) * (j + 1) for j in range(length)], dtype=np.float32) for i in range(n)]
    j1 = np.arange(1, length + 1, dtype=np.float32)
    want = {orc.SUM: 6 * j1, orc.MAX: 3 * j1, orc.MIN: 1 * j1}
    for op, expected in want.items():
        for outs in (orc.ucx_all_reduce(ins, orc.FLOAT32, op), orc.shm_all_reduce(ins, orc.FLOAT32, op),
                     orc.test_all_reduce_f32(ins, op),
                     orc.fold_all_reduce(ins, orc.FLOAT32, op, orc.ORDER_UCX),
                     orc.fold_all_reduce(ins, orc.FLOAT32, op, orc.ORDER_SHM),
                     orc.fold_all_reduce(ins, orc.FLOAT32, op, orc.ORDER_RANK0)):
            for out in outs:
                assert np.array_equal(out, expected)


def test_kat_reduce_scatter_n3_recvlen10():
    # test/test_opr.cpp:361-438: in[i][m] = (i+1)(m+1), out[k][j] over m = k*recvlen + j
    n, recvlen = 3, 10
    ins = [np.array([(i + 1) * (m + 1) for m in range(n * recvlen)], dtype=np.float32)
           for i in range(n)]
    for op, factor in ((orc.SUM, 6), (orc.MAX, 3), (orc.MIN, 1)):
        for outs in (orc.ucx_reduce_scatter(ins, orc.FLOAT32, op),
                     orc.shm_reduce_scatter(ins, orc.FLOAT32, op),
                     orc.test_reduce_scatter_f32(ins, op),
                     orc.fold_reduce_scatter(ins, orc.FLOAT32, op, orc.ORDER_UCX),
                     orc.fold_reduce_scatter(ins, orc.FLOAT32, op, orc.ORDER_SHM)):
            for k in range(n):
                want = np.array([factor * (k * recvlen + j + 1) for j in range(recvlen)],
                                dtype=np.float32)
                assert np.array_equal(outs[k], want)


def test_kat_all_gather():
    # test/test_opr.cpp:243-257: out[k][i*sendlen + j] = in[i][j] = (i+1)(j+1)
    n, sendlen = 3, 10
    ins = [np.array([(i + 1) * (j + 1) for j in range(sendlen)], dtype=np.float32) for i in range(n)]
    want = np.concatenate(ins)
    for outs in (orc.ucx_all_gather(ins, orc.FLOAT32), orc.shm_all_gather(ins, orc.FLOAT32)):
        for out in outs:
            assert np.array_equal(out, want)


def test_kat_all_to_all():
    # test/test_opr.cpp:198-214: in[i][j*len+k] = (i+1)(j+2)(k+3) -> out[j][i*len+k]
    n, length = 3, 6
    ins = [np.array([(i + 1) * (j + 2) * (k + 3) for j in range(n) for k in range(length)],
                    dtype=np.float32) for i in range(n)]
    for outs in (orc.ucx_all_to_all(ins, orc.FLOAT32), orc.shm_all_to_all(ins, orc.FLOAT32)):
        for j in range(n):
            want = np.array([(i + 1) * (j + 2) * (k + 3) for i in range(n) for k in range(length)],
                            dtype=np.float32)
            assert np.array_equal(outs[j], want)


def test_kat_scatter_gather_root1():
    n, length, root = 3, 10, 1
    # test/test_opr.cpp:101-114: root holds (i+1)(j+2) for block i; rank i receives block i
    root_in = np.array([(i + 1) * (j + 2) for i in range(n) for j in range(length)], dtype=np.float32)
    sends = [root_in if r == root else None for r in range(n)]
    outs = orc.ucx_scatter(sends, orc.FLOAT32, root)
    for i in range(n):
        assert np.array_equal(outs[i], np.array([(i + 1) * (j + 2) for j in range(length)], np.float32))
    # test/test_opr.cpp:148-161: the inverse
    ins = [np.array([(i + 1) * (j + 2) for j in range(length)], dtype=np.float32) for i in range(n)]
    outs = orc.ucx_gather(ins, orc.FLOAT32, root)
    assert np.array_equal(outs[root], root_in)


def test_kat_broadcast_and_reduce_root1():
    n, length, root = 3, 10, 1
    ins = [np.array([(i + 1) * (j + 1) for j in range(length)], dtype=np.float32) for i in range(n)]
    # test/test_opr.cpp:440-452
    for out in orc.ucx_broadcast(ins, orc.FLOAT32, root):
        assert np.array_equal(out, ins[root])
    # test/test_opr.cpp:487-551
    j1 = np.arange(1, length + 1, dtype=np.float32)
    for op, expected in ((orc.SUM, 6 * j1), (orc.MAX, 3 * j1), (orc.MIN, j1)):
        assert np.array_equal(orc.ucx_reduce(ins, orc.FLOAT32, op, root)[root], expected)


# ----------------------------------------------------------------------------- integers: order free

@pytest.mark.parametrize("nranks", [1, 2, 3, 4, 5, 8, 9])
@pytest.mark.parametrize("dtype", [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.UINT64])
def test_integer_collectives_equal_numpy(nranks, dtype):
    rng = np.random.default_rng(100 * nranks + dtype)
    for length in (0, 1, nranks - 1, nranks, 2 * nranks + 1, 37, 64):
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        stack = np.stack(ins) if length else np.zeros((nranks, 0), dtype=ins[0].dtype)
        with np.errstate(over="ignore"):
            want = {orc.SUM: np.add.reduce(stack, axis=0, dtype=stack.dtype),
                    orc.MAX: stack.max(axis=0) if length else stack[0],
                    orc.MIN: stack.min(axis=0) if length else stack[0]}
        for op, expected in want.items():
            runs = [orc.ucx_all_reduce(ins, dtype, op),
                    orc.fold_all_reduce(ins, dtype, op, orc.ORDER_UCX),
                    orc.fold_all_reduce(ins, dtype, op, orc.ORDER_SHM),
                    orc.fold_all_reduce(ins, dtype, op, orc.ORDER_RANK0),
                    [orc.ucx_reduce(ins, dtype, op, root=nranks // 2)[nranks // 2]]]
            if dtype in SHM_TYPES:
                runs.append(orc.shm_all_reduce(ins, dtype, op))
            for outs in runs:
                for out in outs:
                    assert np.array_equal(out, expected)


# ----------------------------------------------------------------------------- fold orders by tracing

def digits(value):
    out = []
    while value:
        out.append((value & 0xF) - 1)
        value >>= 4
    return out[::-1]  # most significant digit first = leftmost operand of the concatenation


def expected_orders(nranks):
    """The orders stated by reading the reference loops, written out independently here."""
    n = nranks
    return {
        # chunk c: x_c, x_{c+1}, ..., x_{c-1}; each step is reduce(i0=new, i1=acc)
        "ucx_ar": {c: [(c + j) % n for j in range(n)] for c in range(n)},
        # chunk c: x_{c+1}, ..., x_c; each step is reduce(i0=acc, i1=new)
        "ucx_rs": {c: [(c + 1 + j) % n for j in range(n)] for c in range(n)},
        # chunk w of 2N, owner w//2: x_o, x_{o-1}, ..., x_{o+1}; cpu_reduce(a=acc, b=new)
        "shm": {w: [(w // 2 - j) % n for j in range(n)] for w in range(2 * n)},
    }


@pytest.mark.parametrize("nranks", [1, 2, 3, 4, 5, 7, 8, 9, 15])
def test_fold_orders_match_traced_replays(nranks):
    n = nranks
    want = expected_orders(n)
    for length in (n, 2 * n, 4 * n + 3, 2 * n + 1):
        ins = [np.full(length, r + 1, dtype=np.uint64) for r in range(n)]
        # --- ucx all_reduce
        outs = orc.ucx_all_reduce(ins, orc.UINT64, orc.SUM, trace=True)
        sizes, offs = orc.chunk_partition(length, n)
        for c in range(n):
            ranks, new_wins, nchunks = orc.fold_order(orc.COLL_ALL_REDUCE, orc.ORDER_UCX, n, c)
            assert ranks == want["ucx_ar"][c] and nchunks == n and not new_wins
            for e in range(offs[c], offs[c] + sizes[c]):
                for out in outs:  # every rank holds the same trace
                    # concat(i0=new, i1=acc): the string reads newest first
                    assert digits(int(out[e])) == ranks[::-1]
        # --- shm all_reduce (2N chunks)
        outs = orc.shm_all_reduce(ins, orc.UINT64, orc.SUM, trace=True)
        sizes, offs = orc.chunk_partition(length, 2 * n)
        for w in range(2 * n):
            ranks, new_wins, nchunks = orc.fold_order(orc.COLL_ALL_REDUCE, orc.ORDER_SHM, n, w)
            assert ranks == want["shm"][w] and nchunks == 2 * n and not new_wins
            for e in range(offs[w], offs[w] + sizes[w]):
                for out in outs:
                    assert digits(int(out[e])) == ranks  # concat(acc, new)
    for recvlen in (1, 2, 5):
        ins = [np.full(n * recvlen, r + 1, dtype=np.uint64) for r in range(n)]
        outs = orc.ucx_reduce_scatter(ins, orc.UINT64, orc.SUM, trace=True)
        for c in range(n):
            ranks, new_wins, nchunks = orc.fold_order(orc.COLL_REDUCE_SCATTER, orc.ORDER_UCX, n, c)
            assert ranks == want["ucx_rs"][c] and nchunks == n
            assert new_wins == (True)
            for e in range(recvlen):
                assert digits(int(outs[c][e])) == ranks  # concat(i0=acc, i1=new)
        outs = orc.shm_reduce_scatter(ins, orc.UINT64, orc.SUM, trace=True)
        sizes, offs = orc.chunk_partition(n * recvlen, 2 * n)
        for w in range(2 * n):
            ranks, _, _ = orc.fold_order(orc.COLL_REDUCE_SCATTER, orc.ORDER_SHM, n, w)
            assert ranks == want["shm"][w]
            for e in range(offs[w], offs[w] + sizes[w]):
                assert digits(int(outs[e // recvlen][e % recvlen])) == ranks
    ranks, new_wins, nchunks = orc.fold_order(orc.COLL_ALL_REDUCE, orc.ORDER_RANK0, n, 0)
    assert ranks == list(range(n)) and nchunks == 1 and not new_wins


def test_tree_reduce_trace_root_and_shape():
    # src/ucx/reduce.cpp:56-80: round i merges virtual rank v^bit into v as reduce(incoming, own)
    for n in (1, 2, 3, 4, 5, 8):
        for root in range(n):
            ins = [np.full(3, r + 1, dtype=np.uint64) for r in range(n)]
            out = orc.ucx_reduce(ins, orc.UINT64, orc.SUM, root, trace=True)[root]

            def tree(v, bit_limit):
                # string held by virtual rank v after all rounds below bit_limit
                s = [(v + root) % n]
                bit = 1
                while bit < bit_limit:
                    if v & bit:
                        break
                    if (v ^ bit) < n:
                        s = tree(v ^ bit, bit) + s  # concat(i0=incoming, i1=own)
                    bit <<= 1
                return s

            top = 1
            while top < n:
                top <<= 1
            assert digits(int(out[0])) == tree(0, top)
            assert sorted(digits(int(out[0]))) == list(range(n))


# ----------------------------------------------------------------------------- float folds

def numpy_left_fold(ins, ranks, op, new_wins, acc_dtype=None):
    """Independent restatement: a left fold over `ranks` with numpy's IEEE scalar ops."""
    acc = ins[ranks[0]].astype(acc_dtype or ins[0].dtype)
    for r in ranks[1:]:
        x = ins[r].astype(acc.dtype)
        if op == orc.SUM:
            acc = acc + x
        elif op == orc.MAX:
            acc = np.where(acc > x, acc, x) if new_wins else np.where(x > acc, x, acc)
        else:
            acc = np.where(acc < x, acc, x) if new_wins else np.where(x < acc, x, acc)
    return acc


def bits_equal(a, b):
    return np.array_equal(np.ascontiguousarray(a).view(np.uint8), np.ascontiguousarray(b).view(np.uint8))


@pytest.mark.parametrize("nranks", [2, 3, 4, 8])
@pytest.mark.parametrize("dtype", [orc.FLOAT32, orc.FLOAT64])
def test_float_all_reduce_orders(nranks, dtype):
    rng = np.random.default_rng(nranks * 10 + dtype)
    n = nranks
    for length in (n * 64 + 5, 3, 1000):
        ins = [rand_array(dtype, length, rng) for _ in range(n)]
        for op in (orc.SUM, orc.MAX, orc.MIN):
            lit = orc.ucx_all_reduce(ins, dtype, op)
            fold = orc.fold_all_reduce(ins, dtype, op, orc.ORDER_UCX)
            sizes, offs = orc.chunk_partition(length, n)
            for c in range(n):
                ranks, new_wins, _ = orc.fold_order(orc.COLL_ALL_REDUCE, orc.ORDER_UCX, n, c)
                sl = slice(offs[c], offs[c] + sizes[c])
                want = numpy_left_fold([x[sl] for x in ins], ranks, op, new_wins)
                for r in range(n):
                    assert bits_equal(lit[r][sl], want)
                    assert bits_equal(fold[r][sl], want)
            if dtype in SHM_TYPES:
                lit = orc.shm_all_reduce(ins, dtype, op)
                fold = orc.fold_all_reduce(ins, dtype, op, orc.ORDER_SHM)
                sizes, offs = orc.chunk_partition(length, 2 * n)
                for w in range(2 * n):
                    ranks, new_wins, _ = orc.fold_order(orc.COLL_ALL_REDUCE, orc.ORDER_SHM, n, w)
                    sl = slice(offs[w], offs[w] + sizes[w])
                    want = numpy_left_fold([x[sl] for x in ins], ranks, op, new_wins)
                    for r in range(n):
                        assert bits_equal(lit[r][sl], want)
                        assert bits_equal(fold[r][sl], want)
            if dtype == orc.FLOAT32 and op == orc.SUM:
                t = orc.test_all_reduce_f32(ins, op)
                f0 = orc.fold_all_reduce(ins, dtype, op, orc.ORDER_RANK0)
                want = numpy_left_fold(ins, list(range(n)), op, False)
                for r in range(n):
                    assert bits_equal(t[r], want) and bits_equal(f0[r], want)
                mt = orc.test_all_reduce_f32(ins, op, nthreads=3)
                assert all(bits_equal(mt[r], want) for r in range(n))


def test_orders_differ_on_general_fp32():
    """The data used above can tell the orders apart (otherwise those checks would pin nothing)."""
    rng = np.random.default_rng(5)
    ins = [rand_array(orc.FLOAT32, 4096, rng) for _ in range(8)]
    a = orc.fold_all_reduce(ins, orc.FLOAT32, orc.SUM, orc.ORDER_UCX)[0]
    b = orc.fold_all_reduce(ins, orc.FLOAT32, orc.SUM, orc.ORDER_SHM)[0]
    c = orc.fold_all_reduce(ins, orc.FLOAT32, orc.SUM, orc.ORDER_RANK0)[0]
    assert (a != b).mean() > 0.05 and (a != c).mean() > 0.05 and (b != c).mean() > 0.05
    # chunk 0 of the UCX order IS the rank-0 order
    assert bits_equal(a[:512], c[:512])


@pytest.mark.parametrize("nranks", [2, 3, 8])
@pytest.mark.parametrize("dtype", [orc.FLOAT32, orc.FLOAT64])
def test_float_reduce_scatter_orders(nranks, dtype):
    rng = np.random.default_rng(nranks * 7 + dtype)
    n = nranks
    for recvlen in (1, 17, 256):
        ins = [rand_array(dtype, n * recvlen, rng) for _ in range(n)]
        for op in (orc.SUM, orc.MAX, orc.MIN):
            lit = orc.ucx_reduce_scatter(ins, dtype, op)
            fold = orc.fold_reduce_scatter(ins, dtype, op, orc.ORDER_UCX)
            for c in range(n):
                ranks, new_wins, _ = orc.fold_order(orc.COLL_REDUCE_SCATTER, orc.ORDER_UCX, n, c)
                sl = slice(c * recvlen, (c + 1) * recvlen)
                want = numpy_left_fold([x[sl] for x in ins], ranks, op, new_wins)
                assert bits_equal(lit[c], want) and bits_equal(fold[c], want)
            if dtype in SHM_TYPES:
                lit = orc.shm_reduce_scatter(ins, dtype, op)
                fold = orc.fold_reduce_scatter(ins, dtype, op, orc.ORDER_SHM)
                for c in range(n):
                    assert bits_equal(lit[c], fold[c])


def test_minmax_tie_convention_shows_in_the_fold():
    """+0/-0 ties and NaNs: the UCX all_reduce and SHM folds keep the accumulator, the UCX
    reduce_scatter fold keeps the newcomer (src/ucx/all_reduce.cpp:74-76 vs reduce_scatter.cpp:50-51)."""
    n = 4
    pz, nz = np.float32(0.0), np.float32(-0.0)
    ins = [np.full(n * 2, pz if r % 2 == 0 else nz, dtype=np.float32) for r in range(n)]
    for op in (orc.MAX, orc.MIN):
        ar = orc.ucx_all_reduce(ins, orc.FLOAT32, op)[0]
        rs = orc.ucx_reduce_scatter(ins, orc.FLOAT32, op)
        sh = orc.shm_all_reduce(ins, orc.FLOAT32, op)[0]
        for c in range(n):
            seed_ar = ins[c][0]                 # accumulator survives: the chunk's first rank
            last_rs = ins[c][0]                 # newcomer survives: the chunk's last rank = c
            assert np.signbit(ar[2 * c]) == np.signbit(seed_ar)
            assert np.signbit(rs[c][0]) == np.signbit(last_rs)
        for w in range(2 * n):
            assert np.signbit(sh[w]) == np.signbit(ins[w // 2][0])
    # NaN in the seed sticks, NaN in a later operand is dropped (all_reduce convention)
    ins = [np.ones(n, dtype=np.float32) * (r + 1) for r in range(n)]
    ins[1][1] = np.nan  # chunk 1 is seeded by rank 1; chunk 0 meets rank 1 second
    ins[1][0] = np.nan
    out = orc.ucx_all_reduce(ins, orc.FLOAT32, orc.MAX)[0]
    assert np.isnan(out[1]) and out[0] == 4.0
    assert bits_equal(out, orc.fold_all_reduce(ins, orc.FLOAT32, orc.MAX, orc.ORDER_UCX)[0])


@pytest.mark.parametrize("dtype", ALL_REDUCE_TYPES)
def test_fold_equals_literal_replay_all_dtypes(dtype):
    rng = np.random.default_rng(dtype + 40)
    for n in (2, 3, 5, 8):
        for length in (n - 1, 3 * n + 2, 129):
            ins = [rand_array(dtype, length, rng) for _ in range(n)]
            for op in (orc.SUM, orc.MAX, orc.MIN):
                if dtype == orc.FLOAT16:
                    with pytest.raises(NotImplementedError):  # src/ucx/kernel.cu:95-96
                        orc.ucx_all_reduce(ins, dtype, op)
                    continue
                lit = orc.ucx_all_reduce(ins, dtype, op)
                fold = orc.fold_all_reduce(ins, dtype, op, orc.ORDER_UCX)
                assert all(bits_equal(lit[r], fold[r]) for r in range(n))
                if dtype in SHM_TYPES:
                    lit = orc.shm_all_reduce(ins, dtype, op)
                    fold = orc.fold_all_reduce(ins, dtype, op, orc.ORDER_SHM)
                    assert all(bits_equal(lit[r], fold[r]) for r in range(n))


def test_fp16_fold_is_fp32_accumulate_one_rounding():
    """FLOAT16 has no reference reduce; the definition is checked against numpy: fold in fp32 in the
    chunk's order, round once (and it differs from rounding at every step on this data)."""
    rng = np.random.default_rng(16)
    n, length = 8, 8 * 300 + 3
    ins = [rand_array(orc.FLOAT16, length, rng) for _ in range(n)]
    got = orc.fold_all_reduce(ins, orc.FLOAT16, orc.SUM, orc.ORDER_UCX)
    sizes, offs = orc.chunk_partition(length, n)
    stepwise_differs = 0
    for c in range(n):
        ranks, new_wins, _ = orc.fold_order(orc.COLL_ALL_REDUCE, orc.ORDER_UCX, n, c)
        sl = slice(offs[c], offs[c] + sizes[c])
        with np.errstate(over="ignore"):
            want = numpy_left_fold([x[sl] for x in ins], ranks, orc.SUM, new_wins,
                                   acc_dtype=np.float32).astype(np.float16)
            step = numpy_left_fold([x[sl] for x in ins], ranks, orc.SUM, new_wins)
        for r in range(n):
            assert bits_equal(got[r][sl], want)
        stepwise_differs += int((step.view(np.uint16) != want.view(np.uint16)).sum())
    assert stepwise_differs > 0
    for op in (orc.MAX, orc.MIN):
        got = orc.fold_all_reduce(ins, orc.FLOAT16, op, orc.ORDER_UCX)[0]
        stack = np.stack(ins)
        want = stack.max(axis=0) if op == orc.MAX else stack.min(axis=0)
        assert np.array_equal(got, want)


# ----------------------------------------------------------------------------- permutations & misc

@pytest.mark.parametrize("nranks", [1, 2, 3, 8])
def test_permutation_identities(nranks):
    rng = np.random.default_rng(nranks)
    n = nranks
    for dtype in (orc.UINT8, orc.FLOAT16, orc.INT32, orc.FLOAT64, orc.CHAR):
        for length in (0, 1, 5, 16):
            ins = [rand_array(dtype if dtype != orc.CHAR else orc.UINT8, n * length, rng)
                   for _ in range(n)]
            once = orc.ucx_all_to_all(ins, dtype)
            twice = orc.ucx_all_to_all(once, dtype)
            assert all(bits_equal(twice[r], ins[r]) for r in range(n))
            assert all(bits_equal(a, b) for a, b in zip(once, orc.shm_all_to_all(ins, dtype)))
            for root in range(n):
                parts = orc.ucx_scatter([ins[root] if r == root else None for r in range(n)], dtype, root)
                gathered = orc.ucx_all_gather(parts, dtype)
                assert all(bits_equal(g, ins[root]) for g in gathered)
                assert bits_equal(orc.ucx_gather(parts, dtype, root)[root], ins[root])
                assert all(bits_equal(b, ins[root]) for b in orc.ucx_broadcast(ins, dtype, root))
            assert all(bits_equal(a, b) for a, b in
                       zip(orc.ucx_all_gather(ins, dtype), orc.shm_all_gather(ins, dtype)))


def test_in_place_all_reduce_replay():
    # src/ucx/all_reduce.cpp:44-45 degenerates to a self copy when sendbuff == recvbuff
    rng = np.random.default_rng(3)
    ins = [rand_array(orc.FLOAT32, 50, rng) for _ in range(4)]
    want = orc.ucx_all_reduce(ins, orc.FLOAT32, orc.SUM)
    work = [x.copy() for x in ins]
    got = orc.ucx_all_reduce(work, orc.FLOAT32, orc.SUM, inplace=True)
    assert all(bits_equal(got[r], want[r]) for r in range(4))


def test_reduce_scatter_then_all_gather_is_all_reduce_in_same_order():
    rng = np.random.default_rng(9)
    n, recvlen = 8, 33
    ins = [rand_array(orc.FLOAT32, n * recvlen, rng) for _ in range(n)]
    for order in (orc.ORDER_SHM, orc.ORDER_RANK0):
        rs = orc.fold_reduce_scatter(ins, orc.FLOAT32, orc.SUM, order)
        ag = orc.ucx_all_gather(rs, orc.FLOAT32)
        ar = orc.fold_all_reduce(ins, orc.FLOAT32, orc.SUM, order)
        assert all(bits_equal(ag[r], ar[r]) for r in range(n))


# ----------------------------------------------------------------------------- shm rooted collectives

@pytest.mark.parametrize("nranks", [1, 2, 3, 4, 5, 7, 8, 9, 15])
def test_shm_reduce_replay_has_the_shm_fold_order(nranks):
    """src/shm/reduce.cpp:21-100 replayed with its mutexes: the order the operands of every chunk meet in,
    read off a tracing reduce, is the 2N-chunk descending order of the shm all_reduce (owner w // 2 first,
    then w // 2 - 1, ...), the accumulator being cpu_reduce's first argument; only the root's buffer is
    written."""
    n = nranks
    want = expected_orders(n)["shm"]
    for length in (n, 2 * n, 4 * n + 3, 2 * n + 1, 1):
        ins = [np.full(length, r + 1, dtype=np.uint64) for r in range(n)]
        for root in sorted({0, n // 2, n - 1}):
            outs = orc.shm_reduce(ins, orc.UINT64, orc.SUM, root, trace=True)
            sizes, offs = orc.chunk_partition(length, 2 * n)
            for w in range(2 * n):
                for e in range(offs[w], offs[w] + sizes[w]):
                    assert digits(int(outs[root][e])) == want[w]  # concat(acc, new)
            for r in range(n):
                if r != root:
                    assert not outs[r].any()


def test_shm_reduce_replay_equals_the_chunk_fold_and_the_reference_vectors():
    rng = np.random.default_rng(77)
    for dtype in (orc.FLOAT32, orc.INT32, orc.UINT8, orc.INT64):
        for n in (2, 3, 8):
            for length in (10, 4 * n + 3, 1000):
                ins = [rand_array(dtype, length, rng) for _ in range(n)]
                for op in (orc.SUM, orc.MAX, orc.MIN):
                    root = n - 1
                    got = orc.shm_reduce(ins, dtype, op, root)[root]
                    fold = orc.fold_all_reduce(ins, dtype, op, orc.ORDER_SHM)[0]
                    assert np.array_equal(got.view(np.uint8), fold.view(np.uint8))
                    # independent statement: numpy left fold in the order expected_orders() writes out
                    sizes, offs = orc.chunk_partition(length, 2 * n)
                    want = np.empty_like(ins[0])
                    for w in range(2 * n):
                        sl = slice(offs[w], offs[w] + sizes[w])
                        order = expected_orders(n)["shm"][w]
                        acc = ins[order[0]][sl].copy()
                        for r in order[1:]:
                            with np.errstate(over="ignore"):
                                acc = {orc.SUM: lambda a, b: a + b, orc.MAX: np.maximum, orc.MIN: np.minimum}[op](acc, ins[r][sl])
                        want[sl] = acc
                    if np.issubdtype(ins[0].dtype, np.floating):
                        ok = np.array_equal(got, want, equal_nan=True)
                    else:
                        ok = np.array_equal(got, want)
                    assert ok, (dtype, n, length, op)
    # the reference's own vectors: test/test_opr.cpp:482-552 (ReduceSum, 3 ranks, root 1, in = (i+1)(j+1))
    n, length, root = 3, 10, 1
    ins = [np.array([(i + 1) * (j + 1) for j in range(length)], dtype=np.float32) for i in range(n)]
    assert np.array_equal(orc.shm_reduce(ins, orc.FLOAT32, orc.SUM, root)[root], 6.0 * np.arange(1, length + 1, dtype=np.float32))
    assert np.array_equal(orc.shm_reduce(ins, orc.FLOAT32, orc.MAX, root)[root], ins[2])
    assert np.array_equal(orc.shm_reduce(ins, orc.FLOAT32, orc.MIN, root)[root], ins[0])


def test_shm_broadcast_replay():
    # test/test_opr.cpp:440-480: 3 ranks, root 1, every rank ends up with the root's (i+1)(j+1)
    n, length, root = 3, 10, 1
    ins = [np.array([(i + 1) * (j + 1) for j in range(length)], dtype=np.float32) for i in range(n)]
    outs = orc.shm_broadcast([ins[r] if r == root else None for r in range(n)], orc.FLOAT32, root)
    for r in range(n):
        assert np.array_equal(outs[r], ins[root])
    rng = np.random.default_rng(5)
    for dtype in (orc.UINT8, orc.FLOAT16, orc.INT64):
        ins = [rand_array(dtype, 333, rng) for _ in range(5)]
        for root in range(5):
            a = orc.shm_broadcast(ins, dtype, root)
            b = orc.ucx_broadcast(ins, dtype, root)
            for r in range(5):
                assert np.array_equal(a[r].view(np.uint8), ins[root].view(np.uint8))
                assert np.array_equal(a[r].view(np.uint8), b[r].view(np.uint8))
