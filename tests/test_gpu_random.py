"""Randomised parity: collectives drawn at random (kind, element type, operation, fold order, rank
count, length, buffer offsets, in place or not) against the CPU oracle, bit for bit.  The seed is fixed,
so a failure names a reproducible case; lengths are drawn log-uniformly so that every kernel form
(element tiles, one wavefront per tile, group form; flat, general, pack) is hit."""
import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import Guarded, bits_equal, first_mismatch, rand_array, to_device, to_host  # noqa: E402

REDUCE_TYPES = [orc.INT8, orc.UINT8, orc.INT32, orc.UINT32, orc.INT64, orc.UINT64, orc.FLOAT16, orc.FLOAT32, orc.FLOAT64]
COPY_TYPES = REDUCE_TYPES + [orc.CHAR]


def same(got, want, what):
    assert bits_equal(got, want), f"{what}: first mismatch {first_mismatch(got, want)}"


_guards = []


def empty_device(nbytes, offset_bytes=0):
    """An output buffer between guard bytes, which the end of the case checks."""
    _guards.append(Guarded(nbytes, offset_bytes))
    return _guards[-1].view


def check_guards(what):
    for i, g in enumerate(_guards):
        assert g.intact(), f"{what}: output buffer {i} of the case was written outside its bounds"
    _guards.clear()


def draw_length(rng, nranks):
    bytes_ = int(np.exp(rng.uniform(np.log(1), np.log(2e7))))
    return max(0, bytes_ + int(rng.integers(-3, 4)))


def offsets_for(rng, nranks, size):
    mode = rng.integers(0, 5)
    if mode <= 1:
        return [0] * nranks                       # aligned
    if mode == 2:
        k = int(rng.integers(1, 16 // size + 1)) * size if size < 16 else 0
        return [k % 16] * nranks                  # one common offset from a 16-byte boundary
    if mode == 3:
        return [int(rng.integers(0, 16 // size)) * size for _ in range(nranks)]  # every buffer its own
    return [int(rng.integers(0, 2048 // size)) * size for _ in range(nranks)]   # ... anywhere on the 1 KiB tile grid


@pytest.mark.parametrize("seed", range(6))
def test_random_reductions(seed):
    rng = np.random.default_rng(5000 + seed)
    for case in range(100):
        dtype = REDUCE_TYPES[rng.integers(0, len(REDUCE_TYPES))]
        size = orc.dtype_size(dtype)
        nranks = int(rng.choice([1, 2, 3, 4, 5, 7, 8, 8, 8, 13, 16]))
        op = int(rng.choice([orc.SUM, orc.MAX, orc.MIN]))
        order = int(rng.choice([orc.ORDER_UCX, orc.ORDER_SHM, orc.ORDER_RANK0]))
        kind = rng.choice(["all_reduce", "all_reduce", "reduce_scatter", "reduce"])
        nbytes = draw_length(rng, nranks)
        offs = offsets_for(rng, nranks, size)
        outs = offs if rng.random() < 0.6 else offsets_for(rng, nranks, size)  # outputs at the inputs' offsets, or not
        what = f"seed={seed} case={case} {kind} dtype={dtype} N={nranks} op={op} order={order} offs={offs} outs={outs}"
        if kind == "all_reduce":
            length = nbytes // size
            sched = mr.Schedule.FUSED if rng.random() < 0.7 else mr.Schedule.TWO_PHASE
            inplace = rng.random() < 0.3
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            want = orc.fold_all_reduce(ins, dtype, op, order)
            d_in = [to_device(x, offs[r]) for r, x in enumerate(ins)]
            d_out = d_in if inplace else [empty_device(length * size, outs[r]) for r in range(nranks)]
            mr.all_reduce(d_in, d_out, length, dtype, op, order, sched)
            torch.cuda.synchronize()
            for r in range(nranks):
                same(to_host(d_out[r], ins[0].dtype), want[r], f"{what} len={length} sched={sched} inplace={inplace} rank={r}")
        elif kind == "reduce_scatter":
            recvlen = nbytes // size // nranks
            ins = [rand_array(dtype, recvlen * nranks, rng) for _ in range(nranks)]
            want = orc.fold_reduce_scatter(ins, dtype, op, order)
            d_in = [to_device(x, offs[r]) for r, x in enumerate(ins)]
            d_out = [empty_device(recvlen * size, outs[r]) for r in range(nranks)]
            mr.reduce_scatter(d_in, d_out, recvlen, dtype, op, order)
            torch.cuda.synchronize()
            for r in range(nranks):
                same(to_host(d_out[r], ins[0].dtype), want[r], f"{what} recvlen={recvlen} rank={r}")
        else:
            length = nbytes // size
            root = int(rng.integers(0, nranks))
            order = int(rng.choice([orc.ORDER_SHM, orc.ORDER_RANK0]))  # left folds; the tree has its own tests
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            want = orc.fold_all_reduce(ins, dtype, op, order)[0]
            d_in = [to_device(x, offs[r]) for r, x in enumerate(ins)]
            d_out = empty_device(length * size, outs[root])
            mr.reduce_to_root(d_in, d_out, length, dtype, op, root, order)
            torch.cuda.synchronize()
            same(to_host(d_out, ins[0].dtype), want, f"{what} len={length} root={root}")
        check_guards(what)


@pytest.mark.parametrize("seed", range(3))
def test_random_copies(seed):
    rng = np.random.default_rng(7000 + seed)
    for case in range(100):
        dtype = COPY_TYPES[rng.integers(0, len(COPY_TYPES))]
        gen = orc.UINT8 if dtype == orc.CHAR else dtype
        size = orc.dtype_size(dtype)
        nranks = int(rng.choice([1, 2, 3, 4, 5, 8, 8, 16]))
        kind = rng.choice(["all_gather", "all_to_all", "scatter", "gather", "broadcast"])
        block = draw_length(rng, nranks) // size // (nranks if kind != "broadcast" else 1)
        offs = offsets_for(rng, nranks, size)
        outs = offs if rng.random() < 0.5 else offsets_for(rng, nranks, size)
        root = int(rng.integers(0, nranks))
        what = f"seed={seed} case={case} {kind} dtype={dtype} N={nranks} block={block} offs={offs} outs={outs} root={root}"
        if kind == "all_gather":
            parts = [rand_array(gen, block, rng) for _ in range(nranks)]
            want = orc.ucx_all_gather(parts, dtype)
            d_in = [to_device(x, offs[r]) for r, x in enumerate(parts)]
            d_out = [empty_device(nranks * block * size, outs[r]) for r in range(nranks)]
            mr.all_gather(d_in, d_out, block, dtype)
            torch.cuda.synchronize()
            for r in range(nranks):
                same(to_host(d_out[r], parts[0].dtype), want[r], f"{what} rank={r}")
        elif kind == "all_to_all":
            ins = [rand_array(gen, nranks * block, rng) for _ in range(nranks)]
            want = orc.ucx_all_to_all(ins, dtype)
            d_in = [to_device(x, offs[r]) for r, x in enumerate(ins)]
            d_out = [empty_device(nranks * block * size, outs[r]) for r in range(nranks)]
            mr.all_to_all(d_in, d_out, block, dtype)
            torch.cuda.synchronize()
            for r in range(nranks):
                same(to_host(d_out[r], ins[0].dtype), want[r], f"{what} rank={r}")
        elif kind == "scatter":
            src = rand_array(gen, nranks * block, rng)
            want = orc.ucx_scatter([src if r == root else None for r in range(nranks)], dtype, root)
            d_root = to_device(src, offs[root])
            d_out = [empty_device(block * size, outs[r]) for r in range(nranks)]
            mr.scatter(d_root, d_out, block, dtype, root)
            torch.cuda.synchronize()
            for r in range(nranks):
                same(to_host(d_out[r], src.dtype), want[r], f"{what} rank={r}")
        elif kind == "gather":
            parts = [rand_array(gen, block, rng) for _ in range(nranks)]
            want = orc.ucx_gather(parts, dtype, root)[root]
            d_in = [to_device(x, offs[r]) for r, x in enumerate(parts)]
            d_root = empty_device(nranks * block * size, outs[root])
            mr.gather(d_in, d_root, block, dtype, root)
            torch.cuda.synchronize()
            same(to_host(d_root, parts[0].dtype), want, what)
        else:
            parts = [rand_array(gen, block, rng) for _ in range(nranks)]
            want = orc.ucx_broadcast(parts, dtype, root)
            d_root = to_device(parts[root], offs[root])
            d_out = [empty_device(block * size, outs[r]) for r in range(nranks)]
            mr.broadcast(d_root, d_out, block, dtype, root)
            torch.cuda.synchronize()
            for r in range(nranks):
                same(to_host(d_out[r], parts[0].dtype), want[r], f"{what} rank={r}")
        check_guards(what)
