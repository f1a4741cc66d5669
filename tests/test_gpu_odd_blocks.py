"""Blocks and runs that do not start on 16-byte boundaries (lengths that are no multiple of 16 bytes, buffers at
differing offsets): the pack kernels move 16 bytes per lane from the destination's first 16-byte boundary on, whatever
the source's byte address, and copy the few bytes around the vectors one by one; reduce_scatter of 4- and 8-byte
elements with such a receive length folds 16 bytes per lane with stores on 16-byte boundaries.  Checked against the
oracle's literal replays, with guard bytes around every output."""
import numpy as np
import pytest
import torch

import megray_amd as mr
import oracle as orc
from gpu_util import rand_array

pytestmark = pytest.mark.gpu
GUARD = 64
FILL = 0x5C


def device_in(arr, offset):
    raw = np.ascontiguousarray(arr).view(np.uint8).reshape(-1)
    buf = torch.empty(raw.size + offset + 64, dtype=torch.uint8, device="cuda")
    view = buf[offset:offset + raw.size]
    if raw.size:
        view.copy_(torch.from_numpy(raw.copy()))
    return view


class Guarded:
    """An output of `nbytes` bytes at `offset` from a 256-byte boundary with GUARD bytes of a fill pattern on
    both sides."""

    def __init__(self, nbytes, offset):
        self.buf = torch.full((256 + nbytes + 2 * GUARD + 64,), FILL, dtype=torch.uint8, device="cuda")
        lo = 256 - GUARD + offset  # the torch allocation is 256-byte aligned
        self.lo, self.nbytes = lo + GUARD, nbytes
        self.view = self.buf[self.lo:self.lo + nbytes]

    def check(self, want, what):
        host = self.buf.cpu().numpy()
        got = host[self.lo:self.lo + self.nbytes]
        assert np.array_equal(got, np.ascontiguousarray(want).view(np.uint8).reshape(-1)), what
        assert (host[self.lo - GUARD:self.lo] == FILL).all(), what + ": bytes in front of the output were written"
        assert (host[self.lo + self.nbytes:self.lo + self.nbytes + GUARD] == FILL).all(), what + ": bytes behind the output were written"


# lengths in elements: a few words, under one tile, several tiles with an odd end, group form (>= 128 tiles per block)
LENGTHS = {orc.FLOAT32: (1, 2, 3, 5, 7, 250, 1027, 4099, 33001 * 4 + 1, 33001 * 4 + 2, 33001 * 4 + 3),
           orc.INT64: (1, 3, 125, 1027, 16501 * 4 + 1),
           orc.UINT8: (1, 3, 15, 17, 31, 33, 1000, 4099, 33001 * 16 + 5),
           orc.FLOAT16: (1, 3, 9, 1027, 33001 * 8 + 3)}


@pytest.mark.parametrize("dtype", [orc.FLOAT32, orc.INT64, orc.UINT8, orc.FLOAT16])
@pytest.mark.parametrize("nranks", [2, 3, 8])
def test_pack_collectives_off_the_vector_grid(dtype, nranks):
    rng = np.random.default_rng(700 + dtype * 10 + nranks)
    size = orc.dtype_size(dtype)
    for length in LENGTHS[dtype]:
        if nranks == 8 and length > 40000 and dtype == orc.INT64:
            continue
        slots = 16 // size  # element offsets within a 16-byte vector
        for variant in range(3):
            # 0: every buffer on a 256-byte boundary (only the block length is odd); 1: every buffer at its own
            # offset; 2: all outputs at one offset, all inputs at another
            if variant == 0:
                in_off, out_off = [0] * nranks, [0] * nranks
            elif variant == 1:
                in_off = [size * ((3 * r + 1) % slots) for r in range(nranks)]
                out_off = [size * ((r + 2) % slots) for r in range(nranks)]
            else:
                in_off, out_off = [size * (slots - 1)] * nranks, [size * (1 % slots)] * nranks
            what = f"dtype={dtype} N={nranks} len={length} offsets={variant}"
            ins = [rand_array(dtype, nranks * length, rng) for _ in range(nranks)]
            parts = [x[:length] for x in ins]
            # all_to_all
            d_in = [device_in(x, in_off[r]) for r, x in enumerate(ins)]
            outs = [Guarded(nranks * length * size, out_off[r]) for r in range(nranks)]
            mr.all_to_all(d_in, [o.view for o in outs], length, dtype)
            torch.cuda.synchronize()
            for r, w in enumerate(orc.ucx_all_to_all(ins, dtype)):
                outs[r].check(w, "all_to_all " + what)
            # all_gather (every destination has its own alignment in variant 1)
            d_in = [device_in(x, in_off[r]) for r, x in enumerate(parts)]
            outs = [Guarded(nranks * length * size, out_off[r]) for r in range(nranks)]
            mr.all_gather(d_in, [o.view for o in outs], length, dtype)
            torch.cuda.synchronize()
            for r, w in enumerate(orc.ucx_all_gather(parts, dtype)):
                outs[r].check(w, "all_gather " + what)
            root = nranks - 1
            # scatter
            d_root = device_in(ins[root], in_off[root])
            outs = [Guarded(length * size, out_off[r]) for r in range(nranks)]
            mr.scatter(d_root, [o.view for o in outs], length, dtype, root)
            torch.cuda.synchronize()
            want = orc.ucx_scatter([ins[root] if r == root else None for r in range(nranks)], dtype, root)
            for r in range(nranks):
                outs[r].check(want[r], "scatter " + what)
            # gather
            d_in = [device_in(x, in_off[r]) for r, x in enumerate(parts)]
            out = Guarded(nranks * length * size, out_off[root])
            mr.gather(d_in, out.view, length, dtype, root)
            torch.cuda.synchronize()
            out.check(orc.ucx_gather(parts, dtype, root)[root], "gather " + what)
            # broadcast
            d_root = device_in(parts[root], in_off[root])
            outs = [Guarded(length * size, out_off[r]) for r in range(nranks)]
            mr.broadcast(d_root, [o.view for o in outs], length, dtype, root)
            torch.cuda.synchronize()
            want = orc.ucx_broadcast(parts, dtype, root)
            for r in range(nranks):
                outs[r].check(want[r], "broadcast " + what)


def test_the_vector_forms_are_what_runs():
    """describe(): blocks on 4-byte boundaries still go through the 16-byte kernels (group form when long), and a
    reduce_scatter whose receive length is no multiple of 16 bytes keeps vector bodies."""
    nranks, length = 8, 33001 * 4 + 1
    send = [(1 << 40) + (r << 32) for r in range(nranks)]
    recv = [(2 << 40) + (r << 34) for r in range(nranks)]
    for elems, waves in ((length, 1), (4 * length + 1, 4)):  # an all_gather of eight ranks takes the group form from 2 MiB per block
        runs, _, _ = mr.describe(mr.Collective.ALL_GATHER, send, recv, elems, orc.FLOAT32)
        assert runs and all(r["vector"] == 4 and r["waves"] == waves for r in runs), elems
    # an all_to_all of five ranks and more keeps one wavefront per tile up to 4 MiB per block (its launch is long either way)
    for ranks, elems, waves in ((8, length, 1), (4, length, 4), (8, (1 << 20) + 1, 4)):
        runs, _, _ = mr.describe(mr.Collective.ALL_TO_ALL, send[:ranks], recv[:ranks], elems, orc.FLOAT32)
        assert runs and all(r["vector"] == 4 and r["waves"] == waves for r in runs), (ranks, elems)
    for length, waves in ((33001 * 4 + 1, 1), (300001, 4)):  # folds into one output take the group form beyond 8 MiB per buffer
        runs, _, _ = mr.describe(mr.Collective.REDUCE_SCATTER, send, recv, length, orc.FLOAT32)
        body = sum(r["count"] for r in runs if r["vector"] == 1)
        assert body >= nranks * length - nranks * 3 * 300  # all but heads and tails of at most a tile's worth per run
        assert all(r["waves"] == waves for r in runs), length


@pytest.mark.parametrize("dtype", [orc.FLOAT32, orc.INT32, orc.FLOAT64, orc.INT64, orc.FLOAT16, orc.INT8, orc.UINT8])
def test_reduce_scatter_with_receive_lengths_off_the_vector_grid(dtype):
    rng = np.random.default_rng(800 + dtype)
    size = orc.dtype_size(dtype)
    for nranks in (2, 3, 5, 8):
        for recvlen in (3, 1027, 4099, (33001 * 16 + 4) // size * 1 + 1):
            ins = [rand_array(dtype, nranks * recvlen, rng) for _ in range(nranks)]
            for op in (orc.SUM, orc.MAX):
                for order in (orc.ORDER_UCX, orc.ORDER_SHM):
                    want = orc.fold_reduce_scatter(ins, dtype, op, order)
                    d_in = [device_in(x, 0) for x in ins]
                    outs = [Guarded(recvlen * size, 0) for _ in range(nranks)]
                    mr.reduce_scatter(d_in, [o.view for o in outs], recvlen, dtype, op, order)
                    torch.cuda.synchronize()
                    for r in range(nranks):
                        outs[r].check(want[r], f"reduce_scatter dtype={dtype} N={nranks} recvlen={recvlen} op={op} order={order}")
            if dtype in (orc.FLOAT32, orc.FLOAT64, orc.INT8):
                want = orc.ucx_reduce_scatter(ins, dtype, orc.SUM)  # the literal replay
                d_in = [device_in(x, 0) for x in ins]
                outs = [Guarded(recvlen * size, 0) for _ in range(nranks)]
                mr.reduce_scatter(d_in, [o.view for o in outs], recvlen, dtype, orc.SUM)
                torch.cuda.synchronize()
                for r in range(nranks):
                    outs[r].check(want[r], "reduce_scatter vs literal replay")


@pytest.mark.parametrize("dtype", [orc.FLOAT16, orc.INT8, orc.UINT8, orc.FLOAT32, orc.INT64])
def test_all_reduce_with_every_buffer_at_its_own_element_offset(dtype):
    """Inputs and outputs at differing offsets from a 16-byte boundary, in whole elements: 16 bytes per lane all the
    same, short (one wavefront per tile) and long (group form), for rank counts with and without a kernel of
    their own."""
    rng = np.random.default_rng(900 + dtype)
    size = orc.dtype_size(dtype)
    slots = 16 // size
    for nranks in (2, 5, 8):
        for length in (7, 1027, (700 * 1024) // size + 5):
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            in_off = [size * ((5 * r + 1) % slots) for r in range(nranks)]
            out_off = [size * ((3 * r + 2) % slots) for r in range(nranks)]
            for op, order in ((orc.SUM, orc.ORDER_UCX), (orc.MAX, orc.ORDER_SHM), (orc.MIN, orc.ORDER_RANK0)):
                want = orc.fold_all_reduce(ins, dtype, op, order)
                d_in = [device_in(x, in_off[r]) for r, x in enumerate(ins)]
                outs = [Guarded(length * size, out_off[r]) for r in range(nranks)]
                mr.all_reduce(d_in, [o.view for o in outs], length, dtype, op, order)
                torch.cuda.synchronize()
                for r in range(nranks):
                    outs[r].check(want[r], f"all_reduce dtype={dtype} N={nranks} len={length} op={op} order={order}")


def tree_expectation(ins, dtype, op, root):
    """The oracle's literal replay of the binomial tree towards `root`; FLOAT16 (which the reference cannot reduce)
    as the same tree in fp32 with one rounding at the end."""
    nranks = len(ins)
    if dtype != orc.FLOAT16:
        return orc.ucx_reduce(ins, dtype, op, root)[root]
    a = [ins[(root + v) % nranks].astype(np.float32) for v in range(nranks)]
    bit = 1
    while bit < nranks:
        for v in range(0, nranks - bit, 2 * bit):
            x, y = a[v], a[v + bit]
            with np.errstate(over="ignore"):
                a[v] = x + y if op == orc.SUM else np.where(y > x, y, x)
        bit *= 2
    with np.errstate(over="ignore"):
        return a[0].astype(np.float16)


@pytest.mark.parametrize("dtype", [orc.FLOAT16, orc.INT8, orc.FLOAT32, orc.INT64])
def test_reduce_to_root_with_every_buffer_at_its_own_element_offset(dtype):
    """The rooted reduce in the reference's binomial-tree order, for rank counts with (8) and without (5, 7, 16) a
    kernel of their own, on buffers at differing element offsets: 16 bytes per lane all the same."""
    rng = np.random.default_rng(950 + dtype)
    size = orc.dtype_size(dtype)
    slots = 16 // size
    for nranks in (5, 7, 8, 16):
        for length in (3, 1027, (300 * 1024) // size + 7):
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            in_off = [size * ((5 * r + 1) % slots) for r in range(nranks)]
            for op in (orc.SUM, orc.MAX):
                for root in (0, nranks - 2):
                    want = tree_expectation(ins, dtype, op, root)
                    d_in = [device_in(x, in_off[r]) for r, x in enumerate(ins)]
                    out = Guarded(length * size, size * (3 % slots))
                    mr.reduce_to_root(d_in, out.view, length, dtype, op, root)
                    torch.cuda.synchronize()
                    out.check(want, f"reduce dtype={dtype} N={nranks} len={length} op={op} root={root}")
