"""Lengths around the borders of vectors and tiles, through the flat kernels (2, 3, 4 and 8 ranks): chunk borders that
cut 16-byte vectors, tiles that span several chunks, and the buffers' last tile with a few whole vectors and a few
elements behind them.  The flat kernel folds such a tile run by run out of LDS and, for an all_reduce, stores each
lane's collected vector once; every output lies between guard bytes."""
import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import Guarded, bits_equal, first_mismatch, rand_array, to_device, to_host  # noqa: E402


def lengths_around(elem_size):
    per_vector, per_tile = 16 // elem_size, 1024 // elem_size
    out = set(range(1, 2 * per_vector + 2))
    for base in (per_tile, 4 * per_tile, 9 * per_tile):
        out.update(range(base - per_vector - 1, base + per_vector + 2))
    return sorted(n for n in out if n > 0)


def check(outs, wants, what):
    torch.cuda.synchronize()
    for r, (g, want) in enumerate(zip(outs, wants)):
        got = to_host(g.view, want.dtype)
        assert bits_equal(got, want), f"{what} rank={r}: first mismatch {first_mismatch(got, want)}"
        assert g.intact(), f"{what} rank={r}: written outside the buffer"


@pytest.mark.parametrize("dtype", [orc.UINT8, orc.FLOAT16, orc.FLOAT32, orc.FLOAT64])
@pytest.mark.parametrize("nranks", [2, 3, 4, 8])
def test_lengths_around_vector_and_tile_borders(dtype, nranks):
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(8800 + 16 * dtype + nranks)
    for length in lengths_around(size):
        ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
        d_in = [to_device(x) for x in ins]
        op, order = (orc.SUM, orc.ORDER_UCX) if length % 2 else (orc.MAX, orc.ORDER_SHM)
        outs = [Guarded(length * size) for _ in range(nranks)]
        mr.all_reduce(d_in, [g.view for g in outs], length, dtype, op, order)
        check(outs, orc.fold_all_reduce(ins, dtype, op, order), f"all_reduce dtype={dtype} N={nranks} len={length}")
        # towards a root: the binomial tree (a flat launch with one output)
        if dtype != orc.FLOAT16:  # the oracle's literal tree has no FLOAT16
            root = length % nranks
            out = Guarded(length * size)
            mr.reduce_to_root(d_in, out.view, length, dtype, orc.MIN, root)
            check([out], [orc.ucx_reduce(ins, dtype, orc.MIN, root)[root]], f"reduce dtype={dtype} N={nranks} len={length}")
        # one output per chunk, each in another rank's buffer: the pieces of a cut vector go to two buffers
        recvlen = length // nranks
        if recvlen:
            part = [x[:recvlen * nranks] for x in ins]
            d_part = [to_device(x) for x in part]
            outs = [Guarded(recvlen * size) for _ in range(nranks)]
            mr.reduce_scatter(d_part, [g.view for g in outs], recvlen, dtype, orc.SUM)
            check(outs, orc.fold_reduce_scatter(part, dtype, orc.SUM, orc.ORDER_UCX),
                  f"reduce_scatter dtype={dtype} N={nranks} recvlen={recvlen}")


@pytest.mark.parametrize("dtype", [orc.UINT8, orc.FLOAT32])
def test_the_group_form_at_the_buffers_end(dtype):
    """Long launches (10752 tiles and more for three ranks, 2560 for eight): four wavefronts per workgroup; the
    wavefront that holds the buffers' last tile loads it lane by lane, and tiles across chunk borders come out of the
    group's LDS."""
    size = orc.dtype_size(dtype)
    rng = np.random.default_rng(8900 + dtype)
    per_vector, per_tile = 16 // size, 1024 // size
    for nranks in (3, 8):
        for extra in (1, per_vector - 1, per_vector + 1, per_tile - 1, 5 * per_vector + 3):
            length = {3: 10800, 8: 2600}[nranks] * per_tile + extra
            ins = [rand_array(dtype, length, rng) for _ in range(nranks)]
            d_in = [to_device(x) for x in ins]
            runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, d_in, d_in, length, dtype)
            assert all(r["waves"] == 4 for r in runs)
            outs = [Guarded(length * size) for _ in range(nranks)]
            mr.all_reduce(d_in, [g.view for g in outs], length, dtype, orc.SUM, orc.ORDER_UCX)
            check(outs, orc.fold_all_reduce(ins, dtype, orc.SUM, orc.ORDER_UCX), f"group form dtype={dtype} N={nranks} len={length}")
