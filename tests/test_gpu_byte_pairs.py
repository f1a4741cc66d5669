"""Every pair of byte values through the packed byte paths of the HIP kernels.

The reference's reduce kernels take int8 / uint8 one element per thread (src/ucx/kernel.cu:16-38, dispatch :62-69:
SUM wraps mod 256, MAX / MIN compare as signed or unsigned bytes).  The HIP kernels take sixteen bytes per lane:
SUM adds four bytes per register with the carries cut at the byte borders, MAX / MIN split each word into even and
odd bytes as 16-bit lanes.  A slip in the masks or the sign extension shows on particular operand pairs only, so
this runs ALL 65 536 (a, b) pairs x {INT8, UINT8} x {SUM, MAX, MIN} through every kernel family and compares with the
oracle's element-by-element loops:

  * the two-input reduce (`mrv_reduce`), short (one wavefront per tile) and long (four-wavefront group form);
  * as ranks 0 and 1 of an all_reduce of 3, 4 and 8 ranks (the other ranks random), short (flat kernel) and long (group
    kernel), in the ring order and in the order 0..N-1 (where ranks 0 and 1 meet first in every element);
  * as ranks 0 and 1 of a 5-rank reduce towards rank 0 (binomial tree kernel: the root takes rank 1 in first).
"""
import numpy as np
import pytest

import oracle as orc

torch = pytest.importorskip("torch")
pytestmark = pytest.mark.gpu

import megray_amd as mr  # noqa: E402
from gpu_util import bits_equal, empty_device, first_mismatch, rand_array, to_device, to_host  # noqa: E402

OPS = [orc.SUM, orc.MAX, orc.MIN]
REPEATS = {"short": 1, "long": 240}  # 64 tiles / 15360 tiles of 1 KiB: below and above the group forms' thresholds (two ranks': 15360)


def all_pairs(dtype, repeats):
    npdt = orc.NP_DTYPE[dtype]
    values = np.arange(256, dtype=np.uint8)
    a = np.tile(np.repeat(values, 256), repeats).view(npdt)
    b = np.tile(np.tile(values, 256), repeats).view(npdt)
    return a, b


def same(got, want, what):
    assert bits_equal(got, want), f"{what}: first mismatch (index, got, want, count) = {first_mismatch(got, want)}"


@pytest.mark.parametrize("size", list(REPEATS))
@pytest.mark.parametrize("op", OPS)
@pytest.mark.parametrize("dtype", [orc.INT8, orc.UINT8])
def test_two_input_reduce_on_every_byte_pair(dtype, op, size):
    a, b = all_pairs(dtype, REPEATS[size])
    runs, _, _ = mr.describe(mr.Collective.REDUCE2, [to_device(a), to_device(b)], [empty_device(a.size)], a.size, dtype, nranks=2)
    assert all(r["waves"] == (4 if size == "long" else 1) for r in runs if r["vector"]), runs
    for x, y in ((a, b), (b, a)):
        out = empty_device(x.size)
        mr.reduce(to_device(x), to_device(y), out, x.size, dtype, op)
        torch.cuda.synchronize()
        same(to_host(out, x.dtype), orc.reduce_ucx(x, y, dtype, op), f"reduce dtype={dtype} op={op} {size}")


@pytest.mark.parametrize("size", list(REPEATS))
@pytest.mark.parametrize("nranks", [3, 4, 8])
@pytest.mark.parametrize("dtype", [orc.INT8, orc.UINT8])
def test_all_reduce_with_every_byte_pair_on_ranks_0_and_1(dtype, nranks, size):
    a, b = all_pairs(dtype, REPEATS[size])
    rng = np.random.default_rng(4242 + 10 * dtype + nranks)
    ins = [a, b] + [rand_array(dtype, a.size, rng) for _ in range(nranks - 2)]
    d_in = [to_device(x) for x in ins]
    runs, _, _ = mr.describe(mr.Collective.ALL_REDUCE, d_in, [empty_device(a.size) for _ in range(nranks)], a.size, dtype)
    assert all(r["vector"] == 2 and r["waves"] == (4 if size == "long" else 1) for r in runs), runs
    for op in OPS:
        for order in (orc.ORDER_UCX, orc.ORDER_RANK0):
            d_out = [empty_device(a.size) for _ in range(nranks)]
            mr.all_reduce(d_in, d_out, a.size, dtype, op, order, mr.Schedule.FUSED)
            torch.cuda.synchronize()
            want = orc.fold_all_reduce(ins, dtype, op, order)
            for r in range(nranks):
                same(to_host(d_out[r], a.dtype), want[r], f"all_reduce dtype={dtype} N={nranks} op={op} order={order} {size} rank={r}")


@pytest.mark.parametrize("size", list(REPEATS))
@pytest.mark.parametrize("dtype", [orc.INT8, orc.UINT8])
def test_tree_reduce_with_every_byte_pair_on_ranks_0_and_1(dtype, size):
    nranks, root = 5, 0
    a, b = all_pairs(dtype, REPEATS[size])
    rng = np.random.default_rng(977 + dtype)
    ins = [a, b] + [rand_array(dtype, a.size, rng) for _ in range(nranks - 2)]
    d_in = [to_device(x) for x in ins]
    for op in OPS:
        out = empty_device(a.size)
        mr.reduce_to_root(d_in, out, a.size, dtype, op, root, orc.ORDER_UCX)
        torch.cuda.synchronize()
        same(to_host(out, a.dtype), orc.ucx_reduce(ins, dtype, op, root)[root], f"reduce to root dtype={dtype} op={op} {size}")
