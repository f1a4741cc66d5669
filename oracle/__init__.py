"""ctypes binding of the CPU oracle (oracle/megray_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py`` as the checker.  The product package ``megray_amd`` never
imports this module and has no CPU fallback.
"""
import ctypes
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmegray_oracle.so")

# numeric values of the reference enums (include/megray/common.h:106-127)
INT8, UINT8, INT32, UINT32, INT64, UINT64, FLOAT16, FLOAT32, FLOAT64, CHAR = range(10)
SUM, MAX, MIN = range(3)
ORDER_UCX, ORDER_SHM, ORDER_RANK0 = range(3)
COLL_ALL_REDUCE, COLL_REDUCE_SCATTER = range(2)
OK, UNSUPPORTED, BAD_ARG = 0, -1, -2

NP_DTYPE = {
    INT8: np.int8, UINT8: np.uint8, INT32: np.int32, UINT32: np.uint32, INT64: np.int64,
    UINT64: np.uint64, FLOAT16: np.float16, FLOAT32: np.float32, FLOAT64: np.float64,
    CHAR: np.uint8,
}

_REDUCE2 = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                            ctypes.c_size_t, ctypes.c_int, ctypes.c_int, ctypes.c_void_p)


def build(force=False):
    """Compile the oracle with gcc (oracle/Makefile)."""
    if force:
        subprocess.check_call(["make", "-s", "-C", HERE, "clean"])
    subprocess.check_call(["make", "-s", "-C", HERE])


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        vp, sz, u32, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32, ctypes.c_int
        pp = ctypes.POINTER(ctypes.c_void_p)
        L.orc_dtype_size.restype = sz
        L.orc_dtype_size.argtypes = [i32]
        for name in ("orc_ring_add", "orc_ring_sub"):
            getattr(L, name).restype = u32
            getattr(L, name).argtypes = [u32, u32, u32]
        L.orc_chunk_partition.restype = None
        L.orc_chunk_partition.argtypes = [sz, sz, ctypes.POINTER(sz), ctypes.POINTER(sz)]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f32_to_f16.restype = ctypes.c_uint16
        L.orc_f32_to_f16.argtypes = [ctypes.c_float]
        L.orc_reduce_ucx.argtypes = [vp, vp, vp, sz, i32, i32]
        L.orc_reduce_shm.argtypes = [vp, vp, vp, i32, i32, sz]
        L.orc_trace_reduce2.argtypes = [vp, vp, vp, sz, i32, i32, vp]
        for name in ("orc_ucx_all_reduce", "orc_ucx_reduce_scatter", "orc_shm_all_reduce",
                     "orc_shm_reduce_scatter"):
            getattr(L, name).argtypes = [u32, pp, pp, sz, i32, i32, vp, vp]
        for name in ("orc_ucx_all_gather", "orc_ucx_all_to_all", "orc_shm_all_gather",
                     "orc_shm_all_to_all"):
            getattr(L, name).argtypes = [u32, pp, pp, sz, i32]
        for name in ("orc_ucx_scatter", "orc_ucx_gather", "orc_ucx_broadcast", "orc_shm_broadcast"):
            getattr(L, name).argtypes = [u32, pp, pp, sz, i32, u32]
        L.orc_ucx_reduce.argtypes = [u32, pp, pp, sz, i32, i32, u32, vp, vp]
        L.orc_shm_reduce.argtypes = [u32, pp, pp, sz, i32, i32, u32, vp, vp]
        L.orc_test_all_reduce_f32.restype = None
        L.orc_test_all_reduce_f32.argtypes = [u32, pp, pp, sz, i32]
        L.orc_test_reduce_scatter_f32.restype = None
        L.orc_test_reduce_scatter_f32.argtypes = [u32, pp, pp, sz, i32]
        L.orc_test_all_reduce_f32_mt.restype = None
        L.orc_test_all_reduce_f32_mt.argtypes = [u32, pp, pp, sz, i32, i32]
        L.orc_fold_order.argtypes = [i32, i32, u32, u32, ctypes.POINTER(u32),
                                     ctypes.POINTER(i32), ctypes.POINTER(u32)]
        L.orc_fold_all_reduce.argtypes = [u32, pp, pp, sz, i32, i32, i32]
        L.orc_fold_reduce_scatter.argtypes = [u32, pp, pp, sz, i32, i32, i32]
        _lib = L
    return _lib


def _ptrs(arrays):
    arr = (ctypes.c_void_p * len(arrays))()
    for i, a in enumerate(arrays):
        arr[i] = None if a is None else a.ctypes.data
    return arr


def _check(rc, what):
    if rc == UNSUPPORTED:
        raise NotImplementedError(f"{what}: the reference throws for this dtype/op")
    if rc != OK:
        raise ValueError(f"{what}: bad argument (rc={rc})")


def dtype_size(dtype):
    return lib().orc_dtype_size(dtype)


def ring_add(n, d, m):
    return lib().orc_ring_add(n, d, m)


def ring_sub(n, d, m):
    return lib().orc_ring_sub(n, d, m)


def chunk_partition(length, nchunks):
    sizes = (ctypes.c_size_t * nchunks)()
    offs = (ctypes.c_size_t * nchunks)()
    lib().orc_chunk_partition(length, nchunks, sizes, offs)
    return list(sizes), list(offs)


def f16_to_f32(bits):
    return lib().orc_f16_to_f32(int(bits))


def f32_to_f16(value):
    return lib().orc_f32_to_f16(float(value))


def reduce_ucx(i0, i1, dtype, op):
    """o = reduce(i0, i1) as src/ucx/kernel.cu computes it."""
    out = np.empty_like(i0)
    _check(lib().orc_reduce_ucx(i0.ctypes.data, i1.ctypes.data, out.ctypes.data, i0.size, dtype, op),
           "reduce_ucx")
    return out


def reduce_shm(a, b, dtype, op):
    """dst = cpu_reduce(a, b) as src/shm/utils.cpp computes it."""
    out = np.empty_like(a)
    _check(lib().orc_reduce_shm(out.ctypes.data, a.ctypes.data, b.ctypes.data, dtype, op, a.size),
           "reduce_shm")
    return out


def _trace_fn(trace):
    if not trace:
        return None
    return ctypes.cast(lib().orc_trace_reduce2, ctypes.c_void_p)


def _run_reduce(fn_name, sends, out_len, count, dtype, op, trace=False, inplace=False):
    n = len(sends)
    if inplace:
        recvs = sends
    else:
        recvs = [np.empty(out_len, dtype=sends[0].dtype) for _ in range(n)]
    rc = getattr(lib(), fn_name)(n, _ptrs(sends), _ptrs(recvs), count, dtype, op, _trace_fn(trace),
                                 None)
    _check(rc, fn_name)
    return recvs


def ucx_all_reduce(sends, dtype, op, trace=False, inplace=False):
    return _run_reduce("orc_ucx_all_reduce", sends, sends[0].size, sends[0].size, dtype, op, trace,
                       inplace)


def shm_all_reduce(sends, dtype, op, trace=False):
    return _run_reduce("orc_shm_all_reduce", sends, sends[0].size, sends[0].size, dtype, op, trace)


def ucx_reduce_scatter(sends, dtype, op, trace=False):
    recvlen = sends[0].size // len(sends)
    return _run_reduce("orc_ucx_reduce_scatter", sends, recvlen, recvlen, dtype, op, trace)


def shm_reduce_scatter(sends, dtype, op, trace=False):
    recvlen = sends[0].size // len(sends)
    return _run_reduce("orc_shm_reduce_scatter", sends, recvlen, recvlen, dtype, op, trace)


def _run_copy(fn_name, sends, out_len, count, dtype, *extra):
    n = len(sends)
    proto = next(s for s in sends if s is not None)
    recvs = [np.zeros(out_len, dtype=proto.dtype) for _ in range(n)]
    rc = getattr(lib(), fn_name)(n, _ptrs(sends), _ptrs(recvs), count, dtype, *extra)
    _check(rc, fn_name)
    return recvs


def ucx_all_gather(sends, dtype):
    return _run_copy("orc_ucx_all_gather", sends, sends[0].size * len(sends), sends[0].size, dtype)


def shm_all_gather(sends, dtype):
    return _run_copy("orc_shm_all_gather", sends, sends[0].size * len(sends), sends[0].size, dtype)


def ucx_all_to_all(sends, dtype):
    return _run_copy("orc_ucx_all_to_all", sends, sends[0].size, sends[0].size // len(sends), dtype)


def shm_all_to_all(sends, dtype):
    return _run_copy("orc_shm_all_to_all", sends, sends[0].size, sends[0].size // len(sends), dtype)


def ucx_scatter(sends, dtype, root):
    recvlen = sends[root].size // len(sends)
    return _run_copy("orc_ucx_scatter", sends, recvlen, recvlen, dtype, root)


def ucx_gather(sends, dtype, root):
    """Only recvs[root] is meaningful."""
    return _run_copy("orc_ucx_gather", sends, sends[0].size * len(sends), sends[0].size, dtype, root)


def ucx_broadcast(sends, dtype, root):
    return _run_copy("orc_ucx_broadcast", sends, sends[root].size, sends[root].size, dtype, root)


def shm_reduce(sends, dtype, op, root, trace=False):
    """Literal replay of src/shm/reduce.cpp:21-100.  Only recvs[root] is meaningful."""
    n = len(sends)
    recvs = [np.zeros(sends[0].size, dtype=sends[0].dtype) for _ in range(n)]
    rc = lib().orc_shm_reduce(n, _ptrs(sends), _ptrs(recvs), sends[0].size, dtype, op, root,
                              _trace_fn(trace), None)
    _check(rc, "orc_shm_reduce")
    return recvs


def shm_broadcast(sends, dtype, root):
    """Literal replay of src/shm/broadcast.cpp:19-51 (only sends[root] is read)."""
    return _run_copy("orc_shm_broadcast", sends, sends[root].size, sends[root].size, dtype, root)


def ucx_reduce(sends, dtype, op, root, trace=False):
    """Only recvs[root] is meaningful."""
    n = len(sends)
    recvs = [np.zeros(sends[0].size, dtype=sends[0].dtype) for _ in range(n)]
    rc = lib().orc_ucx_reduce(n, _ptrs(sends), _ptrs(recvs), sends[0].size, dtype, op, root,
                              _trace_fn(trace), None)
    _check(rc, "orc_ucx_reduce")
    return recvs


def test_all_reduce_f32(ins, op, nthreads=0):
    n = len(ins)
    outs = [np.empty_like(ins[0]) for _ in range(n)]
    if nthreads:
        lib().orc_test_all_reduce_f32_mt(n, _ptrs(ins), _ptrs(outs), ins[0].size, op, nthreads)
    else:
        lib().orc_test_all_reduce_f32(n, _ptrs(ins), _ptrs(outs), ins[0].size, op)
    return outs


test_all_reduce_f32.__test__ = False


def test_reduce_scatter_f32(ins, op):
    n = len(ins)
    recvlen = ins[0].size // n
    outs = [np.empty(recvlen, dtype=np.float32) for _ in range(n)]
    lib().orc_test_reduce_scatter_f32(n, _ptrs(ins), _ptrs(outs), recvlen, op)
    return outs


test_reduce_scatter_f32.__test__ = False


def fold_order(coll, order, nranks, chunk):
    """-> (ranks, new_wins_ties, nchunks)"""
    ranks = (ctypes.c_uint32 * nranks)()
    new_wins = ctypes.c_int(0)
    nchunks = ctypes.c_uint32(0)
    rc = lib().orc_fold_order(coll, order, nranks, chunk, ranks, ctypes.byref(new_wins),
                              ctypes.byref(nchunks))
    _check(rc, "orc_fold_order")
    return list(ranks), bool(new_wins.value), nchunks.value


def fold_all_reduce(sends, dtype, op, order=ORDER_UCX):
    n = len(sends)
    recvs = [np.empty_like(sends[0]) for _ in range(n)]
    rc = lib().orc_fold_all_reduce(n, _ptrs(sends), _ptrs(recvs), sends[0].size, dtype, op, order)
    _check(rc, "orc_fold_all_reduce")
    return recvs


def fold_reduce_scatter(sends, dtype, op, order=ORDER_UCX):
    n = len(sends)
    recvlen = sends[0].size // n
    recvs = [np.empty(recvlen, dtype=sends[0].dtype) for _ in range(n)]
    rc = lib().orc_fold_reduce_scatter(n, _ptrs(sends), _ptrs(recvs), recvlen, dtype, op, order)
    _check(rc, "orc_fold_reduce_scatter")
    return recvs
