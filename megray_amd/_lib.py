"""ctypes binding of libmegray_vrank.so (the C ABI declared in include/megray_vrank.h).

There is no fallback: if the library is missing or fails to load, importing a function from it
raises.  Build it with ``python -m megray_amd.build``.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmegray_vrank.so")


class PlanRun(ctypes.Structure):
    """struct mrv_plan_run"""
    _fields_ = [
        ("step", ctypes.c_uint32), ("kind", ctypes.c_uint32), ("nfold", ctypes.c_uint32),
        ("nout", ctypes.c_uint32), ("new_wins_ties", ctypes.c_uint32), ("vector", ctypes.c_uint32),
        ("start", ctypes.c_uint32), ("dir", ctypes.c_int32), ("out_first", ctypes.c_uint32),
        ("tiles", ctypes.c_uint32), ("reads_recv", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
        ("in_begin", ctypes.c_uint64), ("out_begin", ctypes.c_uint64),
        ("count", ctypes.c_uint64),
    ]


_lib = None


def load():
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: the HIP extension is not built "
            "(run `python -m megray_amd.build`); there is no CPU fallback")
    L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
    vp, sz, u32, i32 = ctypes.c_void_p, ctypes.c_size_t, ctypes.c_uint32, ctypes.c_int
    pp = ctypes.POINTER(ctypes.c_void_p)
    L.mrv_abi_version.restype = i32
    L.mrv_abi_version.argtypes = []
    L.mrv_last_error.restype = ctypes.c_char_p
    L.mrv_last_error.argtypes = []
    L.mrv_dtype_size.restype = sz
    L.mrv_dtype_size.argtypes = [i32]
    L.mrv_reduce.argtypes = [vp, vp, vp, sz, i32, i32, vp]
    L.mrv_all_reduce.argtypes = [pp, pp, u32, sz, i32, i32, i32, i32, vp]
    L.mrv_reduce_scatter.argtypes = [pp, pp, u32, sz, i32, i32, i32, vp]
    L.mrv_all_gather.argtypes = [pp, pp, u32, sz, i32, vp]
    L.mrv_all_to_all.argtypes = [pp, pp, u32, sz, i32, vp]
    L.mrv_scatter.argtypes = [vp, pp, u32, sz, i32, u32, vp]
    L.mrv_gather.argtypes = [pp, vp, u32, sz, i32, u32, vp]
    L.mrv_broadcast.argtypes = [vp, pp, u32, sz, i32, u32, vp]
    L.mrv_chunk_partition.argtypes = [sz, u32, ctypes.POINTER(sz), ctypes.POINTER(sz)]
    L.mrv_fold_order.argtypes = [i32, i32, u32, u32, ctypes.POINTER(u32), ctypes.POINTER(i32),
                                 ctypes.POINTER(u32), ctypes.POINTER(u32)]
    L.mrv_describe.argtypes = [i32, pp, pp, u32, sz, i32, i32, i32, u32, ctypes.POINTER(PlanRun), sz,
                               ctypes.POINTER(sz), ctypes.POINTER(ctypes.c_uint64),
                               ctypes.POINTER(ctypes.c_uint64)]
    for name in ("mrv_reduce", "mrv_all_reduce", "mrv_reduce_scatter", "mrv_all_gather",
                 "mrv_all_to_all", "mrv_scatter", "mrv_gather", "mrv_broadcast", "mrv_chunk_partition",
                 "mrv_fold_order", "mrv_describe"):
        getattr(L, name).restype = i32
    _lib = L
    return L
