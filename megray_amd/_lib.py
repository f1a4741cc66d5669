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
        ("tiles", ctypes.c_uint32), ("reads_recv", ctypes.c_uint32), ("waves", ctypes.c_uint32),
        ("in_begin", ctypes.c_uint64), ("out_begin", ctypes.c_uint64),
        ("count", ctypes.c_uint64), ("deal", ctypes.c_uint32), ("paced", ctypes.c_uint32),
        ("keep", ctypes.c_uint32), ("reserved", ctypes.c_uint32),
    ]


# void (*mrv_bcast_fn)(char* data, size_t len, void* user)
BCAST_FN = ctypes.CFUNCTYPE(None, ctypes.POINTER(ctypes.c_char), ctypes.c_size_t, ctypes.c_void_p)

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
    L.mrv_plan_create.argtypes = [i32, pp, pp, u32, sz, i32, i32, i32, i32, u32, u32, ctypes.POINTER(vp)]
    L.mrv_plan_create.restype = i32
    L.mrv_plan_launch.argtypes = [vp, vp]
    L.mrv_plan_launch.restype = i32
    L.mrv_plan_launch_count.argtypes = [vp]
    L.mrv_plan_launch_count.restype = sz
    L.mrv_plan_destroy.argtypes = [vp]
    L.mrv_plan_destroy.restype = None
    L.mrv_reduce_to_root.argtypes = [pp, vp, u32, sz, i32, i32, i32, u32, vp]
    L.mrv_probe_bounded_wait.argtypes = [ctypes.c_uint64, vp, ctypes.POINTER(ctypes.c_uint64)]
    L.mrv_probe_bounded_wait.restype = i32
    L.mrv_rank_buffers_layout.argtypes = [i32, ctypes.POINTER(sz), ctypes.POINTER(sz), ctypes.POINTER(sz)]
    L.mrv_rank_buffers_alloc.argtypes = [i32, ctypes.POINTER(sz), ctypes.POINTER(vp), ctypes.POINTER(vp)]
    L.mrv_rank_buffers_free.argtypes = [vp]
    u8p = ctypes.POINTER(ctypes.c_ubyte)
    L.mrv_rank_buffers_layout_for.argtypes = [i32, i32, ctypes.POINTER(sz), u8p, ctypes.POINTER(sz), ctypes.POINTER(sz)]
    L.mrv_rank_buffers_alloc_for.argtypes = [i32, i32, ctypes.POINTER(sz), u8p, ctypes.POINTER(vp), ctypes.POINTER(vp)]
    L.mrv_rank_buffers_layout_for.restype = L.mrv_rank_buffers_alloc_for.restype = i32
    L.mrv_get_free_port.argtypes = []
    L.mrv_create_server.argtypes = [u32, i32]
    L.mrv_comm_create.argtypes = [u32, u32, i32, ctypes.POINTER(vp)]
    L.mrv_comm_destroy.argtypes = [vp]
    L.mrv_comm_destroy.restype = None
    L.mrv_comm_init.argtypes = [vp, ctypes.c_char_p, i32]
    L.mrv_comm_init_callback.argtypes = [vp, BCAST_FN, vp]
    L.mrv_comm_check.argtypes = [vp, vp]
    u64p = ctypes.POINTER(ctypes.c_uint64)
    L.mrv_comm_stats.argtypes = [vp, u64p, u64p, u64p]
    L.mrv_comm_configure.argtypes = [vp, i32, i32]
    L.mrv_comm_send.argtypes = [vp, vp, sz, i32, u32, vp]
    L.mrv_comm_recv.argtypes = [vp, vp, sz, i32, u32, vp]
    L.mrv_comm_scatter.argtypes = [vp, vp, vp, sz, i32, u32, vp]
    L.mrv_comm_gather.argtypes = [vp, vp, vp, sz, i32, u32, vp]
    L.mrv_comm_all_to_all.argtypes = [vp, vp, vp, sz, i32, vp]
    L.mrv_comm_all_gather.argtypes = [vp, vp, vp, sz, i32, vp]
    L.mrv_comm_all_reduce.argtypes = [vp, vp, vp, sz, i32, i32, vp]
    L.mrv_comm_all_reduce_no_alloc.argtypes = [vp, vp, vp, sz, i32, i32, vp]
    L.mrv_comm_reduce_scatter.argtypes = [vp, vp, vp, sz, i32, i32, vp]
    L.mrv_comm_broadcast.argtypes = [vp, vp, vp, sz, i32, u32, vp]
    L.mrv_comm_reduce.argtypes = [vp, vp, vp, sz, i32, i32, u32, vp]
    L.mrv_comm_group_start.argtypes = [vp]
    L.mrv_comm_group_end.argtypes = [vp]
    L.mrv_client_create.argtypes = [u32, u32, ctypes.POINTER(vp)]
    L.mrv_client_destroy.argtypes = [vp]
    L.mrv_client_destroy.restype = None
    L.mrv_client_connect.argtypes = [vp, ctypes.c_char_p, i32]
    L.mrv_client_barrier.argtypes = [vp]
    L.mrv_client_broadcast.argtypes = [vp, vp, vp, sz, u32]
    L.mrv_client_allgather.argtypes = [vp, vp, vp, sz]
    for name in ("mrv_reduce_to_root", "mrv_get_free_port", "mrv_create_server", "mrv_comm_create",
                 "mrv_comm_init", "mrv_comm_init_callback", "mrv_comm_check", "mrv_comm_stats", "mrv_comm_configure", "mrv_comm_send", "mrv_comm_recv", "mrv_comm_scatter",
                 "mrv_comm_gather", "mrv_comm_all_to_all", "mrv_comm_all_gather", "mrv_comm_all_reduce",
                 "mrv_comm_all_reduce_no_alloc",
                 "mrv_comm_reduce_scatter", "mrv_comm_broadcast", "mrv_comm_reduce", "mrv_comm_group_start",
                 "mrv_comm_group_end", "mrv_client_create", "mrv_client_connect", "mrv_client_barrier",
                 "mrv_client_broadcast", "mrv_client_allgather"):
        getattr(L, name).restype = i32
    for name in ("mrv_reduce", "mrv_all_reduce", "mrv_reduce_scatter", "mrv_all_gather",
                 "mrv_all_to_all", "mrv_scatter", "mrv_gather", "mrv_broadcast", "mrv_chunk_partition",
                 "mrv_fold_order", "mrv_describe"):
        getattr(L, name).restype = i32
    _lib = L
    return L
