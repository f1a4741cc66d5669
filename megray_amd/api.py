"""Host-side mirror of the MegRay interface for the virtual-rank backend.

Names, argument meaning and error behaviour follow the reference's C++ API
(include/megray/common.h, include/megray/communicator.h): ``DType`` / ``ReduceOp`` / ``Status``
carry the same numeric values, lengths are element counts, contract violations raise
``MegRayError`` where the reference throws ``MegRay::Exception``.

The flat functions here take the buffers of all N virtual ranks at once (device pointers as ints,
or anything with ``data_ptr()``); they are thin wrappers over the C ABI.
"""
import ctypes
import enum

from . import _lib


class Status(enum.IntEnum):
    OK = 0
    SYS_ERROR = 1
    CUDA_ERR = 2
    NCCL_ERR = 3
    UCX_ERR = 4
    ENV_ERROR = 5
    INVALID_ARGUMENT = 6
    INVALID_USAGE = 7
    UNEXPECTED_ERR = 8
    NOT_IMPLEMENTED = 9
    HIP_ERR = 10
    RCCL_ERR = 11


class Backend(enum.IntEnum):
    NCCL = 0
    UCX = 1
    RCCL = 2
    SHM = 3
    VRANK = 4


class DType(enum.IntEnum):
    INT8 = 0
    UINT8 = 1
    INT32 = 2
    UINT32 = 3
    INT64 = 4
    UINT64 = 5
    FLOAT16 = 6
    FLOAT32 = 7
    FLOAT64 = 8
    CHAR = 9


class ReduceOp(enum.IntEnum):
    SUM = 0
    MAX = 1
    MIN = 2


class FoldOrder(enum.IntEnum):
    UCX = 0
    SHM = 1
    RANK0 = 2


class Schedule(enum.IntEnum):
    FUSED = 0
    TWO_PHASE = 1
    RING = 2


class Collective(enum.IntEnum):
    ALL_REDUCE = 0
    REDUCE_SCATTER = 1
    ALL_GATHER = 2
    ALL_TO_ALL = 3
    SCATTER = 4
    GATHER = 5
    BROADCAST = 6
    REDUCE2 = 7
    REDUCE = 8


MAX_RANKS = 16


class MegRayError(RuntimeError):
    """Raised where the reference throws MegRay::Exception or returns a non-OK Status."""

    def __init__(self, status, message):
        super().__init__(f"[{Status(status).name}] {message}")
        self.status = Status(status)
        self.message = message


def _check(status):
    if status != 0:
        raise MegRayError(status, _lib.load().mrv_last_error().decode())


def _ptr(buf):
    if buf is None:
        return None
    if hasattr(buf, "data_ptr"):
        return buf.data_ptr()
    return int(buf)


def _ptr_array(bufs):
    arr = (ctypes.c_void_p * len(bufs))()
    for i, b in enumerate(bufs):
        arr[i] = _ptr(b)
    return arr


def _rank_arrays(sendbuffs, recvbuffs, nranks=None):
    """The two per-rank pointer arrays of a flat call, both `nranks` long (the library indexes both up to
    nranks): lists of different lengths are rejected here, like any other invalid argument; a shorter list is
    allowed only where `nranks` says that its missing ranks are not used (root-only forms pad with None)."""
    n = nranks if nranks is not None else len(sendbuffs)
    if nranks is None and len(recvbuffs) != len(sendbuffs):
        raise MegRayError(Status.INVALID_ARGUMENT,
                          f"{len(sendbuffs)} send buffers but {len(recvbuffs)} receive buffers: one of each per rank")
    if len(sendbuffs) > n or len(recvbuffs) > n:
        raise MegRayError(Status.INVALID_ARGUMENT, f"more buffers than ranks ({n})")
    pad = lambda bufs: list(bufs) + [None] * (n - len(bufs))  # noqa: E731
    return _ptr_array(pad(sendbuffs)), _ptr_array(pad(recvbuffs)), n


def _stream(stream):
    if stream is None:
        return None
    if hasattr(stream, "cuda_stream"):
        return stream.cuda_stream
    return int(stream)


def get_dtype_size(dtype):
    """MegRay::get_dtype_size (src/core/common.cpp:19-38); raises 'unknown dtype'."""
    size = _lib.load().mrv_dtype_size(int(dtype))
    if size == 0:
        raise MegRayError(Status.INVALID_ARGUMENT, _lib.load().mrv_last_error().decode())
    return size


def reduce(i0, i1, o, length, dtype, op, stream=None):
    """o = i0 OP i1 (MegRay::reduce, src/ucx/utils.h:21-22)."""
    _check(_lib.load().mrv_reduce(_ptr(i0), _ptr(i1), _ptr(o), length, int(dtype), int(op), _stream(stream)))


def all_reduce(sendbuffs, recvbuffs, length, dtype, op, order=FoldOrder.UCX, schedule=Schedule.FUSED,
               stream=None):
    send, recv, nranks = _rank_arrays(sendbuffs, recvbuffs)
    _check(_lib.load().mrv_all_reduce(send, recv, nranks, length,
                                      int(dtype), int(op), int(order), int(schedule), _stream(stream)))


def reduce_scatter(sendbuffs, recvbuffs, recvlen, dtype, op, order=FoldOrder.UCX, stream=None):
    send, recv, nranks = _rank_arrays(sendbuffs, recvbuffs)
    _check(_lib.load().mrv_reduce_scatter(send, recv, nranks, recvlen,
                                          int(dtype), int(op), int(order), _stream(stream)))


def all_gather(sendbuffs, recvbuffs, sendlen, dtype, stream=None):
    send, recv, nranks = _rank_arrays(sendbuffs, recvbuffs)
    _check(_lib.load().mrv_all_gather(send, recv, nranks, sendlen,
                                      int(dtype), _stream(stream)))


def all_to_all(sendbuffs, recvbuffs, length, dtype, stream=None):
    send, recv, nranks = _rank_arrays(sendbuffs, recvbuffs)
    _check(_lib.load().mrv_all_to_all(send, recv, nranks, length,
                                      int(dtype), _stream(stream)))


def scatter(sendbuff_root, recvbuffs, recvlen, dtype, root, stream=None):
    _check(_lib.load().mrv_scatter(_ptr(sendbuff_root), _ptr_array(recvbuffs), len(recvbuffs), recvlen,
                                   int(dtype), root, _stream(stream)))


def gather(sendbuffs, recvbuff_root, sendlen, dtype, root, stream=None):
    _check(_lib.load().mrv_gather(_ptr_array(sendbuffs), _ptr(recvbuff_root), len(sendbuffs), sendlen,
                                  int(dtype), root, _stream(stream)))


def broadcast(sendbuff_root, recvbuffs, length, dtype, root, stream=None):
    _check(_lib.load().mrv_broadcast(_ptr(sendbuff_root), _ptr_array(recvbuffs), len(recvbuffs), length,
                                     int(dtype), root, _stream(stream)))


def reduce_to_root(sendbuffs, recvbuff_root, length, dtype, op, root, order=FoldOrder.UCX, stream=None):
    _check(_lib.load().mrv_reduce_to_root(_ptr_array(sendbuffs), _ptr(recvbuff_root), len(sendbuffs), length,
                                          int(dtype), int(op), int(order), root, _stream(stream)))


def probe_bounded_wait(limit_us, stream=None):
    """Launch one cross-stream wait that nothing will ever satisfy, with a time limit of `limit_us`; returns how
    many waits gave up (1).  mrv_probe_bounded_wait."""
    gave_up = ctypes.c_uint64(0)
    _check(_lib.load().mrv_probe_bounded_wait(int(limit_us), _stream(stream), ctypes.byref(gave_up)))
    return gave_up.value


def _written_array(written, count):
    if written is None:
        return None
    if len(written) != count:
        raise MegRayError(Status.INVALID_ARGUMENT, f"{count} buffers but {len(written)} written flags")
    return (ctypes.c_ubyte * max(count, 1))(*[1 if w else 0 for w in written])


def rank_buffers_layout(sizes, collective=None, written=None):
    """-> (offsets, total): where buffers of `sizes` bytes go inside one allocation so that a collective over them is
    served well by the memory system (buffers of 8 MiB and more an odd multiple of 128 MiB apart; with
    `collective` ALL_GATHER the buffers flagged in `written` a multiple of 128 MiB plus 32 MiB apart).
    mrv_rank_buffers_layout / mrv_rank_buffers_layout_for; needs no GPU."""
    count = len(sizes)
    arr = (ctypes.c_size_t * max(count, 1))(*[int(b) for b in sizes])
    offs = (ctypes.c_size_t * max(count, 1))()
    total = ctypes.c_size_t(0)
    if collective is None:
        _check(_lib.load().mrv_rank_buffers_layout(count, arr, offs, ctypes.byref(total)))
    else:
        _check(_lib.load().mrv_rank_buffers_layout_for(int(collective), count, arr, _written_array(written, count), offs,
                                                       ctypes.byref(total)))
    return list(offs)[:count], total.value


class RankBuffers:
    """Buffers of `sizes` bytes in one device allocation, placed by mrv_rank_buffers_alloc; `.ptrs` are their
    addresses.  free() (or the end of a with block) releases the allocation."""

    def __init__(self, sizes, collective=None, written=None):
        count = len(sizes)
        arr = (ctypes.c_size_t * max(count, 1))(*[int(b) for b in sizes])
        ptrs = (ctypes.c_void_p * max(count, 1))()
        base = ctypes.c_void_p(None)
        if collective is None:
            _check(_lib.load().mrv_rank_buffers_alloc(count, arr, ptrs, ctypes.byref(base)))
        else:
            _check(_lib.load().mrv_rank_buffers_alloc_for(int(collective), count, arr, _written_array(written, count),
                                                          ptrs, ctypes.byref(base)))
        self.ptrs = [int(p or 0) for p in ptrs][:count]
        self.sizes = [int(b) for b in sizes]
        self._base = base

    def free(self):
        if self._base is not None and self._base.value:
            _check(_lib.load().mrv_rank_buffers_free(self._base))
        self._base = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.free()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def place_tensors(torch, specs, device="cuda", collective=None, written=None):
    """Tensors of the given (numel, dtype) pairs as views into ONE torch allocation, placed by rank_buffers_layout:
    the way to hand torch-owned memory to a collective in the placement the library recommends (`collective` and
    `written` as for rank_buffers_layout).  The views keep the allocation alive."""
    sizes = [int(numel) * torch.empty((), dtype=dtype).element_size() for numel, dtype in specs]
    offsets, total = rank_buffers_layout(sizes, collective, written)
    align = 2 << 20
    arena = torch.empty(total + align, dtype=torch.uint8, device=device)
    skew = (-arena.data_ptr()) % align
    return [arena[skew + off:skew + off + size].view(dtype) for off, size, (_, dtype) in zip(offsets, sizes, specs)]


def chunk_partition(length, nchunks):
    sizes = (ctypes.c_size_t * nchunks)()
    offs = (ctypes.c_size_t * nchunks)()
    _check(_lib.load().mrv_chunk_partition(length, nchunks, sizes, offs))
    return list(sizes), list(offs)


def fold_order(collective, order, nranks, chunk):
    """-> (ranks, new_wins_ties, nchunks, owner)"""
    ranks = (ctypes.c_uint32 * max(nranks, 1))()
    new_wins = ctypes.c_int(0)
    nchunks = ctypes.c_uint32(0)
    owner = ctypes.c_uint32(0)
    _check(_lib.load().mrv_fold_order(int(collective), int(order), nranks, chunk, ranks, ctypes.byref(new_wins),
                                      ctypes.byref(nchunks), ctypes.byref(owner)))
    return list(ranks)[:nranks], bool(new_wins.value), nchunks.value, owner.value


def describe(collective, sendptrs, recvptrs, count, dtype, order=FoldOrder.UCX, schedule=Schedule.FUSED,
             root=0, nranks=None):
    """Plan a collective on the host only.  -> (list of run dicts, bytes_read, bytes_written)"""
    nranks = nranks if nranks is not None else max(len(sendptrs), len(recvptrs))
    send, recv, nranks = _rank_arrays(sendptrs, recvptrs, nranks)
    cap = 4096
    runs = (_lib.PlanRun * cap)()
    n = ctypes.c_size_t(0)
    br = ctypes.c_uint64(0)
    bw = ctypes.c_uint64(0)
    _check(_lib.load().mrv_describe(int(collective), send, recv, nranks, count,
                                    int(dtype), int(order), int(schedule), root, runs, cap, ctypes.byref(n),
                                    ctypes.byref(br), ctypes.byref(bw)))
    out = []
    for i in range(min(n.value, cap)):
        r = runs[i]
        out.append({name: getattr(r, name) for name, _ in _lib.PlanRun._fields_})
    return out, br.value, bw.value


class CollectivePlan:
    """A collective planned once and launched many times (mrv_plan_*).  `graph=True` instantiates
    the launches of a multi-launch plan as one HIP graph.  The buffers must outlive the plan."""

    def __init__(self, collective, sendbuffs, recvbuffs, count, dtype, op=ReduceOp.SUM, order=FoldOrder.UCX,
                 schedule=Schedule.FUSED, root=0, graph=False, nranks=None):
        self._h = ctypes.c_void_p()
        self._keep = (sendbuffs, recvbuffs)
        nranks = nranks if nranks is not None else max(len(sendbuffs), len(recvbuffs))
        send, recv, nranks = _rank_arrays(sendbuffs, recvbuffs, nranks)
        _check(_lib.load().mrv_plan_create(int(collective), send, recv, nranks,
                                           count, int(dtype), int(op), int(order), int(schedule), root,
                                           1 if graph else 0, ctypes.byref(self._h)))
        self._launch = _lib.load().mrv_plan_launch

    @property
    def launch_count(self):
        return _lib.load().mrv_plan_launch_count(self._h)

    def launch(self, stream=None):
        status = self._launch(self._h, _stream(stream))
        if status:
            _check(status)

    def close(self):
        if self._h:
            _lib.load().mrv_plan_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # at interpreter shutdown the modules this needs may be gone already
            pass


# ---------------------------------------------------------------------------------------------
# the Communicator API, one object per rank (include/megray/communicator.h:32-123)

def get_free_port():
    """MegRay::get_free_port (include/megray/server.h:21)."""
    port = _lib.load().mrv_get_free_port()
    if port <= 0:
        raise MegRayError(Status.SYS_ERROR, _lib.load().mrv_last_error().decode())
    return port


def create_server(nranks, port):
    """MegRay::create_server (include/megray/server.h:24)."""
    _check(_lib.load().mrv_create_server(nranks, port))


class Client:
    """MegRay::Client (include/megray/client.h:24-49): host-side barrier / broadcast / allgather."""

    def __init__(self, nranks, rank):
        self._h = ctypes.c_void_p()
        self.nranks = nranks
        _check(_lib.load().mrv_client_create(nranks, rank, ctypes.byref(self._h)))

    def connect(self, master_ip, port):
        _check(_lib.load().mrv_client_connect(self._h, master_ip.encode(), port))

    def barrier(self):
        _check(_lib.load().mrv_client_barrier(self._h))

    def broadcast(self, data, root, is_root):
        """data: bytes on the root (any bytes-like of the same length elsewhere) -> bytes"""
        out = ctypes.create_string_buffer(len(data))
        src = ctypes.create_string_buffer(bytes(data), len(data)) if is_root else None
        _check(_lib.load().mrv_client_broadcast(self._h, src, out, len(data), root))
        return out.raw

    def allgather(self, data):
        out = ctypes.create_string_buffer(len(data) * self.nranks)
        src = ctypes.create_string_buffer(bytes(data), len(data))
        _check(_lib.load().mrv_client_allgather(self._h, src, out, len(data)))
        return out.raw

    def close(self):
        if self._h:
            _lib.load().mrv_client_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # at interpreter shutdown the modules this needs may be gone already
            pass


class Communicator:
    """One rank's communicator, as returned by MegRay::get_communicator (include/megray.h:33-34).

    Every method takes the device pointers of THIS rank and an optional stream, and must be called
    from this rank's own thread; it returns when all ranks of the group have made the same call
    and the work is enqueued.
    """

    def __init__(self, nranks, rank, backend=Backend.VRANK):
        self._h = ctypes.c_void_p()
        self.nranks, self.rank = nranks, rank
        _check(_lib.load().mrv_comm_create(nranks, rank, int(backend), ctypes.byref(self._h)))

    def init(self, master_ip, port):
        _check(_lib.load().mrv_comm_init(self._h, master_ip.encode(), port))

    def init_callback(self, broadcast):
        """Communicator::init(BcastCallback) (include/megray/communicator.h:49): form the group through the
        caller's own broadcast instead of the bootstrap server.  `broadcast(data: bytearray) -> bytes-like` is
        called once on this rank's thread with this rank's bytes (meaningful on rank 0 only) and returns rank 0's."""
        def trampoline(data, length, _user):
            mine = ctypes.string_at(data, length)
            got = bytes(broadcast(bytearray(mine)))
            if len(got) != length:
                raise ValueError(f"the broadcast returned {len(got)} bytes, {length} were handed in")
            ctypes.memmove(data, got, length)
        fn = _lib.BCAST_FN(trampoline)
        _check(_lib.load().mrv_comm_init_callback(self._h, fn, None))

    def check(self, stream=None):
        """Raises if a stream wait of this rank's group has given up (mrv_comm_check; synchronous)."""
        _check(_lib.load().mrv_comm_check(self._h, _stream(stream)))

    def stats(self):
        """{"collectives", "plans_built", "sleeps"} of this rank's group since it was formed (mrv_comm_stats)."""
        c, p, s = ctypes.c_uint64(0), ctypes.c_uint64(0), ctypes.c_uint64(0)
        _check(_lib.load().mrv_comm_stats(self._h, ctypes.byref(c), ctypes.byref(p), ctypes.byref(s)))
        return {"collectives": c.value, "plans_built": p.value, "sleeps": s.value}

    def configure(self, order=FoldOrder.UCX, schedule=Schedule.FUSED):
        _check(_lib.load().mrv_comm_configure(self._h, int(order), int(schedule)))

    def send(self, sendbuff, length, dtype, rank, stream=None):
        _check(_lib.load().mrv_comm_send(self._h, _ptr(sendbuff), length, int(dtype), rank, _stream(stream)))

    def recv(self, recvbuff, length, dtype, rank, stream=None):
        _check(_lib.load().mrv_comm_recv(self._h, _ptr(recvbuff), length, int(dtype), rank, _stream(stream)))

    def scatter(self, sendbuff, recvbuff, recvlen, dtype, root, stream=None):
        _check(_lib.load().mrv_comm_scatter(self._h, _ptr(sendbuff), _ptr(recvbuff), recvlen, int(dtype), root,
                                            _stream(stream)))

    def gather(self, sendbuff, recvbuff, sendlen, dtype, root, stream=None):
        _check(_lib.load().mrv_comm_gather(self._h, _ptr(sendbuff), _ptr(recvbuff), sendlen, int(dtype), root,
                                           _stream(stream)))

    def all_to_all(self, sendbuff, recvbuff, length, dtype, stream=None):
        _check(_lib.load().mrv_comm_all_to_all(self._h, _ptr(sendbuff), _ptr(recvbuff), length, int(dtype),
                                               _stream(stream)))

    def all_gather(self, sendbuff, recvbuff, sendlen, dtype, stream=None):
        _check(_lib.load().mrv_comm_all_gather(self._h, _ptr(sendbuff), _ptr(recvbuff), sendlen, int(dtype),
                                               _stream(stream)))

    def all_reduce(self, sendbuff, recvbuff, length, dtype, op, stream=None):
        _check(_lib.load().mrv_comm_all_reduce(self._h, _ptr(sendbuff), _ptr(recvbuff), length, int(dtype),
                                               int(op), _stream(stream)))

    def all_reduce_no_alloc(self, sendbuff, recvbuff, length, dtype, op, stream=None):
        """all_reduce for callers that may not allocate device memory: the counters that order the ranks'
        streams are a block of the library's static device array (mrv_comm_all_reduce_no_alloc)."""
        _check(_lib.load().mrv_comm_all_reduce_no_alloc(self._h, _ptr(sendbuff), _ptr(recvbuff), length, int(dtype),
                                                        int(op), _stream(stream)))

    def reduce_scatter(self, sendbuff, recvbuff, recvlen, dtype, op, stream=None):
        _check(_lib.load().mrv_comm_reduce_scatter(self._h, _ptr(sendbuff), _ptr(recvbuff), recvlen, int(dtype),
                                                   int(op), _stream(stream)))

    def broadcast(self, sendbuff, recvbuff, length, dtype, root, stream=None):
        _check(_lib.load().mrv_comm_broadcast(self._h, _ptr(sendbuff), _ptr(recvbuff), length, int(dtype), root,
                                              _stream(stream)))

    def reduce(self, sendbuff, recvbuff, length, dtype, op, root, stream=None):
        _check(_lib.load().mrv_comm_reduce(self._h, _ptr(sendbuff), _ptr(recvbuff), length, int(dtype), int(op),
                                           root, _stream(stream)))

    def group_start(self):
        _check(_lib.load().mrv_comm_group_start(self._h))

    def group_end(self):
        _check(_lib.load().mrv_comm_group_end(self._h))

    def close(self):
        if self._h:
            _lib.load().mrv_comm_destroy(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:  # at interpreter shutdown the modules this needs may be gone already
            pass


def get_communicator(nranks, rank, backend=Backend.VRANK):
    """MegRay::get_communicator (include/megray.h:33-34); raises 'unknown backend' like src/megray.cpp:56-57."""
    return Communicator(nranks, rank, backend)
