/*
 * megray_vrank.h -- C ABI of the MI355X virtual-rank MegRay library (libmegray_vrank.so).
 *
 * The library's C++ face is MegRay's own API (megray.h: get_communicator, Communicator,
 * HipContext).  This header is the flat, language-neutral face of the same code: plain pointers,
 * sizes and integers, no C++ or torch types.  It is what a foreign-function binding (ctypes, cgo,
 * JNI ...) or a single-threaded benchmark driver calls.
 *
 * Conventions
 *   - dtype / op / status integers carry the numeric values of MegRay::DType, MegRay::ReduceOp and
 *     MegRay::Status (include/megray/common.h:23-37,106-127 of the reference).
 *   - every buffer pointer is device memory of the current HIP device; `stream` is a hipStream_t
 *     passed as void* (NULL = the default stream).  Calls enqueue work and return; results are
 *     ready when the stream reaches that point.
 *   - "rank" arrays have `nranks` entries, entry r belonging to virtual rank r.  Lengths are
 *     element counts with the meaning of the reference's Communicator comments
 *     (include/megray/communicator.h:63-101).
 *   - where the reference throws MegRay::Exception (unknown dtype / op, wrong context ...) these
 *     functions return MEGRAY_INVALID_ARGUMENT (6) and keep the message for mrv_last_error().
 */
#ifndef MEGRAY_VRANK_H
#define MEGRAY_VRANK_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MRV_API __attribute__((visibility("default")))

#define MRV_MAX_RANKS 32

/* Which reference loop fixes the order a chunk's contributions are combined in. */
enum {
    MRV_ORDER_UCX = 0,   /* src/ucx/all_reduce.cpp:61-82, src/ucx/reduce_scatter.cpp:44-53 */
    MRV_ORDER_SHM = 1,   /* src/shm/all_reduce.cpp:38-127 + src/shm/communicator.cpp:24-75 */
    MRV_ORDER_RANK0 = 2  /* ranks 0..N-1 for every element, test/test_opr.cpp:321-330 */
};

/* How the collective is laid out in kernel launches. */
enum {
    MRV_SCHED_FUSED = 0,     /* one launch: N reads, all destinations written */
    MRV_SCHED_TWO_PHASE = 1, /* reduce-scatter launch + broadcast-copy launch */
    MRV_SCHED_RING = 2       /* the reference's 2(N-1) two-input ring steps, one launch each */
};

/* Collective selector of mrv_describe(). */
enum {
    MRV_ALL_REDUCE = 0,
    MRV_REDUCE_SCATTER = 1,
    MRV_ALL_GATHER = 2,
    MRV_ALL_TO_ALL = 3,
    MRV_SCATTER = 4,
    MRV_GATHER = 5,
    MRV_BROADCAST = 6,
    MRV_REDUCE2 = 7,
    MRV_REDUCE = 8
};

/* ---- library ------------------------------------------------------------------------------ */

/* Bumped when a signature below changes. */
MRV_API int mrv_abi_version(void);

/* Message of the last call on this thread that returned a non-zero status ("" if none). */
MRV_API const char* mrv_last_error(void);

/* MegRay::get_dtype_size (src/core/common.cpp:19-38); 0 where the reference throws "unknown dtype". */
MRV_API size_t mrv_dtype_size(int dtype);

/* ---- the hot path on the current device ---------------------------------------------------- */

/*
 * o[i] = i0[i] OP i1[i], MAX/MIN keeping i1 on equal / unordered operands.
 * Replaces MegRay::reduce(i0, i1, o, len, dtype, op, stream) (src/ucx/utils.h:21-22,
 * src/ucx/kernel.cu:60-98) and MegRay::cpu_reduce (src/shm/utils.h:32).  FLOAT16 is accepted
 * (fp32 arithmetic, one rounding); CHAR is rejected like the reference ("unknown dtype").
 */
MRV_API int mrv_reduce(const void* i0, const void* i1, void* o, size_t len, int dtype, int op,
                       void* stream);

/*
 * recvbuffs[r][0..len) = fold over ranks of sendbuffs[*][0..len), for every r.
 * Replaces UcxCommunicator::all_reduce (src/ucx/all_reduce.cpp:23-109) and
 * ShmCommunicator::_shm_all_reduce (src/shm/all_reduce.cpp:38-127) run on all N ranks.
 * recvbuffs[r] may equal sendbuffs[r].
 */
MRV_API int mrv_all_reduce(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                           size_t len, int dtype, int op, int order, int schedule, void* stream);

/*
 * recvbuffs[r][0..recvlen) = fold over ranks of sendbuffs[*][r*recvlen .. (r+1)*recvlen).
 * Replaces UcxCommunicator::reduce_scatter (src/ucx/reduce_scatter.cpp:21-61) and
 * ShmCommunicator::_shm_reduce_scatter (src/shm/reduce_scatter.cpp:21-97).
 */
MRV_API int mrv_reduce_scatter(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                               size_t recvlen, int dtype, int op, int order, void* stream);

/*
 * recvbuffs[k][i*sendlen + j] = sendbuffs[i][j] for every k.
 * Replaces UcxCommunicator::all_gather (src/ucx/all_gather.cpp:21-63) and _shm_all_gather
 * (src/shm/all_gather.cpp:28-55).
 */
MRV_API int mrv_all_gather(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                           size_t sendlen, int dtype, void* stream);

/*
 * recvbuffs[j][i*len + k] = sendbuffs[i][j*len + k].
 * Replaces UcxCommunicator::all_to_all (src/ucx/all_to_all.cpp:21-43) and _shm_all_to_all
 * (src/shm/all_to_all.cpp:18-59).
 */
MRV_API int mrv_all_to_all(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                           size_t len, int dtype, void* stream);

/*
 * recvbuffs[i][j] = sendbuff_root[i*recvlen + j].
 * Replaces UcxCommunicator::scatter (src/ucx/scatter.cpp:21-46), ShmCommunicator::scatter
 * (src/shm/scatter.cpp:21-42).
 */
MRV_API int mrv_scatter(const void* sendbuff_root, void* const* recvbuffs, uint32_t nranks,
                        size_t recvlen, int dtype, uint32_t root, void* stream);

/*
 * recvbuff_root[i*sendlen + j] = sendbuffs[i][j].
 * Replaces UcxCommunicator::gather (src/ucx/gather.cpp:21-46), _shm_gather (src/shm/gather.cpp:19-49).
 */
MRV_API int mrv_gather(const void* const* sendbuffs, void* recvbuff_root, uint32_t nranks,
                       size_t sendlen, int dtype, uint32_t root, void* stream);

/*
 * recvbuffs[r][j] = sendbuff_root[j] for every r.
 * Replaces UcxCommunicator::broadcast (src/ucx/broadcast.cpp:21-76), ShmCommunicator::broadcast
 * (src/shm/broadcast.cpp:19-51).
 */
MRV_API int mrv_broadcast(const void* sendbuff_root, void* const* recvbuffs, uint32_t nranks,
                          size_t len, int dtype, uint32_t root, void* stream);

/* ---- host-side planning, no device access -------------------------------------------------- */

/* len/C split with the remainder on the first chunks (src/ucx/all_reduce.cpp:33-38,48-51). */
MRV_API int mrv_chunk_partition(size_t len, uint32_t nchunks, size_t* sizes, size_t* offsets);

/*
 * Fold order of chunk `chunk` for `collective` (MRV_ALL_REDUCE or MRV_REDUCE_SCATTER): ranks[0]
 * seeds the accumulator.  *new_wins_ties: MAX/MIN keep the newcomer on equal / unordered operands.
 * *nchunks: number of chunks the order splits the buffer into.  *owner: rank the ring leaves the
 * finished chunk on.
 */
MRV_API int mrv_fold_order(int collective, int order, uint32_t nranks, uint32_t chunk, uint32_t* ranks,
                           int* new_wins_ties, uint32_t* nchunks, uint32_t* owner);

/* One run of a planned launch, as mrv_describe() reports it. */
typedef struct mrv_plan_run {
    uint32_t step;          /* launch index within the collective */
    uint32_t kind;          /* 0 = fold run, 1 = block copy of a pack launch */
    uint32_t nfold;         /* fold: inputs combined per element (1 = copy) */
    uint32_t nout;          /* destinations: ranks out_first .. out_first + nout - 1 (mod nranks) */
    uint32_t new_wins_ties; /* fold */
    uint32_t vector;        /* fold: 0 = element by element, 1 = 16-byte vectors, 2 = run of a flat launch
                               (vectors on the buffer's own 1 KiB tile grid); pack: what every block address and the
                               block size are a multiple of (16, 8, 4, 2 or 1; lanes move 16 bytes whichever it is) */
    uint32_t start;         /* fold: seed rank; pack: source rank */
    int32_t dir;            /* fold: +1 / -1; 0 = binomial tree towards rank `start` */
    uint32_t out_first;     /* fold: first destination rank; pack: destination rank */
    uint32_t tiles;         /* workgroups this run occupies (flat: those wholly inside it) */
    uint32_t reads_recv;    /* 1 = the launch reads the receive buffers (a later step of a multi-launch plan) */
    uint32_t waves;         /* wavefronts per workgroup of the launch (4: the group form, four tiles per workgroup) */
    uint64_t in_begin;      /* fold: first element in the inputs; pack: source byte offset */
    uint64_t out_begin;     /* fold: first element in the outputs; pack: destination byte offset */
    uint64_t count;         /* fold: elements; pack: bytes */
    uint32_t deal;          /* fold, group form: 1 = the run's tiles share cache lines with their neighbours, so runs of
                               workgroups are dealt to one XCD (one L2) each; pack decides this per copy on the device */
    uint32_t paced;         /* group form: 1 = the launch spaces its accesses out (a wavefront keeps two loads and two stores in
                               flight; a pack launch issues a wavefront's stores one at a time): long launches, see vrank_plan.cpp */
    uint32_t keep;          /* 1 = the launch's stores leave their data in the last-level cache (collectives that write 128 MiB
                               or less); 0 = they stream past the caches */
    uint32_t reserved;
} mrv_plan_run;

/*
 * Plans `collective` exactly as the device entry points do, without touching a device, and writes
 * up to `cap` runs.  Pointers are only inspected for alignment and aliasing.  For MRV_SCATTER /
 * MRV_BROADCAST only sendbuffs[root] is read from the send array, for MRV_GATHER only
 * recvbuffs[root]; for MRV_REDUCE2 sendbuffs = {i0, i1}, recvbuffs = {o}.
 * *nruns receives the number of runs the plan has (which may exceed cap), *bytes_read /
 * *bytes_written the algorithmic HBM bytes of the whole plan.
 */
MRV_API int mrv_describe(int collective, const void* const* sendbuffs, void* const* recvbuffs,
                         uint32_t nranks, size_t count, int dtype, int order, int schedule, uint32_t root,
                         mrv_plan_run* runs, size_t cap, size_t* nruns, uint64_t* bytes_read,
                         uint64_t* bytes_written);

/* ---- planned collectives: plan once, launch many times ------------------------------------- */

/*
 * A training loop repeats the same collective on the same buffers.  mrv_plan_create does the
 * host-side planning once (no reference counterpart: the reference re-derives chunk sizes and
 * re-allocates its workspace on every call, src/ucx/all_reduce.cpp:33-51); mrv_plan_launch then
 * only enqueues the prepared launches.  With MRV_PLAN_GRAPH the launches of a multi-launch plan
 * (two-phase, ring) are additionally instantiated as one HIP graph of kernel nodes and replayed
 * with a single hipGraphLaunch.
 * `collective` is one of the MRV_* selectors, arguments as for mrv_describe; `op` is ignored by the
 * copy collectives.  The buffers must stay valid and unchanged in address until mrv_plan_destroy.
 */
typedef struct mrv_plan mrv_plan;
#define MRV_PLAN_GRAPH 1u
MRV_API int mrv_plan_create(int collective, const void* const* sendbuffs, void* const* recvbuffs,
                            uint32_t nranks, size_t count, int dtype, int op, int order, int schedule,
                            uint32_t root, uint32_t flags, mrv_plan** plan);
MRV_API int mrv_plan_launch(const mrv_plan* plan, void* stream);
/* number of kernel launches one mrv_plan_launch stands for */
MRV_API size_t mrv_plan_launch_count(const mrv_plan* plan);
MRV_API void mrv_plan_destroy(mrv_plan* plan);

/* ---- the MegRay::Communicator API, one handle per rank ------------------------------------- */

/*
 * These bind the C++ API one to one for callers that cannot link C++: a handle owns the
 * std::shared_ptr<MegRay::Communicator> that MegRay::get_communicator returns
 * (include/megray.h:33-34), every call wraps `stream` in a MegRay::HipContext
 * (include/megray/hip_context.h:43-54) and forwards to the virtual of the same name
 * (include/megray/communicator.h:60-109).  As with the C++ API, each rank's calls come from its own
 * thread and every rank of a group makes the same calls in the same order; a collective returns
 * once all ranks have arrived and the work is enqueued.
 */
typedef struct mrv_comm mrv_comm;

/* MegRay::get_free_port / MegRay::create_server (include/megray/server.h:19-24). */
MRV_API int mrv_get_free_port(void);
MRV_API int mrv_create_server(uint32_t nranks, int port);

/* get_communicator(nranks, rank, backend); backend 4 = MEGRAY_VRANK, anything else: "unknown backend". */
MRV_API int mrv_comm_create(uint32_t nranks, uint32_t rank, int backend, mrv_comm** comm);
MRV_API void mrv_comm_destroy(mrv_comm* comm);
/* Communicator::init(master_ip, port) (src/core/communicator.cpp:17-21). */
MRV_API int mrv_comm_init(mrv_comm* comm, const char* master_ip, int port);
/*
 * Communicator::init(BcastCallback) (include/megray/communicator.h:49, src/core/communicator.cpp:23-25): the group
 * is formed through a broadcast the CALLER supplies instead of the bootstrap server, the way the reference's NCCL
 * backend hands its unique id to one (src/nccl/communicator.cpp:54-64).  Every rank calls this from its own thread;
 * `broadcast(data, len, user)` must leave rank 0's `len` bytes of `data` in every rank's `data` before it returns
 * (rank 0 passes its own bytes in, the others receive).  `len` is 16 for this backend (the group's id).
 */
typedef void (*mrv_bcast_fn)(char* data, size_t len, void* user);
MRV_API int mrv_comm_init_callback(mrv_comm* comm, mrv_bcast_fn broadcast, void* user);
/*
 * No counterpart in the reference (whose ranks block the host at every step and cannot run ahead of a peer).
 * Here a rank's stream waits for its peers' streams on the device, and such a wait gives up after
 * MEGRAY_VRANK_WAIT_LIMIT_MS (default 10 000).  A wait that gives up poisons its group: the kernels behind it
 * store nothing, and every later call of the group returns MEGRAY_UNEXPECTED_ERR.  This call asks now: it waits
 * for `stream`, reads the group's counters back and returns MEGRAY_OK or, for good, MEGRAY_UNEXPECTED_ERR.
 */
MRV_API int mrv_comm_check(mrv_comm* comm, void* stream);
/*
 * Diagnostic, no counterpart in the reference: counts kept by this rank's group since it was formed (any pointer may
 * be null).  *collectives: collectives launched; *plans_built: how many of them had to be planned rather than found in
 * the group's plan cache; *sleeps: times a rank waiting for the others stopped polling and slept on a condition
 * variable.
 */
MRV_API int mrv_comm_stats(mrv_comm* comm, uint64_t* collectives, uint64_t* plans_built, uint64_t* sleeps);
/* Fold order / schedule of this rank's communicator (MRV_ORDER_*, MRV_SCHED_*); no reference counterpart. */
MRV_API int mrv_comm_configure(mrv_comm* comm, int order, int schedule);

/* Communicator::send / recv (include/megray/communicator.h:51-57): `len` elements of `dtype` to / from rank `rank`.
 * A send and the matching receive become one block copy between the two ranks' buffers, enqueued on the receiver's
 * stream behind everything the sender's stream held at the send; the sender's stream goes on when the copy is done.
 * Outside mrv_comm_group_start / _end a call returns when its counterpart has been posted and the copy is enqueued. */
MRV_API int mrv_comm_send(mrv_comm* comm, const void* sendbuff, size_t len, int dtype, uint32_t rank,
                          void* stream);
MRV_API int mrv_comm_recv(mrv_comm* comm, void* recvbuff, size_t len, int dtype, uint32_t rank, void* stream);
MRV_API int mrv_comm_scatter(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t recvlen, int dtype,
                             uint32_t root, void* stream);
MRV_API int mrv_comm_gather(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t sendlen, int dtype,
                            uint32_t root, void* stream);
MRV_API int mrv_comm_all_to_all(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype,
                                void* stream);
MRV_API int mrv_comm_all_gather(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t sendlen,
                                int dtype, void* stream);
MRV_API int mrv_comm_all_reduce(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype,
                                int op, void* stream);
/*
 * mrv_comm_all_reduce for callers that cannot allocate device memory (harnesses that forbid
 * hipMalloc, tight serving loops).  No counterpart in the reference.  Same arguments, same result
 * bit for bit.  mrv_comm_all_reduce orders the ranks' streams through counters it allocates at the
 * group's first collective (hipMalloc + hipHostMalloc), or through events; this entry point keeps
 * the counters in a 2 KiB array that is part of the library's device code (every GPU the library
 * runs on holds its copy until the process ends), cut into 32 blocks of 64 bytes, one per
 * communicator group.  It calls no hipMalloc / hipFree / hipHostMalloc / hipEventCreate.
 *   - at most 32 groups per process can use it at the same time; the 33rd gets
 *     MEGRAY_INVALID_USAGE ("every counter block of the static array is in use") on every rank;
 *   - a group's first call clears its block (a 64-byte fill on the null stream, waited for): a block keeps what
 *     the last group that held it left there;
 *   - every rank of a group must make this same call (mixing it with mrv_comm_all_reduce in one
 *     collective is rejected like any other mismatch); a group's collectives follow one another, so
 *     its block is never used by two calls at once, and groups do not share blocks;
 *   - a stream wait that gives up (see mrv_comm_check) stops the kernels behind it from storing, as everywhere;
 *     but with no pinned host word to report to, the host finds out by reading the block back: a synchronous
 *     64-byte copy behind `stream` once half the wait limit has passed since the last one (never under stream
 *     capture), so the first call that fails comes up to one and a half limits after the wait gave up, not at
 *     the very next call; mrv_comm_check and the group's teardown read it as well.
 */
MRV_API int mrv_comm_all_reduce_no_alloc(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len,
                                         int dtype, int op, void* stream);
MRV_API int mrv_comm_reduce_scatter(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t recvlen,
                                    int dtype, int op, void* stream);
MRV_API int mrv_comm_broadcast(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype,
                               uint32_t root, void* stream);
MRV_API int mrv_comm_reduce(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype, int op,
                            uint32_t root, void* stream);
/*
 * Diagnostic, no counterpart in the reference.  The kernels that make one stream wait for another
 * (thread-per-rank API with a stream per rank) give up after a time limit instead of spinning for
 * ever.  This launches one such wait on `stream` for a count that nothing ever raises, with a limit
 * of `limit_us` microseconds, waits for the stream, and returns how many waits gave up (1) in
 * *gave_up: a way to see, from the host and without hanging anything, that the limit works.
 */
MRV_API int mrv_probe_bounded_wait(uint64_t limit_us, void* stream, uint64_t* gave_up);

/*
 * Placement of the ranks' buffers in HBM.  No counterpart in the reference, whose ranks are devices and allocate
 * their own buffers (test/performance.cpp:108-110, test/test_base.h:57-66); optional: every entry point of this
 * library takes buffers from anywhere.
 *
 * A collective touches the same offset of up to 2N buffers at the same time, and the memory system derives channel
 * and bank from address bits: buffers whose starts differ by a multiple of a large power of two (what separate
 * allocations of a power-of-two size give) are served 6 - 10 points of the HBM peak slower than buffers an odd
 * multiple of 128 MiB apart (8-rank fp32 all_reduce, 1 GiB per rank: 75 - 78 % against 84 %; 16 MiB per rank: 66 %
 * against 78 %).  These calls lay `count` buffers of bytes[i] bytes out in ONE allocation accordingly: buffers of
 * 8 MiB and more start an odd multiple of 128 MiB after the one before, smaller ones (they live in the caches) at
 * the next 2 MiB or 4 KiB boundary.  Pass the buffers of one collective together, inputs and outputs, in any order.
 *
 * mrv_rank_buffers_layout  only computes: offsets[i] from a common base (2 MiB aligned or better) and *total, the
 *                          bytes to allocate, for callers with an allocator of their own.  Needs no GPU.
 * mrv_rank_buffers_alloc   allocates (hipMalloc) and returns the addresses in ptrs[0..count) and the allocation in
 *                          *base; mrv_rank_buffers_free(base) releases it (null is allowed).
 */
MRV_API int mrv_rank_buffers_layout(int count, const size_t* bytes, size_t* offsets, size_t* total);
MRV_API int mrv_rank_buffers_alloc(int count, const size_t* bytes, void** ptrs, void** base);
MRV_API int mrv_rank_buffers_free(void* base);
/*
 * The same for callers that know what the buffers are for (no counterpart in the reference either).  The best
 * distance depends on it: the buffers an all_gather stores every rank's block into (one read stream, N write
 * streams) are served best a multiple of 128 MiB PLUS 32 MiB apart (all_gather of 8 x 16 MiB fp16: 79 % of the HBM
 * peak with the outputs 128 MiB apart, 84 % at 160 MiB), where the folds and the pairwise copies lose one to two
 * points at such distances and a broadcast does not care.  `collective` is one of the MRV_* selectors (or -1: no
 * particular use, as above); written[i] != 0 marks the buffers the collective writes (null: none).  For every
 * collective but MRV_ALL_GATHER the result is that of the calls above.
 */
MRV_API int mrv_rank_buffers_layout_for(int collective, int count, const size_t* bytes, const unsigned char* written,
                                        size_t* offsets, size_t* total);
MRV_API int mrv_rank_buffers_alloc_for(int collective, int count, const size_t* bytes, const unsigned char* written,
                                       void** ptrs, void** base);
MRV_API int mrv_comm_group_start(mrv_comm* comm);
MRV_API int mrv_comm_group_end(mrv_comm* comm);

/* recv_root = combination of sendbuffs[*] for rank `root`, all ranks' buffers at once.
 * Replaces UcxCommunicator::reduce (src/ucx/reduce.cpp:21-87: binomial tree, MRV_ORDER_UCX) and
 * ShmCommunicator reduce (src/shm/reduce.cpp:21-100: MRV_ORDER_SHM). */
MRV_API int mrv_reduce_to_root(const void* const* sendbuffs, void* recvbuff_root, uint32_t nranks, size_t len,
                               int dtype, int op, int order, uint32_t root, void* stream);

/* The bootstrap client (include/megray/client.h:24-49), host memory only. */
typedef struct mrv_client mrv_client;
MRV_API int mrv_client_create(uint32_t nranks, uint32_t rank, mrv_client** client);
MRV_API void mrv_client_destroy(mrv_client* client);
MRV_API int mrv_client_connect(mrv_client* client, const char* master_ip, int port);
MRV_API int mrv_client_barrier(mrv_client* client);
MRV_API int mrv_client_broadcast(mrv_client* client, const void* sendbuff, void* recvbuff, size_t len,
                                 uint32_t root);
MRV_API int mrv_client_allgather(mrv_client* client, const void* sendbuff, void* recvbuff, size_t sendlen);

#ifdef __cplusplus
}
#endif
#endif /* MEGRAY_VRANK_H */
