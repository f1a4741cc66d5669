/*
 * megray_oracle.h -- CPU restatement of MegRay's ring reduce / pack path.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker the HIP path is
 * compared against (tests, the smoke check, the CPU-baseline leg of the
 * benchmark).  Nothing that ships may call it: the product library never links
 * or loads it and has no CPU fallback.
 *
 * Citations are into the reference tree (MegEngine/MegRay), path:line.
 *
 * Pinning status (what independent evidence fixes each function's result):
 *   orc_dtype_size            table in src/core/common.cpp:19-38, checked value by value.
 *   orc_reduce_ucx/_shm       textbook two's-complement / IEEE-754 arithmetic, checked against
 *                             numpy on every (a,b) byte pair for int8/uint8 and on random and
 *                             special values (+-0, NaN, inf, denormals) for the wider types.
 *   orc_chunk_partition       exhaustive enumeration N<=9, len<=64 (tiles [0,len), sizes differ
 *                             by <=1, larger first).
 *   orc_ucx_* / orc_shm_*     literal replays of the cited loops; checked against the closed-form
 *                             expectations the reference's own tests hold (test/test_opr.cpp),
 *                             against numpy on integers (order independent), and their fold
 *                             order is extracted with the tracing reduce (orc_trace_reduce2).
 *   orc_fold_*                per-chunk folds in the order orc_fold_order reports; must equal the
 *                             literal replays bit for bit on every dtype the reference supports.
 *   FLOAT16                   PARITY UNPINNED BY THE REFERENCE: neither reference reduce
 *                             (src/ucx/kernel.cu:60-98, src/shm/utils.cpp:39-69) accepts FLOAT16.
 *                             Defined here as: convert to fp32, fold in the chunk's order in
 *                             fp32, round once to binary16 (RNE).  The conversions are checked
 *                             on all 65536 bit patterns against numpy.float16.
 */
#ifndef MEGRAY_ORACLE_H
#define MEGRAY_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* numeric values of include/megray/common.h:106-127 */
enum {
    ORC_INT8 = 0, ORC_UINT8 = 1, ORC_INT32 = 2, ORC_UINT32 = 3, ORC_INT64 = 4,
    ORC_UINT64 = 5, ORC_FLOAT16 = 6, ORC_FLOAT32 = 7, ORC_FLOAT64 = 8, ORC_CHAR = 9
};
enum { ORC_SUM = 0, ORC_MAX = 1, ORC_MIN = 2 };

/* fold orders */
enum {
    ORC_ORDER_UCX = 0,  /* src/ucx/all_reduce.cpp:61-82, src/ucx/reduce_scatter.cpp:44-53 */
    ORC_ORDER_SHM = 1,  /* src/shm/all_reduce.cpp:38-127 + src/shm/communicator.cpp:24-75 */
    ORC_ORDER_RANK0 = 2 /* test/test_opr.cpp:321-330: ranks 0..N-1 for every element */
};
enum { ORC_COLL_ALL_REDUCE = 0, ORC_COLL_REDUCE_SCATTER = 1 };

#define ORC_OK 0
#define ORC_UNSUPPORTED (-1) /* the reference throws for this dtype / op */
#define ORC_BAD_ARG (-2)

size_t orc_dtype_size(int dtype);

uint32_t orc_ring_add(uint32_t n, uint32_t delta, uint32_t m);
uint32_t orc_ring_sub(uint32_t n, uint32_t delta, uint32_t m);
void orc_chunk_partition(size_t len, size_t nchunks, size_t* sizes, size_t* offsets);

float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_f16(float f);

int orc_reduce_ucx(const void* i0, const void* i1, void* o, size_t len, int dtype, int op);
int orc_reduce_shm(void* dst, const void* a, const void* b, int dtype, int op, size_t len);

/* 2-input reduce callback used by the replays: o = f(i0, i1) in the ucx argument order. */
typedef int (*orc_reduce2_fn)(const void* i0, const void* i1, void* o, size_t len, int dtype,
                              int op, void* user);
/* UINT64 tracing reduce: every value is a string of non-zero hex digits; o = digits(i0)digits(i1). */
int orc_trace_reduce2(const void* i0, const void* i1, void* o, size_t len, int dtype, int op,
                      void* user);

/* literal replays, N ranks simulated in one address space ("send/recv" = memcpy) */
int orc_ucx_all_reduce(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                       int dtype, int op, orc_reduce2_fn fn, void* user);
int orc_ucx_reduce_scatter(uint32_t nranks, const void* const* send, void* const* recv,
                           size_t recvlen, int dtype, int op, orc_reduce2_fn fn, void* user);
int orc_ucx_all_gather(uint32_t nranks, const void* const* send, void* const* recv, size_t sendlen,
                       int dtype);
int orc_ucx_all_to_all(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                       int dtype);
int orc_ucx_scatter(uint32_t nranks, const void* const* send, void* const* recv, size_t recvlen,
                    int dtype, uint32_t root);
int orc_ucx_gather(uint32_t nranks, const void* const* send, void* const* recv, size_t sendlen,
                   int dtype, uint32_t root);
int orc_ucx_reduce(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                   int dtype, int op, uint32_t root, orc_reduce2_fn fn, void* user);
int orc_ucx_broadcast(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                      int dtype, uint32_t root);

int orc_shm_all_reduce(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                       int dtype, int op, orc_reduce2_fn fn, void* user);
int orc_shm_reduce_scatter(uint32_t nranks, const void* const* send, void* const* recv,
                           size_t recvlen, int dtype, int op, orc_reduce2_fn fn, void* user);
/* Only recv[root] is written. */
int orc_shm_reduce(uint32_t nranks, const void* const* send, void* const* recv, size_t len, int dtype,
                   int op, uint32_t root, orc_reduce2_fn fn, void* user);
int orc_shm_broadcast(uint32_t nranks, const void* const* send, void* const* recv, size_t len, int dtype,
                      uint32_t root);
int orc_shm_all_gather(uint32_t nranks, const void* const* send, void* const* recv, size_t sendlen,
                       int dtype);
int orc_shm_all_to_all(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                       int dtype);

/* The expected-value loops of the reference's tests, FLOAT32 only. */
void orc_test_all_reduce_f32(uint32_t nranks, const float* const* in, float* const* out, size_t len,
                             int op);
void orc_test_reduce_scatter_f32(uint32_t nranks, const float* const* in, float* const* out,
                                 size_t recvlen, int op);
/* same SUM loop split over element ranges on `nthreads` host threads (CPU baseline only) */
void orc_test_all_reduce_f32_mt(uint32_t nranks, const float* const* in, float* const* out,
                                size_t len, int op, int nthreads);

/*
 * Fold order of one chunk: ranks[0] seeds the accumulator, ranks[1..] are folded in.
 * *new_wins_ties = 1 when a tie / unordered compare of MAX/MIN keeps the incoming operand.
 * nchunks_out: number of chunks the order splits the buffer into (N, or 2N for SHM, 1 for RANK0).
 */
int orc_fold_order(int coll, int order, uint32_t nranks, uint32_t chunk, uint32_t* ranks,
                   int* new_wins_ties, uint32_t* nchunks_out);
/* Per-chunk fold with a wide accumulator (fp32 for FLOAT16); all nine arithmetic dtypes. */
int orc_fold_all_reduce(uint32_t nranks, const void* const* send, void* const* recv, size_t len,
                        int dtype, int op, int order);
int orc_fold_reduce_scatter(uint32_t nranks, const void* const* send, void* const* recv,
                            size_t recvlen, int dtype, int op, int order);

#ifdef __cplusplus
}
#endif
#endif
