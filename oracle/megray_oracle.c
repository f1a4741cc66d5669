/*
 * megray_oracle.c -- CPU restatement of MegRay's ring reduce / pack path.
 *
 * TEST INFRASTRUCTURE ONLY (see megray_oracle.h for the rules and for what pins each
 * function).  Plain C99, no dependencies beyond libc + pthreads; built by oracle/Makefile with
 * -O2 -ffp-contract=off and never with -ffast-math, so every float operation below is a single
 * correctly rounded IEEE-754 operation.
 *
 * Every function cites the reference lines it follows (paths relative to the MegRay tree).
 */
#include "megray_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>

static void* xalloc(size_t n) { return malloc(n ? n : 1); }

/* ------------------------------------------------------------------ dtype table */

/* src/core/common.cpp:19-38.  The reference throws "unknown dtype" for anything else; 0 here. */
size_t orc_dtype_size(int dtype) {
    switch (dtype) {
        case ORC_CHAR:
        case ORC_INT8:
        case ORC_UINT8:
            return 1;
        case ORC_FLOAT16:
            return 2;
        case ORC_INT32:
        case ORC_UINT32:
        case ORC_FLOAT32:
            return 4;
        case ORC_INT64:
        case ORC_UINT64:
        case ORC_FLOAT64:
            return 8;
        default:
            return 0;
    }
}

/* ------------------------------------------------------------------ ring arithmetic */

/* src/ucx/utils.h:24-30 and src/shm/utils.h:21-27 (identical). */
uint32_t orc_ring_add(uint32_t n, uint32_t delta, uint32_t m) { return (n + delta) % m; }
uint32_t orc_ring_sub(uint32_t n, uint32_t delta, uint32_t m) { return (n + m - delta % m) % m; }

/*
 * src/ucx/all_reduce.cpp:33-38,48-51 (N chunks) and src/shm/all_reduce.cpp:54-65 (2N chunks):
 * quotient/remainder split, the first `remainder` chunks get one extra element, offsets are the
 * running sum.  Offsets here are in ELEMENTS (the reference multiplies by the dtype size).
 */
void orc_chunk_partition(size_t len, size_t nchunks, size_t* sizes, size_t* offsets) {
    size_t quotient = len / nchunks, remainder = len % nchunks;
    for (size_t i = 0; i < nchunks; i++) sizes[i] = quotient + (i < remainder ? 1 : 0);
    offsets[0] = 0;
    for (size_t i = 1; i < nchunks; i++) offsets[i] = offsets[i - 1] + sizes[i - 1];
}

/* ------------------------------------------------------------------ binary16 <-> binary32 */

/* IEEE 754 binary16 -> binary32, exact.  (No reference code: FLOAT16 reduce is an extension.) */
float orc_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1fu;
    uint32_t man = h & 0x3ffu;
    uint32_t bits;
    if (exp == 0) {
        if (man == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int shift = 0;
            while (!(man & 0x400u)) {
                man <<= 1;
                shift++;
            }
            man &= 0x3ffu;
            bits = sign | ((uint32_t)(127 - 15 + 1 - shift) << 23) | (man << 13);
        }
    } else if (exp == 31) {
        bits = sign | 0x7f800000u | (man << 13);
    } else {
        bits = sign | ((exp + 127 - 15) << 23) | (man << 13);
    }
    float f;
    memcpy(&f, &bits, 4);
    return f;
}

/* IEEE 754 binary32 -> binary16, round to nearest even; NaN keeps its top payload bits. */
uint16_t orc_f32_to_f16(float f) {
    uint32_t x;
    memcpy(&x, &f, 4);
    uint32_t sign = (x >> 16) & 0x8000u;
    uint32_t mag = x & 0x7fffffffu;
    if (mag >= 0x7f800000u) {
        if (mag == 0x7f800000u) return (uint16_t)(sign | 0x7c00u);
        uint32_t r = 0x7c00u + ((mag & 0x7fffffu) >> 13);
        if (r == 0x7c00u) r++;
        return (uint16_t)(sign | r);
    }
    int32_t e = (int32_t)(mag >> 23) - 127 + 15;
    uint32_t m = mag & 0x7fffffu;
    if (e >= 31) return (uint16_t)(sign | 0x7c00u);
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;
        m |= 0x800000u;
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t r = m >> shift;
        uint32_t rem = m & ((1u << shift) - 1u);
        uint32_t half = 1u << (shift - 1);
        if (rem > half || (rem == half && (r & 1u))) r++;
        return (uint16_t)(sign | r);
    }
    uint32_t r = ((uint32_t)e << 10) | (m >> 13);
    uint32_t rem = m & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (r & 1u))) r++;
    return (uint16_t)(sign | r);
}

/* ------------------------------------------------------------------ 2-input reduces */

/*
 * Integer SUM is computed in the unsigned type of the same width: identical to the reference's
 * `i0[i] + i1[i]` for int8/uint8 (promote to int, narrow mod 256) and for the unsigned types,
 * and it DEFINES the signed int32/int64 overflow case (undefined behaviour in the reference
 * source) as two's-complement wrap.
 */
#define UCX_LOOP(T, UT, IS_INT)                                                        \
    do {                                                                               \
        const T* a = (const T*)i0;                                                     \
        const T* b = (const T*)i1;                                                     \
        T* out = (T*)o;                                                                \
        switch (op) {                                                                  \
            case ORC_SUM: /* src/ucx/kernel.cu:16-22 */                                \
                for (size_t i = 0; i < len; i++)                                       \
                    out[i] = IS_INT ? (T)(UT)((UT)a[i] + (UT)b[i]) : (T)(a[i] + b[i]); \
                break;                                                                 \
            case ORC_MAX: /* src/ucx/kernel.cu:24-30: equal / unordered -> i1 */       \
                for (size_t i = 0; i < len; i++) out[i] = (a[i] > b[i]) ? a[i] : b[i]; \
                break;                                                                 \
            case ORC_MIN: /* src/ucx/kernel.cu:32-38: equal / unordered -> i1 */       \
                for (size_t i = 0; i < len; i++) out[i] = (a[i] < b[i]) ? a[i] : b[i]; \
                break;                                                                 \
            default: /* src/ucx/kernel.cu:55-56 throws "unknown reduce op" */          \
                return ORC_UNSUPPORTED;                                                \
        }                                                                              \
    } while (0)

/* src/ucx/kernel.cu:60-98: eight dtypes; FLOAT16 and CHAR throw "unknown dtype" (:95-96). */
int orc_reduce_ucx(const void* i0, const void* i1, void* o, size_t len, int dtype, int op) {
    switch (dtype) {
        case ORC_INT8: UCX_LOOP(int8_t, uint8_t, 1); break;
        case ORC_UINT8: UCX_LOOP(uint8_t, uint8_t, 1); break;
        case ORC_INT32: UCX_LOOP(int32_t, uint32_t, 1); break;
        case ORC_UINT32: UCX_LOOP(uint32_t, uint32_t, 1); break;
        case ORC_INT64: UCX_LOOP(int64_t, uint64_t, 1); break;
        case ORC_UINT64: UCX_LOOP(uint64_t, uint64_t, 1); break;
        case ORC_FLOAT32: UCX_LOOP(float, float, 0); break;
        case ORC_FLOAT64: UCX_LOOP(double, double, 0); break;
        default: return ORC_UNSUPPORTED;
    }
    return ORC_OK;
}

#define SHM_LOOP(T, UT, IS_INT)                                                          \
    do {                                                                                 \
        T* d = (T*)dst;                                                                  \
        const T* x = (const T*)a;                                                        \
        const T* y = (const T*)b;                                                        \
        switch (op) {                                                                    \
            case ORC_SUM: /* src/shm/utils.cpp:19-22 */                                  \
                for (size_t i = 0; i < len; i++)                                         \
                    d[i] = IS_INT ? (T)(UT)((UT)x[i] + (UT)y[i]) : (T)(x[i] + y[i]);     \
                break;                                                                   \
            case ORC_MAX: /* :24-27 std::max(a,b) == (a < b) ? b : a */                  \
                for (size_t i = 0; i < len; i++) d[i] = (x[i] < y[i]) ? y[i] : x[i];     \
                break;                                                                   \
            case ORC_MIN: /* :29-32 std::min(a,b) == (b < a) ? b : a */                  \
                for (size_t i = 0; i < len; i++) d[i] = (y[i] < x[i]) ? y[i] : x[i];     \
                break;                                                                   \
            default: /* :34-35 throws "unsupported op type" */                           \
                return ORC_UNSUPPORTED;                                                  \
        }                                                                                \
    } while (0)

/* src/shm/utils.cpp:39-69: six dtypes; UINT64, FLOAT64, FLOAT16, CHAR throw (:66-67). */
int orc_reduce_shm(void* dst, const void* a, const void* b, int dtype, int op, size_t len) {
    switch (dtype) {
        case ORC_INT8: SHM_LOOP(int8_t, uint8_t, 1); break;
        case ORC_UINT8: SHM_LOOP(uint8_t, uint8_t, 1); break;
        case ORC_INT32: SHM_LOOP(int32_t, uint32_t, 1); break;
        case ORC_UINT32: SHM_LOOP(uint32_t, uint32_t, 1); break;
        case ORC_INT64: SHM_LOOP(int64_t, uint64_t, 1); break;
        case ORC_FLOAT32: SHM_LOOP(float, float, 0); break;
        default: return ORC_UNSUPPORTED;
    }
    return ORC_OK;
}

/* Tracing reduce (test device, no reference counterpart): concatenates hex-digit strings. */
int orc_trace_reduce2(const void* i0, const void* i1, void* o, size_t len, int dtype, int op,
                      void* user) {
    (void)op;
    (void)user;
    if (dtype != ORC_UINT64) return ORC_BAD_ARG;
    const uint64_t* a = (const uint64_t*)i0;
    const uint64_t* b = (const uint64_t*)i1;
    uint64_t* out = (uint64_t*)o;
    for (size_t i = 0; i < len; i++) {
        int digits = 0;
        for (uint64_t t = b[i]; t; t >>= 4) digits++;
        out[i] = (digits >= 16) ? 0 : ((a[i] << (4 * digits)) | b[i]);
    }
    return ORC_OK;
}

static int ucx_reduce2(orc_reduce2_fn fn, void* user, const void* i0, const void* i1, void* o,
                       size_t len, int dtype, int op) {
    return fn ? fn(i0, i1, o, len, dtype, op, user) : orc_reduce_ucx(i0, i1, o, len, dtype, op);
}

static int shm_reduce2(orc_reduce2_fn fn, void* user, void* dst, const void* a, const void* b,
                       size_t len, int dtype, int op) {
    return fn ? fn(a, b, dst, len, dtype, op, user) : orc_reduce_shm(dst, a, b, dtype, op, len);
}

/* ------------------------------------------------------------------ ucx replays */

/*
 * src/ucx/all_reduce.cpp:23-109.  Every rank runs the same loop; a step's sends all leave
 * before its reduces start (the chunk a rank sends in step i is not the one it reduces into in
 * step i), so the simulation moves all messages of a step, then runs all reduces of that step.
 */
int orc_ucx_all_reduce(uint32_t N, const void* const* send, void* const* recv, size_t len,
                       int dtype, int op, orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t* sizes = (size_t*)malloc(sizeof(size_t) * N * 2);
    size_t* offs = sizes + N;
    orc_chunk_partition(len, N, sizes, offs); /* :33-38,48-51 */
    char* work = (char*)malloc((sizes[0] ? sizes[0] : 1) * size * N); /* :43, one per rank */
    int rc = ORC_OK;
    for (uint32_t r = 0; r < N; r++) /* :44-45 */
        if (recv[r] != send[r]) memmove(recv[r], send[r], len * size);
    for (uint32_t i = 0; i + 1 < N && rc == ORC_OK; i++) { /* :61-82 */
        for (uint32_t r = 0; r < N; r++) {                 /* rank r sends to r+1 (:68-70) */
            uint32_t send_chunk = orc_ring_sub(r, i, N);
            uint32_t right = (r + 1) % N;
            memcpy(work + (size_t)right * sizes[0] * size, (char*)recv[r] + offs[send_chunk] * size,
                   sizes[send_chunk] * size);
        }
        for (uint32_t r = 0; r < N && rc == ORC_OK; r++) { /* :74-76 reduce(local, workspace) */
            uint32_t recv_chunk = orc_ring_sub(r, i + 1, N);
            char* local = (char*)recv[r] + offs[recv_chunk] * size;
            rc = ucx_reduce2(fn, user, local, work + (size_t)r * sizes[0] * size, local,
                             sizes[recv_chunk], dtype, op);
        }
    }
    for (uint32_t i = 0; i + 1 < N && rc == ORC_OK; i++) { /* :88-101 ring all-gather */
        for (uint32_t r = 0; r < N; r++) {
            uint32_t send_chunk = orc_ring_sub(r + 1, i, N);
            uint32_t right = (r + 1) % N;
            /* the receiver files it under recv_chunk = ring_sub(right, i) == send_chunk */
            memcpy((char*)recv[right] + offs[send_chunk] * size,
                   (char*)recv[r] + offs[send_chunk] * size, sizes[send_chunk] * size);
        }
    }
    free(work);
    free(sizes);
    return rc;
}

/* src/ucx/reduce_scatter.cpp:21-61. */
int orc_ucx_reduce_scatter(uint32_t N, const void* const* send, void* const* recv, size_t recvlen,
                           int dtype, int op, orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t chunk = recvlen * size;
    size_t alloc = chunk ? chunk : 1;
    char* lbuf = (char*)malloc(alloc * N);     /* :34 per rank */
    char* rbuf = (char*)malloc(alloc * N * N); /* :35 per rank */
    int rc = ORC_OK;
    for (uint32_t r = 0; r < N; r++) memcpy(rbuf + (size_t)r * N * chunk, send[r], N * chunk); /* :37 */
    for (uint32_t i = 1; i < N && rc == ORC_OK; i++) { /* :44-53 */
        for (uint32_t r = 0; r < N; r++) {
            uint32_t right = orc_ring_add(r, 1, N);
            size_t send_off = chunk * orc_ring_sub(r, i, N);
            memcpy(lbuf + (size_t)right * chunk, rbuf + (size_t)r * N * chunk + send_off, chunk);
        }
        for (uint32_t r = 0; r < N && rc == ORC_OK; r++) {
            size_t recv_off = chunk * orc_ring_sub(r, i + 1, N);
            char* local = rbuf + (size_t)r * N * chunk + recv_off;
            /* :50-51 reduce(lbuffer, rbuffer + recv_offset, rbuffer + recv_offset) */
            rc = ucx_reduce2(fn, user, lbuf + (size_t)r * chunk, local, local, recvlen, dtype, op);
        }
    }
    for (uint32_t r = 0; r < N; r++) /* :54-56 */
        memcpy(recv[r], rbuf + (size_t)r * N * chunk + chunk * r, chunk);
    free(lbuf);
    free(rbuf);
    return rc;
}

/* src/ucx/all_gather.cpp:21-63. */
int orc_ucx_all_gather(uint32_t N, const void* const* send, void* const* recv, size_t sendlen,
                       int dtype) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t bytes = sendlen * size;
    for (uint32_t r = 0; r < N; r++) memmove((char*)recv[r] + r * bytes, send[r], bytes); /* :31-32 */
    for (uint32_t i = 0; i + 1 < N; i++) { /* :42-60 */
        for (uint32_t r = 0; r < N; r++) {
            uint32_t send_rank = orc_ring_sub(r, i, N);
            uint32_t right = (r + 1) % N;
            memcpy((char*)recv[right] + send_rank * bytes, (char*)recv[r] + send_rank * bytes, bytes);
        }
    }
    return ORC_OK;
}

/* src/ucx/all_to_all.cpp:21-43: rank m sends block r to rank r, files what r sends under r. */
int orc_ucx_all_to_all(uint32_t N, const void* const* send, void* const* recv, size_t len,
                       int dtype) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t bytes = len * size;
    for (uint32_t m = 0; m < N; m++)
        for (uint32_t r = 0; r < N; r++)
            memcpy((char*)recv[r] + m * bytes, (const char*)send[m] + r * bytes, bytes);
    return ORC_OK;
}

/* src/ucx/scatter.cpp:21-46.  Only send[root] and recv[*] are touched. */
int orc_ucx_scatter(uint32_t N, const void* const* send, void* const* recv, size_t recvlen,
                    int dtype, uint32_t root) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N || root >= N) return ORC_BAD_ARG;
    size_t bytes = recvlen * size;
    for (uint32_t r = 0; r < N; r++) memcpy(recv[r], (const char*)send[root] + r * bytes, bytes);
    return ORC_OK;
}

/* src/ucx/gather.cpp:21-46.  Only send[*] and recv[root] are touched. */
int orc_ucx_gather(uint32_t N, const void* const* send, void* const* recv, size_t sendlen,
                   int dtype, uint32_t root) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N || root >= N) return ORC_BAD_ARG;
    size_t bytes = sendlen * size;
    for (uint32_t r = 0; r < N; r++) memcpy((char*)recv[root] + r * bytes, send[r], bytes);
    return ORC_OK;
}

static uint32_t tree_rounds(uint32_t N) {
    uint32_t d = 0, t = N - 1;
    while (t > 0) {
        ++d;
        t >>= 1;
    }
    return d;
}

/* src/ucx/reduce.cpp:21-87: binomial tree towards virtual rank 0 (= root). */
int orc_ucx_reduce(uint32_t N, const void* const* send, void* const* recv, size_t len, int dtype,
                   int op, uint32_t root, orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N || root >= N) return ORC_BAD_ARG;
    size_t bytes = len * size, alloc = bytes ? bytes : 1;
    char* lbuf = (char*)malloc(alloc * N);
    char* rbuf = (char*)malloc(alloc * N);
    int rc = ORC_OK;
    for (uint32_t r = 0; r < N; r++) memcpy(rbuf + r * bytes, send[r], bytes); /* :38-39 */
    uint32_t d = tree_rounds(N);
    uint32_t mask = 0;
    for (uint32_t i = 0; i < d && rc == ORC_OK; i++) { /* :56-80 */
        uint32_t bit = 1u << i;
        for (uint32_t r = 0; r < N; r++) { /* senders first */
            uint32_t vr = orc_ring_sub(r, root, N);
            if ((vr & mask) == 0 && (vr & bit) != 0) {
                uint32_t vdest = vr ^ bit;
                if (vdest < N) {
                    uint32_t dest = orc_ring_add(vdest, root, N);
                    memcpy(lbuf + dest * bytes, rbuf + r * bytes, bytes);
                }
            }
        }
        for (uint32_t r = 0; r < N && rc == ORC_OK; r++) {
            uint32_t vr = orc_ring_sub(r, root, N);
            if ((vr & mask) == 0 && (vr & bit) == 0) {
                uint32_t vsrc = vr ^ bit;
                if (vsrc < N) /* :73-74 reduce(lbuffer, rbuffer, rbuffer) */
                    rc = ucx_reduce2(fn, user, lbuf + r * bytes, rbuf + r * bytes, rbuf + r * bytes,
                                     len, dtype, op);
            }
        }
        mask ^= bit;
    }
    memcpy(recv[root], rbuf + root * bytes, bytes); /* :82-85 */
    free(lbuf);
    free(rbuf);
    return rc;
}

/* src/ucx/broadcast.cpp:21-76: every rank ends with the root's data. */
int orc_ucx_broadcast(uint32_t N, const void* const* send, void* const* recv, size_t len,
                      int dtype, uint32_t root) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N || root >= N) return ORC_BAD_ARG;
    size_t bytes = len * size;
    memmove(recv[root], send[root], bytes); /* :31-34 */
    uint32_t d = tree_rounds(N);
    uint32_t mask = (1u << d) - 1u;
    for (int i = (int)d - 1; i >= 0; --i) { /* :54-73 */
        uint32_t bit = 1u << i;
        mask ^= bit;
        for (uint32_t r = 0; r < N; r++) {
            uint32_t vr = orc_ring_sub(r, root, N);
            if ((vr & mask) == 0 && (vr & bit) == 0) {
                uint32_t vdest = vr ^ bit;
                if (vdest < N) {
                    uint32_t dest = orc_ring_add(vdest, root, N);
                    memcpy(recv[dest], recv[r], bytes);
                }
            }
        }
    }
    return ORC_OK;
}

/* ------------------------------------------------------------------ shm replays */

/*
 * The shared arena of src/shm/all_reduce.cpp:49,69 is two buffer-sized areas: A (accumulators)
 * and S (staging).  Rank m seeds A with its own k=2 chunks (:91-94); for i = k+1..2N it stages
 * chunk w from its sendbuff into S (:100-109) and its CPU thread runs
 * cpu_reduce(A[w], A[w], S[w]) (src/shm/communicator.cpp:56-68), w starting at the right
 * neighbour's first chunk and advancing by one.  Step i of rank m waits for step i-k of rank m+1
 * (:101), which is the previous fold of the same chunk, so running i outermost is a valid
 * serialisation.
 */
static int shm_fold(uint32_t N, const void* const* send, char* A, size_t total, int dtype, int op,
                    orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    size_t k = 2, chunks = (size_t)N * k;
    size_t* sizes = (size_t*)malloc(sizeof(size_t) * chunks * 2);
    size_t* offs = sizes + chunks;
    orc_chunk_partition(total, chunks, sizes, offs);
    char* S = (char*)xalloc(total * size);
    int rc = ORC_OK;
    for (uint32_t m = 0; m < N; m++)
        for (size_t j = 0; j < k; j++) {
            size_t w = m * k + j;
            memcpy(A + offs[w] * size, (const char*)send[m] + offs[w] * size, sizes[w] * size);
        }
    for (size_t i = k + 1; i <= chunks && rc == ORC_OK; i++) {
        for (uint32_t m = 0; m < N && rc == ORC_OK; m++) {
            size_t w = (m * k + k + (i - k - 1)) % chunks;
            memcpy(S + offs[w] * size, (const char*)send[m] + offs[w] * size, sizes[w] * size);
            rc = shm_reduce2(fn, user, A + offs[w] * size, A + offs[w] * size, S + offs[w] * size,
                             sizes[w], dtype, op);
        }
    }
    free(S);
    free(sizes);
    return rc;
}

/* src/shm/all_reduce.cpp:38-127: every rank copies all of A back (:110-123). */
int orc_shm_all_reduce(uint32_t N, const void* const* send, void* const* recv, size_t len,
                       int dtype, int op, orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    char* A = (char*)xalloc(len * size);
    int rc = shm_fold(N, send, A, len, dtype, op, fn, user);
    if (rc == ORC_OK)
        for (uint32_t r = 0; r < N; r++) memcpy(recv[r], A, len * size);
    free(A);
    return rc;
}

/* src/shm/reduce_scatter.cpp:21-97: same fold over N*recvlen elements, rank r reads its slice (:91-93). */
int orc_shm_reduce_scatter(uint32_t N, const void* const* send, void* const* recv, size_t recvlen,
                           int dtype, int op, orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t total = (size_t)N * recvlen;
    char* A = (char*)xalloc(total * size);
    int rc = shm_fold(N, send, A, total, dtype, op, fn, user);
    if (rc == ORC_OK)
        for (uint32_t r = 0; r < N; r++)
            memcpy(recv[r], A + (size_t)r * recvlen * size, recvlen * size);
    free(A);
    return rc;
}

/*
 * src/shm/reduce.cpp:21-100, replayed with its own bookkeeping.  Every rank m seeds the accumulator
 * area A with its k = 2 chunks (:55-58), then runs i = k .. chunks-1 (:73-93): before step i it spins
 * until the right neighbour's mutex has reached i - k (:75-76, an unsigned comparison: the `int` is
 * converted), stages chunk `work_rank` of its own sendbuff in S and runs
 * cpu_reduce(A[w], A[w], S[w]) (:83-86), publishes mutex[m] = i - 1 (:87) and moves to the next
 * chunk; work_rank starts at ring_add(m * k, k, chunks) (:65).  The root then reads all of A
 * (:95-99).  The ranks run concurrently in the reference; here they are stepped one at a time,
 * highest rank first, each taking a step whenever its wait condition holds - any interleaving the
 * mutexes allow gives the same result, and this one differs from the rank-ascending, step-outermost
 * order of shm_fold above.
 */
int orc_shm_reduce(uint32_t N, const void* const* send, void* const* recv, size_t len, int dtype,
                   int op, uint32_t root, orc_reduce2_fn fn, void* user) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N || root >= N) return ORC_BAD_ARG;
    size_t k = 2, chunks = (size_t)N * k;
    size_t* sizes = (size_t*)malloc(sizeof(size_t) * chunks * 2);
    size_t* offs = sizes + chunks;
    orc_chunk_partition(len, chunks, sizes, offs);
    char* A = (char*)xalloc(len * size);
    char* S = (char*)xalloc(len * size);
    int* mutex = (int*)malloc(sizeof(int) * N);
    size_t* step = (size_t*)malloc(sizeof(size_t) * N * 2);
    size_t* work = step + N;
    int rc = ORC_OK;
    for (uint32_t m = 0; m < N; m++) {
        size_t seeded = 0;
        for (size_t j = 0; j < k; j++) seeded += sizes[m * k + j];
        memcpy(A + offs[m * k] * size, (const char*)send[m] + offs[m * k] * size, seeded * size);
        mutex[m] = 0;
        step[m] = k;
        work[m] = orc_ring_add((uint32_t)(m * k), (uint32_t)k, (uint32_t)chunks);
    }
    for (int progress = 1; progress && rc == ORC_OK;) {
        progress = 0;
        for (uint32_t back = 0; back < N && rc == ORC_OK; back++) {
            uint32_t m = N - 1 - back;
            if (step[m] >= chunks) continue;
            uint32_t right = orc_ring_add(m, 1, N);
            if ((size_t)mutex[right] < step[m] - k) continue; /* still spinning at :75-76 */
            size_t w = work[m];
            memcpy(S + offs[w] * size, (const char*)send[m] + offs[w] * size, sizes[w] * size);
            rc = shm_reduce2(fn, user, A + offs[w] * size, A + offs[w] * size, S + offs[w] * size,
                             sizes[w], dtype, op);
            mutex[m] = (int)(step[m] - 1);
            work[m] = orc_ring_add((uint32_t)w, 1, (uint32_t)chunks);
            step[m]++;
            progress = 1;
        }
    }
    for (uint32_t m = 0; m < N && rc == ORC_OK; m++)
        if (step[m] < chunks) rc = ORC_BAD_ARG; /* a wait that never ends: cannot happen */
    if (rc == ORC_OK) memcpy(recv[root], A, len * size);
    free(step);
    free(mutex);
    free(S);
    free(A);
    free(sizes);
    return rc;
}

/*
 * src/shm/broadcast.cpp:19-51: the root copies its sendbuff into the arena and into its own recvbuff
 * (:32-38); after the barrier every other rank copies the arena into its recvbuff (:43-46).
 */
int orc_shm_broadcast(uint32_t N, const void* const* send, void* const* recv, size_t len, int dtype,
                      uint32_t root) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N || root >= N) return ORC_BAD_ARG;
    size_t bytes = len * size;
    char* arena = (char*)xalloc(bytes);
    memcpy(arena, send[root], bytes);
    memmove(recv[root], send[root], bytes);
    for (uint32_t m = 0; m < N; m++)
        if (m != root) memcpy(recv[m], arena, bytes);
    free(arena);
    return ORC_OK;
}

/* src/shm/all_gather.cpp:28-55: slot `rank` of the arena <- sendbuff; everybody reads the arena. */
int orc_shm_all_gather(uint32_t N, const void* const* send, void* const* recv, size_t sendlen,
                       int dtype) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t bytes = sendlen * size;
    char* arena = (char*)xalloc(bytes * N);
    for (uint32_t r = 0; r < N; r++) memcpy(arena + r * bytes, send[r], bytes);
    for (uint32_t r = 0; r < N; r++) memcpy(recv[r], arena, bytes * N);
    free(arena);
    return ORC_OK;
}

/* src/shm/all_to_all.cpp:18-59: block i of rank m goes to arena[i][m]; rank m reads row m. */
int orc_shm_all_to_all(uint32_t N, const void* const* send, void* const* recv, size_t len,
                       int dtype) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t bytes = len * size;
    char* arena = (char*)xalloc(bytes * N * N);
    for (uint32_t m = 0; m < N; m++)
        for (uint32_t i = 0; i < N; i++)
            memcpy(arena + bytes * N * i + m * bytes, (const char*)send[m] + bytes * i, bytes);
    for (uint32_t m = 0; m < N; m++) memcpy(recv[m], arena + (size_t)m * N * bytes, bytes * N);
    free(arena);
    return ORC_OK;
}

/* ------------------------------------------------------------------ the tests' expected-value loops */

/*
 * test/test_opr.cpp:321-330 (SUM: `float sum = 0`, ranks 0..N-1), :334-345 (MAX from
 * numeric_limits<float>::min(), the smallest positive normal), :347-358 (MIN from max()).
 */
static float test_fold_f32(uint32_t N, const float* const* in, size_t j, int op) {
    if (op == ORC_SUM) {
        float sum = 0;
        for (uint32_t i = 0; i < N; i++) sum += in[i][j];
        return sum;
    }
    if (op == ORC_MAX) {
        float v = 1.17549435e-38f;
        for (uint32_t i = 0; i < N; i++) v = (v < in[i][j]) ? in[i][j] : v;
        return v;
    }
    float v = 3.40282347e+38f;
    for (uint32_t i = 0; i < N; i++) v = (in[i][j] < v) ? in[i][j] : v;
    return v;
}

void orc_test_all_reduce_f32(uint32_t N, const float* const* in, float* const* out, size_t len,
                             int op) {
    for (size_t j = 0; j < len; j++) {
        float v = test_fold_f32(N, in, j, op);
        for (uint32_t i = 0; i < N; i++) out[i][j] = v;
    }
}

/* test/test_opr.cpp:397-435: out[k][j] = fold over ranks of in[i][k*recvlen + j]. */
void orc_test_reduce_scatter_f32(uint32_t N, const float* const* in, float* const* out,
                                 size_t recvlen, int op) {
    for (uint32_t k = 0; k < N; k++)
        for (size_t j = 0; j < recvlen; j++) out[k][j] = test_fold_f32(N, in, k * recvlen + j, op);
}

struct mt_job {
    uint32_t N;
    const float* const* in;
    float* const* out;
    size_t begin, end;
    int op;
};

static void* mt_worker(void* p) {
    struct mt_job* job = (struct mt_job*)p;
    for (size_t j = job->begin; j < job->end; j++) {
        float v = test_fold_f32(job->N, job->in, j, job->op);
        for (uint32_t i = 0; i < job->N; i++) job->out[i][j] = v;
    }
    return NULL;
}

void orc_test_all_reduce_f32_mt(uint32_t N, const float* const* in, float* const* out, size_t len,
                                int op, int nthreads) {
    if (nthreads < 1) nthreads = 1;
    pthread_t* tids = (pthread_t*)malloc(sizeof(pthread_t) * nthreads);
    struct mt_job* jobs = (struct mt_job*)malloc(sizeof(struct mt_job) * nthreads);
    for (int t = 0; t < nthreads; t++) {
        jobs[t].N = N;
        jobs[t].in = in;
        jobs[t].out = out;
        jobs[t].begin = len * (size_t)t / nthreads;
        jobs[t].end = len * (size_t)(t + 1) / nthreads;
        jobs[t].op = op;
        pthread_create(&tids[t], NULL, mt_worker, &jobs[t]);
    }
    for (int t = 0; t < nthreads; t++) pthread_join(tids[t], NULL);
    free(jobs);
    free(tids);
}

/* ------------------------------------------------------------------ fold orders and wide folds */

/*
 * The order in which one chunk's N contributions meet, read off the replays above:
 *   UCX all_reduce   chunk c: x_c, x_{c+1}, ..., x_{c-1}; step reduce(local=new, incoming=acc),
 *                    ties/unordered -> i1 = acc           (src/ucx/all_reduce.cpp:61-82)
 *   UCX reduce_scatter chunk c: x_{c+1}, ..., x_{c-1}, x_c; reduce(incoming=acc, local=new),
 *                    ties/unordered -> i1 = new           (src/ucx/reduce_scatter.cpp:44-53)
 *   SHM (both)       chunk w of 2N, owner o = w/2: x_o, x_{o-1}, ..., x_{o+1};
 *                    cpu_reduce(A, A=acc, S=new), std::max/min keep the first on ties -> acc
 *   RANK0            every element: x_0, ..., x_{N-1}, ties -> acc (test/test_opr.cpp:321-358)
 */
int orc_fold_order(int coll, int order, uint32_t N, uint32_t chunk, uint32_t* ranks,
                   int* new_wins_ties, uint32_t* nchunks_out) {
    if (!N) return ORC_BAD_ARG;
    uint32_t nchunks, start;
    int dir, new_wins = 0;
    switch (order) {
        case ORC_ORDER_UCX:
            nchunks = N;
            dir = 1;
            if (coll == ORC_COLL_ALL_REDUCE) {
                start = chunk % N;
            } else {
                start = (chunk + 1) % N;
                new_wins = 1;
            }
            break;
        case ORC_ORDER_SHM:
            nchunks = 2 * N;
            dir = -1;
            start = (chunk / 2) % N;
            break;
        case ORC_ORDER_RANK0:
            nchunks = 1;
            dir = 1;
            start = 0;
            break;
        default:
            return ORC_BAD_ARG;
    }
    if (chunk >= nchunks) return ORC_BAD_ARG;
    for (uint32_t j = 0; j < N; j++)
        ranks[j] = dir > 0 ? (start + j) % N : (start + N - j % N) % N;
    if (new_wins_ties) *new_wins_ties = new_wins;
    if (nchunks_out) *nchunks_out = nchunks;
    return ORC_OK;
}

#define FOLD_STEP(acc, x)                                                         \
    do {                                                                          \
        if (op == ORC_SUM) {                                                      \
            acc = acc + x;                                                        \
        } else if (op == ORC_MAX) {                                               \
            acc = new_wins ? ((acc > x) ? acc : x) : ((x > acc) ? x : acc);       \
        } else {                                                                  \
            acc = new_wins ? ((acc < x) ? acc : x) : ((x < acc) ? x : acc);       \
        }                                                                         \
    } while (0)

/* ACC is the accumulator type: the unsigned twin for integer SUM wrap is applied via UT casts. */
#define FOLD_INT(T, UT)                                                               \
    for (size_t e = begin; e < end; e++) {                                            \
        T acc = ((const T*)send[ranks[0]])[e];                                        \
        for (uint32_t j = 1; j < N; j++) {                                            \
            T x = ((const T*)send[ranks[j]])[e];                                      \
            if (op == ORC_SUM) acc = (T)(UT)((UT)acc + (UT)x);                        \
            else FOLD_STEP(acc, x);                                                   \
        }                                                                             \
        ((T*)out)[e] = acc;                                                           \
    }

#define FOLD_FLT(T)                                                                   \
    for (size_t e = begin; e < end; e++) {                                            \
        T acc = ((const T*)send[ranks[0]])[e];                                        \
        for (uint32_t j = 1; j < N; j++) {                                            \
            T x = ((const T*)send[ranks[j]])[e];                                      \
            FOLD_STEP(acc, x);                                                        \
        }                                                                             \
        ((T*)out)[e] = acc;                                                           \
    }

static int fold_buffer(int coll, int order, uint32_t N, const void* const* send, void* out,
                       size_t total, int dtype, int op) {
    if (op != ORC_SUM && op != ORC_MAX && op != ORC_MIN) return ORC_UNSUPPORTED;
    if (dtype == ORC_CHAR || !orc_dtype_size(dtype)) return ORC_UNSUPPORTED;
    uint32_t* ranks = (uint32_t*)malloc(sizeof(uint32_t) * N);
    uint32_t nchunks = 0;
    int new_wins = 0;
    int rc = orc_fold_order(coll, order, N, 0, ranks, &new_wins, &nchunks);
    if (rc != ORC_OK) {
        free(ranks);
        return rc;
    }
    size_t* sizes = (size_t*)malloc(sizeof(size_t) * nchunks * 2);
    size_t* offs = sizes + nchunks;
    orc_chunk_partition(total, nchunks, sizes, offs);
    for (uint32_t c = 0; c < nchunks; c++) {
        orc_fold_order(coll, order, N, c, ranks, &new_wins, NULL);
        size_t begin = offs[c], end = offs[c] + sizes[c];
        switch (dtype) {
            case ORC_INT8: FOLD_INT(int8_t, uint8_t) break;
            case ORC_UINT8: FOLD_INT(uint8_t, uint8_t) break;
            case ORC_INT32: FOLD_INT(int32_t, uint32_t) break;
            case ORC_UINT32: FOLD_INT(uint32_t, uint32_t) break;
            case ORC_INT64: FOLD_INT(int64_t, uint64_t) break;
            case ORC_UINT64: FOLD_INT(uint64_t, uint64_t) break;
            case ORC_FLOAT32: FOLD_FLT(float) break;
            case ORC_FLOAT64: FOLD_FLT(double) break;
            case ORC_FLOAT16:
                for (size_t e = begin; e < end; e++) {
                    float acc = orc_f16_to_f32(((const uint16_t*)send[ranks[0]])[e]);
                    for (uint32_t j = 1; j < N; j++) {
                        float x = orc_f16_to_f32(((const uint16_t*)send[ranks[j]])[e]);
                        FOLD_STEP(acc, x);
                    }
                    ((uint16_t*)out)[e] = orc_f32_to_f16(acc);
                }
                break;
            default: break;
        }
    }
    free(sizes);
    free(ranks);
    return ORC_OK;
}

int orc_fold_all_reduce(uint32_t N, const void* const* send, void* const* recv, size_t len,
                        int dtype, int op, int order) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    void* tmp = xalloc(len * size);
    int rc = fold_buffer(ORC_COLL_ALL_REDUCE, order, N, send, tmp, len, dtype, op);
    if (rc == ORC_OK)
        for (uint32_t r = 0; r < N; r++) memcpy(recv[r], tmp, len * size);
    free(tmp);
    return rc;
}

int orc_fold_reduce_scatter(uint32_t N, const void* const* send, void* const* recv, size_t recvlen,
                            int dtype, int op, int order) {
    size_t size = orc_dtype_size(dtype);
    if (!size || !N) return ORC_BAD_ARG;
    size_t total = (size_t)N * recvlen;
    char* tmp = (char*)xalloc(total * size);
    int rc = fold_buffer(ORC_COLL_REDUCE_SCATTER, order, N, send, tmp, total, dtype, op);
    if (rc == ORC_OK)
        for (uint32_t r = 0; r < N; r++)
            memcpy(recv[r], tmp + (size_t)r * recvlen * size, recvlen * size);
    free(tmp);
    return rc;
}
