/*
 * selftest.c -- drives every oracle entry point on small ragged inputs so that a build with
 * -fsanitize=address,undefined (make -C oracle selftest_asan) can catch out-of-bounds accesses,
 * leaks and undefined arithmetic in the oracle itself.  TEST INFRASTRUCTURE ONLY.
 * Also cross-checks the fold form against the literal replays for every dtype the reference has.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "megray_oracle.h"

static uint64_t state = 0x9E3779B97F4A7C15ull;
static uint64_t next_u64(void) {
    state ^= state << 13;
    state ^= state >> 7;
    state ^= state << 17;
    return state;
}

static void fill(void* p, size_t bytes, int dtype) {
    unsigned char* b = (unsigned char*)p;
    for (size_t i = 0; i < bytes; i++) b[i] = (unsigned char)next_u64();
    if (dtype == ORC_FLOAT32) { /* keep floats finite and of mixed magnitude */
        float* f = (float*)p;
        for (size_t i = 0; i < bytes / 4; i++) f[i] = (float)((double)(int64_t)next_u64() / 9.2e18 * (1 << (next_u64() % 20)));
    } else if (dtype == ORC_FLOAT64) {
        double* f = (double*)p;
        for (size_t i = 0; i < bytes / 8; i++) f[i] = (double)(int64_t)next_u64() / 9.2e18 * (1 << (next_u64() % 20));
    } else if (dtype == ORC_FLOAT16) {
        uint16_t* h = (uint16_t*)p;
        for (size_t i = 0; i < bytes / 2; i++) h[i] = orc_f32_to_f16((float)((double)(int64_t)next_u64() / 9.2e18 * 64.0));
    }
}

#define MAXN 9
int main(void) {
    int failures = 0;
    const int dtypes[] = {ORC_INT8, ORC_UINT8, ORC_INT32, ORC_UINT32, ORC_INT64, ORC_UINT64, ORC_FLOAT16, ORC_FLOAT32, ORC_FLOAT64};
    for (unsigned d = 0; d < sizeof(dtypes) / sizeof(dtypes[0]); d++) {
        int dtype = dtypes[d];
        size_t size = orc_dtype_size(dtype);
        for (uint32_t n = 1; n <= MAXN; n++) {
            for (size_t len = 0; len <= 3 * n + 2; len += (len < n + 2 ? 1 : n)) {
                void* send[MAXN];
                void* recv[MAXN];
                void* recv2[MAXN];
                for (uint32_t r = 0; r < n; r++) {
                    send[r] = malloc(len * n * size + 1);
                    recv[r] = malloc(len * n * size + 1);
                    recv2[r] = malloc(len * n * size + 1);
                    fill(send[r], len * n * size, dtype);
                }
                for (int op = ORC_SUM; op <= ORC_MIN; op++) {
                    int lit = orc_ucx_all_reduce(n, (const void* const*)send, recv, len, dtype, op, NULL, NULL);
                    int fold = orc_fold_all_reduce(n, (const void* const*)send, recv2, len, dtype, op, ORC_ORDER_UCX);
                    if (dtype == ORC_FLOAT16) {
                        if ((n > 1 && lit != ORC_UNSUPPORTED) || fold != ORC_OK) { printf("f16 rc lit=%d fold=%d n=%u len=%zu op=%d\n", lit, fold, n, len, op); failures++; }
                    } else if (lit != ORC_OK || fold != ORC_OK || memcmp(recv[n - 1], recv2[n - 1], len * size)) {
                        printf("all_reduce mismatch dtype=%d n=%u len=%zu op=%d\n", dtype, n, len, op);
                        failures++;
                    }
                    lit = orc_ucx_reduce_scatter(n, (const void* const*)send, recv, len, dtype, op, NULL, NULL);
                    fold = orc_fold_reduce_scatter(n, (const void* const*)send, recv2, len, dtype, op, ORC_ORDER_UCX);
                    if (dtype != ORC_FLOAT16 && (lit != ORC_OK || fold != ORC_OK || memcmp(recv[0], recv2[0], len * size))) {
                        printf("reduce_scatter mismatch dtype=%d n=%u len=%zu op=%d\n", dtype, n, len, op);
                        failures++;
                    }
                    lit = orc_shm_all_reduce(n, (const void* const*)send, recv, len, dtype, op, NULL, NULL);
                    fold = orc_fold_all_reduce(n, (const void* const*)send, recv2, len, dtype, op, ORC_ORDER_SHM);
                    if (lit == ORC_OK && (fold != ORC_OK || memcmp(recv[0], recv2[0], len * size))) {
                        printf("shm all_reduce mismatch dtype=%d n=%u len=%zu op=%d\n", dtype, n, len, op);
                        failures++;
                    }
                    orc_shm_reduce_scatter(n, (const void* const*)send, recv, len, dtype, op, NULL, NULL);
                    orc_fold_reduce_scatter(n, (const void* const*)send, recv2, len, dtype, op, ORC_ORDER_SHM);
                    orc_fold_all_reduce(n, (const void* const*)send, recv2, len, dtype, op, ORC_ORDER_RANK0);
                    orc_ucx_reduce(n, (const void* const*)send, recv, len, dtype, op, n / 2, NULL, NULL);
                }
                orc_ucx_all_gather(n, (const void* const*)send, recv, len, dtype);
                orc_shm_all_gather(n, (const void* const*)send, recv2, len, dtype);
                if (memcmp(recv[0], recv2[0], len * n * size)) { printf("all_gather mismatch\n"); failures++; }
                orc_ucx_all_to_all(n, (const void* const*)send, recv, len, dtype);
                orc_shm_all_to_all(n, (const void* const*)send, recv2, len, dtype);
                if (memcmp(recv[n - 1], recv2[n - 1], len * n * size)) { printf("all_to_all mismatch\n"); failures++; }
                orc_ucx_scatter(n, (const void* const*)send, recv, len, dtype, n - 1);
                orc_ucx_gather(n, (const void* const*)send, recv, len, dtype, 0);
                orc_ucx_broadcast(n, (const void* const*)send, recv, len, dtype, n / 2);
                if (dtype == ORC_FLOAT32) {
                    orc_test_all_reduce_f32(n, (const float* const*)send, (float* const*)recv, len, ORC_SUM);
                    orc_test_all_reduce_f32_mt(n, (const float* const*)send, (float* const*)recv2, len, ORC_SUM, 3);
                    if (memcmp(recv[0], recv2[0], len * size)) failures++;
                    orc_test_reduce_scatter_f32(n, (const float* const*)send, (float* const*)recv, len, ORC_MAX);
                }
                if (dtype == ORC_UINT64) /* the tracing reduce */
                    orc_ucx_all_reduce(n, (const void* const*)send, recv, len, dtype, ORC_SUM, orc_trace_reduce2, NULL);
                for (uint32_t r = 0; r < n; r++) {
                    free(send[r]);
                    free(recv[r]);
                    free(recv2[r]);
                }
            }
        }
    }
    uint32_t ranks[16];
    int wins;
    uint32_t chunks;
    for (uint32_t n = 1; n <= 16; n++)
        for (int order = 0; order < 3; order++)
            for (int coll = 0; coll < 2; coll++) {
                orc_fold_order(coll, order, n, 0, ranks, &wins, &chunks);
                for (uint32_t c = 0; c < chunks; c++)
                    if (orc_fold_order(coll, order, n, c, ranks, &wins, NULL) != ORC_OK) failures++;
                if (orc_fold_order(coll, order, n, chunks, ranks, &wins, NULL) != ORC_BAD_ARG) failures++;
            }
    for (uint32_t h = 0; h < 65536; h++) {
        float f = orc_f16_to_f32((uint16_t)h);
        if (f == f && orc_f32_to_f16(f) != h) { printf("f16 roundtrip %x\n", h); failures++; }
    }
    printf(failures ? "selftest FAILED (%d)\n" : "selftest ok\n", failures);
    return failures ? 1 : 0;
}
