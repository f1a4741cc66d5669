// gfx950 kernels of the virtual-rank backend.
//
// fold_kernel / fold_flat_kernel
//              : every output element is a left fold, in a fixed rank order, over the same element
//                of K input buffers, stored to M output buffers.  They replace the 2-input
//                reduce_{sum,max,min}_kernel of the reference (src/ucx/kernel.cu:16-38) and the
//                cpu_reduce_kernel loop (src/shm/utils.cpp:16-37): a whole ring of N-1 two-input
//                steps on one chunk is one pass here, the ring order surviving as the fold order.
//                fold_flat_kernel is the fast form for K == rank count on aligned buffers;
//                fold_kernel takes everything else (any K, unaligned buffers, shifted copies).
// pack_kernel  : equally sized block copies between rank buffers (all_to_all / scatter / gather),
//                replacing the per-peer send/recv pairs of src/ucx/all_to_all.cpp:30-41,
//                src/ucx/scatter.cpp:30-44 and src/ucx/gather.cpp:30-44.
//
// All are pure streaming kernels: HBM-bound, one 128-bit access per lane per buffer, no LDS, no
// matrix instructions.  A workgroup is ONE 64-wide wavefront whose lanes read consecutive 16-byte
// vectors, so every load and store instruction covers one contiguous KiB and a tile is 1 KiB per
// buffer: on MI355X many small tiles sustain more HBM bandwidth than fewer large ones.
#include "vrank_kernels.h"

#include <hip/hip_runtime.h>

#include <type_traits>

namespace MegRay {
namespace vrank {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

enum : int { kSum = 0, kMax = 1, kMin = 2, kCopy = 3 };

// Accumulator type: FLOAT16 is widened to fp32, folded there and rounded once at the end.
template <typename T>
struct Wide {
    using type = T;
};
template <>
struct Wide<_Float16> {
    using type = float;
};

template <int OP, typename A>
__device__ __forceinline__ A combine(A acc, A x, bool new_wins) {
    if constexpr (OP == kSum) {
        return static_cast<A>(acc + x);  // unsigned element types: wraps
    } else if constexpr (OP == kMax) {
        if constexpr (std::is_floating_point<A>::value) {
            // explicit compare + select: ties, +-0 and NaN follow the reference's ?: exactly
            return new_wins ? ((acc > x) ? acc : x) : ((x > acc) ? x : acc);
        } else {
            return (x > acc) ? x : acc;
        }
    } else if constexpr (OP == kMin) {
        if constexpr (std::is_floating_point<A>::value) {
            return new_wins ? ((acc < x) ? acc : x) : ((x < acc) ? x : acc);
        } else {
            return (x < acc) ? x : acc;
        }
    } else {
        return x;
    }
}

template <typename T>
union VecOf {
    u32x4 raw;
    T v[kVecBytes / sizeof(T)];
};

__device__ __forceinline__ u32x4 load_vec(const char* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
}
__device__ __forceinline__ void store_vec(char* p, u32x4 x) {
    __builtin_nontemporal_store(x, reinterpret_cast<u32x4*>(p));
}

__device__ __forceinline__ uint32_t rotate_rank(uint32_t start, int dir, uint32_t j, uint32_t n) {
    // (start + dir*j) mod n for j < n, without a division
    if (dir > 0) {
        uint32_t r = start + j;
        return r >= n ? r - n : r;
    }
    return start >= j ? start - j : start + n - j;
}

template <typename T, int OP>
__device__ __forceinline__ u32x4 fold_vec(u32x4 acc_raw, u32x4 x_raw, bool new_wins) {
    using A = typename Wide<T>::type;
    VecOf<T> a, x;
    a.raw = acc_raw;
    x.raw = x_raw;
#pragma unroll
    for (uint32_t e = 0; e < kVecBytes / sizeof(T); ++e)
        a.v[e] = static_cast<T>(combine<OP, A>(static_cast<A>(a.v[e]), static_cast<A>(x.v[e]), new_wins));
    return a.raw;
}

// FLOAT16 keeps its accumulators in fp32 across the whole fold.
template <int OP>
struct HalfAcc {
    float v[8];
    __device__ __forceinline__ void seed(u32x4 raw) {
        VecOf<_Float16> x;
        x.raw = raw;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = static_cast<float>(x.v[e]);
    }
    __device__ __forceinline__ void fold(u32x4 raw, bool new_wins) {
        VecOf<_Float16> x;
        x.raw = raw;
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = combine<OP, float>(v[e], static_cast<float>(x.v[e]), new_wins);
    }
    __device__ __forceinline__ u32x4 finish() const {
        VecOf<_Float16> x;
#pragma unroll
        for (int e = 0; e < 8; ++e) x.v[e] = static_cast<_Float16>(v[e]);
        return x.raw;
    }
};

template <typename T, int OP>
struct VecAcc {
    u32x4 raw;
    __device__ __forceinline__ void seed(u32x4 r) { raw = r; }
    __device__ __forceinline__ void fold(u32x4 r, bool new_wins) { raw = fold_vec<T, OP>(raw, r, new_wins); }
    __device__ __forceinline__ u32x4 finish() const { return raw; }
};

template <typename T, int OP>
using AccFor = typename std::conditional<std::is_same<T, _Float16>::value, HalfAcc<OP>, VecAcc<T, OP>>::type;

// K > 0: fold count known at compile time, all K loads of a lane are issued before the first use.
// K == 0: fold count read from the launch, loads issued in groups of four.
template <typename T, int OP, int K, int U>
__global__ void __launch_bounds__(kThreads) fold_kernel(const FoldLaunch L) {
    using A = typename Wide<T>::type;
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    const uint32_t tile = blockIdx.x;
    // segment lookup: first_tile is ascending and padded with 0xffffffff, so the segment is the
    // number of entries <= tile, minus one; eight entries per scalar load
    uint32_t s = 0;
    for (uint32_t base = 0; base < L.nseg; base += 8) {
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) s += L.first_tile[base + i] <= tile ? 1u : 0u;
    }
    s -= 1;
    const uint64_t in_begin = L.seg[s].in_begin;
    const uint64_t out_begin = L.seg[s].out_begin;
    const uint64_t count = L.seg[s].count;
    const uint32_t local_tile = tile - L.first_tile[s];
    const uint32_t start = L.seg[s].start;
    const int dir = L.seg[s].dir;
    const uint32_t out_first = L.seg[s].out_first;
    const bool vector = (L.seg[s].flags & kSegVector) != 0;
    const uint32_t nr = L.nranks;
    const uint32_t nfold = K > 0 ? uint32_t(K) : L.nfold;
    const uint32_t nout = L.nout;
    const bool new_wins = L.new_wins_ties != 0;
    const uint32_t tid = threadIdx.x;

    if (vector) {
        const uint64_t nvec = count / EPV;
        const uint64_t vbase = uint64_t(local_tile) * (kThreads * U);
        const uint64_t in_off = in_begin * sizeof(T) + vbase * kVecBytes;
        const uint64_t out_off = out_begin * sizeof(T) + vbase * kVecBytes;
        const uint64_t left = nvec - vbase;  // vectors from this tile's start to the segment's end
        AccFor<T, OP> acc[U];
        if (left >= uint64_t(kThreads) * U) {
            // full tile: no predicates
            if constexpr (K > 0) {
                u32x4 x[K][U];
#pragma unroll
                for (int j = 0; j < K; ++j) {
                    const char* src = static_cast<const char*>(L.in[rotate_rank(start, dir, j, nr)]) + in_off;
#pragma unroll
                    for (int u = 0; u < U; ++u) x[j][u] = load_vec(src + (u * kThreads + tid) * kVecBytes);
                }
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    acc[u].seed(x[0][u]);
#pragma unroll
                    for (int j = 1; j < K; ++j) acc[u].fold(x[j][u], new_wins);
                }
            } else {
                {
                    const char* src = static_cast<const char*>(L.in[start]) + in_off;
#pragma unroll
                    for (int u = 0; u < U; ++u) acc[u].seed(load_vec(src + (u * kThreads + tid) * kVecBytes));
                }
                uint32_t j = 1;
                for (; j + 4 <= nfold; j += 4) {
                    u32x4 x[4][U];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        const char* src =
                                static_cast<const char*>(L.in[rotate_rank(start, dir, j + q, nr)]) + in_off;
#pragma unroll
                        for (int u = 0; u < U; ++u) x[q][u] = load_vec(src + (u * kThreads + tid) * kVecBytes);
                    }
#pragma unroll
                    for (int q = 0; q < 4; ++q)
#pragma unroll
                        for (int u = 0; u < U; ++u) acc[u].fold(x[q][u], new_wins);
                }
                for (; j < nfold; ++j) {
                    const char* src = static_cast<const char*>(L.in[rotate_rank(start, dir, j, nr)]) + in_off;
#pragma unroll
                    for (int u = 0; u < U; ++u)
                        acc[u].fold(load_vec(src + (u * kThreads + tid) * kVecBytes), new_wins);
                }
            }
            u32x4 res[U];
#pragma unroll
            for (int u = 0; u < U; ++u) res[u] = acc[u].finish();
            for (uint32_t m = 0; m < nout; ++m) {
                char* dst = static_cast<char*>(L.out[rotate_rank(out_first, 1, m, nr)]) + out_off;
#pragma unroll
                for (int u = 0; u < U; ++u) store_vec(dst + (u * kThreads + tid) * kVecBytes, res[u]);
            }
        } else {
            // last tile of the segment: predicate every vector
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const uint32_t v = u * kThreads + tid;
                if (v < left) {
                    AccFor<T, OP> a;
                    a.seed(load_vec(static_cast<const char*>(L.in[start]) + in_off + v * kVecBytes));
                    for (uint32_t j = 1; j < nfold; ++j)
                        a.fold(load_vec(static_cast<const char*>(L.in[rotate_rank(start, dir, j, nr)]) + in_off +
                                        v * kVecBytes),
                               new_wins);
                    const u32x4 r = a.finish();
                    for (uint32_t m = 0; m < nout; ++m)
                        store_vec(static_cast<char*>(L.out[rotate_rank(out_first, 1, m, nr)]) + out_off +
                                          v * kVecBytes,
                                  r);
                }
            }
        }
    } else {
        // element tiles: chunk heads / tails and buffers that are not 16-byte aligned
        const uint64_t ebase = uint64_t(local_tile) * (kThreads * U);
        const uint64_t left = count - ebase;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t e = u * kThreads + tid;
            if (e < left) {
                const uint64_t ie = in_begin + ebase + e;
                const uint64_t oe = out_begin + ebase + e;
                A a = static_cast<A>(static_cast<const T*>(L.in[start])[ie]);
                for (uint32_t j = 1; j < nfold; ++j)
                    a = combine<OP, A>(
                            a, static_cast<A>(static_cast<const T*>(L.in[rotate_rank(start, dir, j, nr)])[ie]),
                            new_wins);
                const T r = static_cast<T>(a);
                for (uint32_t m = 0; m < nout; ++m) static_cast<T*>(L.out[rotate_rank(out_first, 1, m, nr)])[oe] = r;
            }
        }
    }
}


// ---------------------------------------------------------------------------------------------
// Flat fold: tile t covers bytes [1024 t, 1024 t + 1024) of every input, whatever run it is in.
// The K loads of a lane therefore depend on nothing but blockIdx and the kernel arguments and are
// issued first; the run lookup (fold order, destinations) happens while they are in flight.

template <typename T, int OP, int K, int START, int DIR>
__device__ __forceinline__ u32x4 fold_static(const u32x4 (&x)[K], bool new_wins) {
    AccFor<T, OP> acc;
    acc.seed(x[START]);
#pragma unroll
    for (int j = 1; j < K; ++j) acc.fold(x[((START + DIR * j) % K + K) % K], new_wins);
    return acc.finish();
}

// Uniform dispatch on the seed rank: each case is a straight-line fold with fixed registers.
template <typename T, int OP, int K, int S = 0>
__device__ __forceinline__ u32x4 fold_from(const u32x4 (&x)[K], uint32_t start, int dir, bool new_wins) {
    if constexpr (S == K - 1) {
        return dir > 0 ? fold_static<T, OP, K, S, 1>(x, new_wins) : fold_static<T, OP, K, S, -1>(x, new_wins);
    } else {
        if (start == S)
            return dir > 0 ? fold_static<T, OP, K, S, 1>(x, new_wins) : fold_static<T, OP, K, S, -1>(x, new_wins);
        return fold_from<T, OP, K, S + 1>(x, start, dir, new_wins);
    }
}

template <typename T, int OP, int K>
__global__ void __launch_bounds__(kThreads) fold_flat_kernel(const FlatLaunch L) {
    using A = typename Wide<T>::type;
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;  // elements per tile
    const uint32_t tile = blockIdx.x;
    const uint32_t tid = threadIdx.x;
    const uint64_t byte_off = (uint64_t(tile) * kThreads + tid) * kVecBytes;
    const bool whole = (uint64_t(tile) + 1) * TILE <= L.count;  // tile lies inside the buffer

    u32x4 x[K];
    if (whole) {
#pragma unroll
        for (int r = 0; r < K; ++r) x[r] = load_vec(static_cast<const char*>(L.in[r]) + byte_off);
    }

    // run lookup, eight runs per pair of scalar loads
    int run = -1;
    for (uint32_t base = 0; base < L.nruns; base += 8) {
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i)
            if (tile >= L.tile_lo[base + i] && tile < L.tile_hi[base + i]) run = int(base + i);
    }
    const bool new_wins = L.new_wins_ties != 0;
    const uint32_t nout = L.nout;

    if (run >= 0) {
        // the whole tile shares one fold order (and lies inside the buffer)
        const uint32_t start = L.run[run].start;
        const int dir = L.run[run].dir;
        const uint32_t out_first = L.run[run].out_first;
        const uint64_t out_off = byte_off - uint64_t(L.run[run].out_shift) * sizeof(T);
        const u32x4 res = fold_from<T, OP, K>(x, start, dir, new_wins);
        if (nout == uint32_t(K)) {
#pragma unroll
            for (int m = 0; m < K; ++m) store_vec(static_cast<char*>(L.out[m]) + out_off, res);
        } else {
            for (uint32_t m = 0; m < nout; ++m)
                store_vec(static_cast<char*>(L.out[rotate_rank(out_first, 1, m, K)]) + out_off, res);
        }
        return;
    }

    // A tile that straddles a run border or the end of the buffer: element by element, one run at a
    // time so that ranks and destinations stay uniform.
    const uint64_t e_lo = uint64_t(tile) * TILE;
    const uint64_t e_hi = e_lo + TILE < L.count ? e_lo + TILE : L.count;
    for (uint32_t i = 0; i < L.nruns; ++i) {
        const uint64_t b = L.run[i].begin > e_lo ? L.run[i].begin : e_lo;
        const uint64_t e = L.run[i].end < e_hi ? L.run[i].end : e_hi;
        if (b >= e) continue;
        const uint32_t start = L.run[i].start;
        const int dir = L.run[i].dir;
        const uint32_t out_first = L.run[i].out_first;
        const uint64_t shift = uint64_t(L.run[i].out_shift);
        for (uint32_t k = 0; k < EPV; ++k) {
            const uint64_t el = e_lo + uint64_t(tid) * EPV + k;
            if (el < b || el >= e) continue;
            A a = static_cast<A>(static_cast<const T*>(L.in[start])[el]);
            for (uint32_t j = 1; j < uint32_t(K); ++j)
                a = combine<OP, A>(a, static_cast<A>(static_cast<const T*>(L.in[rotate_rank(start, dir, j, K)])[el]),
                                   new_wins);
            const T r = static_cast<T>(a);
            for (uint32_t m = 0; m < nout; ++m)
                static_cast<T*>(L.out[rotate_rank(out_first, 1, m, K)])[el - shift] = r;
        }
    }
}

template <typename W>
__device__ __forceinline__ W load_w(const char* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const W*>(p));
}
template <typename W>
__device__ __forceinline__ void store_w(char* p, W x) {
    __builtin_nontemporal_store(x, reinterpret_cast<W*>(p));
}

template <typename W, int U>
__global__ void __launch_bounds__(kThreads) pack_kernel(const PackLaunch L) {
    const uint32_t copy = blockIdx.x / L.tiles_per_copy;
    const uint32_t tile = blockIdx.x - copy * L.tiles_per_copy;
    const uint32_t n = L.nranks;
    uint32_t src_rank, dst_rank, src_block, dst_block;
    if (L.mode == kPackAllToAll) {
        src_rank = copy / n;
        src_block = copy - src_rank * n;
        dst_rank = src_block;
        dst_block = src_rank;
    } else if (L.mode == kPackScatter) {
        src_rank = L.root;
        src_block = copy;
        dst_rank = copy;
        dst_block = 0;
    } else {
        src_rank = copy;
        src_block = 0;
        dst_rank = L.root;
        dst_block = copy;
    }
    const uint64_t base = uint64_t(tile) * (kThreads * U) * sizeof(W);
    const char* src = static_cast<const char*>(L.in[src_rank]) + src_block * L.block_bytes + base;
    char* dst = static_cast<char*>(L.out[dst_rank]) + dst_block * L.block_bytes + base;
    const uint64_t left = (L.block_bytes - base) / sizeof(W);
    const uint32_t tid = threadIdx.x;
    if (left >= uint64_t(kThreads) * U) {
        W x[U];
#pragma unroll
        for (int u = 0; u < U; ++u) x[u] = load_w<W>(src + (u * kThreads + tid) * sizeof(W));
#pragma unroll
        for (int u = 0; u < U; ++u) store_w<W>(dst + (u * kThreads + tid) * sizeof(W), x[u]);
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const uint32_t i = u * kThreads + tid;
            if (i < left) store_w<W>(dst + i * sizeof(W), load_w<W>(src + i * sizeof(W)));
        }
    }
}

using FoldFn = void (*)(const FoldLaunch);

template <typename T, int OP>
FoldFn pick_fold(uint32_t nfold) {
    switch (nfold) {
        case 2: return fold_kernel<T, OP, 2, fold_unroll(2)>;
        case 3: return fold_kernel<T, OP, 3, fold_unroll(3)>;
        case 4: return fold_kernel<T, OP, 4, fold_unroll(4)>;
        case 8: return fold_kernel<T, OP, 8, fold_unroll(8)>;
        default: return fold_kernel<T, OP, 0, fold_unroll(0)>;
    }
}

template <typename T>
FoldFn pick_minmax(int op, uint32_t nfold) {
    return op == kMax ? pick_fold<T, kMax>(nfold) : pick_fold<T, kMin>(nfold);
}

FoldFn pick_copy(uint32_t elem_size) {
    switch (elem_size) {
        case 1: return fold_kernel<uint8_t, kCopy, 1, fold_unroll(1)>;
        case 2: return fold_kernel<uint16_t, kCopy, 1, fold_unroll(1)>;
        case 4: return fold_kernel<uint32_t, kCopy, 1, fold_unroll(1)>;
        default: return fold_kernel<uint64_t, kCopy, 1, fold_unroll(1)>;
    }
}


using FlatFn = void (*)(const FlatLaunch);

template <typename T, int OP>
FlatFn pick_flat(uint32_t nranks) {
    switch (nranks) {
        case 2: return fold_flat_kernel<T, OP, 2>;
        case 3: return fold_flat_kernel<T, OP, 3>;
        case 4: return fold_flat_kernel<T, OP, 4>;
        case 8: return fold_flat_kernel<T, OP, 8>;
        default: return nullptr;
    }
}

template <typename T>
FlatFn pick_flat_minmax(int op, uint32_t nranks) {
    return op == kMax ? pick_flat<T, kMax>(nranks) : pick_flat<T, kMin>(nranks);
}

}  // namespace

hipError_t launch_fold(const FoldLaunch& L, DType dtype, ReduceOp op, hipStream_t stream) {
    if (L.total_tiles == 0) return hipSuccess;
    FoldFn fn = nullptr;
    if (L.nfold == 1) {
        fn = pick_copy(L.elem_size);
    } else if (op == MEGRAY_SUM) {
        // integer SUM wraps: computed in the unsigned type of the same width for both signs
        switch (dtype) {
            case MEGRAY_INT8:
            case MEGRAY_UINT8: fn = pick_fold<uint8_t, kSum>(L.nfold); break;
            case MEGRAY_INT32:
            case MEGRAY_UINT32: fn = pick_fold<uint32_t, kSum>(L.nfold); break;
            case MEGRAY_INT64:
            case MEGRAY_UINT64: fn = pick_fold<uint64_t, kSum>(L.nfold); break;
            case MEGRAY_FLOAT16: fn = pick_fold<_Float16, kSum>(L.nfold); break;
            case MEGRAY_FLOAT32: fn = pick_fold<float, kSum>(L.nfold); break;
            case MEGRAY_FLOAT64: fn = pick_fold<double, kSum>(L.nfold); break;
            default: return hipErrorInvalidValue;
        }
    } else if (op == MEGRAY_MAX || op == MEGRAY_MIN) {
        switch (dtype) {
            case MEGRAY_INT8: fn = pick_minmax<int8_t>(op, L.nfold); break;
            case MEGRAY_UINT8: fn = pick_minmax<uint8_t>(op, L.nfold); break;
            case MEGRAY_INT32: fn = pick_minmax<int32_t>(op, L.nfold); break;
            case MEGRAY_UINT32: fn = pick_minmax<uint32_t>(op, L.nfold); break;
            case MEGRAY_INT64: fn = pick_minmax<int64_t>(op, L.nfold); break;
            case MEGRAY_UINT64: fn = pick_minmax<uint64_t>(op, L.nfold); break;
            case MEGRAY_FLOAT16: fn = pick_minmax<_Float16>(op, L.nfold); break;
            case MEGRAY_FLOAT32: fn = pick_minmax<float>(op, L.nfold); break;
            case MEGRAY_FLOAT64: fn = pick_minmax<double>(op, L.nfold); break;
            default: return hipErrorInvalidValue;
        }
    } else {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(fn, dim3(L.total_tiles), dim3(kThreads), 0, stream, L);
    return hipGetLastError();
}


hipError_t launch_flat(const FlatLaunch& L, DType dtype, ReduceOp op, hipStream_t stream) {
    if (L.total_tiles == 0) return hipSuccess;
    FlatFn fn = nullptr;
    if (op == MEGRAY_SUM) {
        switch (dtype) {
            case MEGRAY_INT8:
            case MEGRAY_UINT8: fn = pick_flat<uint8_t, kSum>(L.nranks); break;
            case MEGRAY_INT32:
            case MEGRAY_UINT32: fn = pick_flat<uint32_t, kSum>(L.nranks); break;
            case MEGRAY_INT64:
            case MEGRAY_UINT64: fn = pick_flat<uint64_t, kSum>(L.nranks); break;
            case MEGRAY_FLOAT16: fn = pick_flat<_Float16, kSum>(L.nranks); break;
            case MEGRAY_FLOAT32: fn = pick_flat<float, kSum>(L.nranks); break;
            case MEGRAY_FLOAT64: fn = pick_flat<double, kSum>(L.nranks); break;
            default: return hipErrorInvalidValue;
        }
    } else if (op == MEGRAY_MAX || op == MEGRAY_MIN) {
        switch (dtype) {
            case MEGRAY_INT8: fn = pick_flat_minmax<int8_t>(op, L.nranks); break;
            case MEGRAY_UINT8: fn = pick_flat_minmax<uint8_t>(op, L.nranks); break;
            case MEGRAY_INT32: fn = pick_flat_minmax<int32_t>(op, L.nranks); break;
            case MEGRAY_UINT32: fn = pick_flat_minmax<uint32_t>(op, L.nranks); break;
            case MEGRAY_INT64: fn = pick_flat_minmax<int64_t>(op, L.nranks); break;
            case MEGRAY_UINT64: fn = pick_flat_minmax<uint64_t>(op, L.nranks); break;
            case MEGRAY_FLOAT16: fn = pick_flat_minmax<_Float16>(op, L.nranks); break;
            case MEGRAY_FLOAT32: fn = pick_flat_minmax<float>(op, L.nranks); break;
            case MEGRAY_FLOAT64: fn = pick_flat_minmax<double>(op, L.nranks); break;
            default: return hipErrorInvalidValue;
        }
    }
    if (!fn) return hipErrorInvalidValue;
    hipLaunchKernelGGL(fn, dim3(L.total_tiles), dim3(kThreads), 0, stream, L);
    return hipGetLastError();
}

hipError_t launch_pack(const PackLaunch& L, hipStream_t stream) {
    const uint64_t blocks = uint64_t(L.ncopies) * L.tiles_per_copy;
    if (blocks == 0) return hipSuccess;
    void (*fn)(const PackLaunch) = nullptr;
    switch (L.width) {
        case 16: fn = pack_kernel<u32x4, pack_unroll()>; break;
        case 8: fn = pack_kernel<u32x2, pack_unroll()>; break;
        case 4: fn = pack_kernel<uint32_t, pack_unroll()>; break;
        case 2: fn = pack_kernel<uint16_t, pack_unroll()>; break;
        case 1: fn = pack_kernel<uint8_t, pack_unroll()>; break;
        default: return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(fn, dim3(uint32_t(blocks)), dim3(kThreads), 0, stream, L);
    return hipGetLastError();
}

}  // namespace vrank
}  // namespace MegRay
