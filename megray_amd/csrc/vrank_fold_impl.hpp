// Templates of the fold kernels of the virtual-rank backend (gfx950).  Included by one translation
// unit per element type (vrank_fold_<type>.hip), each of which instantiates the launchers for its
// type, so that the types compile in parallel.
//
// Every output element is a combination, in a fixed rank order, of the same element of K input
// buffers, stored to M output buffers.  The kernels replace the 2-input reduce_{sum,max,min}_kernel
// of the reference (src/ucx/kernel.cu:16-38) and the cpu_reduce_kernel loop
// (src/shm/utils.cpp:16-37): a whole ring of N-1 two-input steps on one chunk is one pass here, the
// ring order surviving as the fold order.
//
//   flat launches     K == rank count in {2, 3, 4, 8}, buffers 16-byte aligned: tile t is the same
//                     KiB of every buffer, so loads need nothing but the block index.
//                     fold_group_kernel (2048 tiles and more) / fold_flat_kernel (fewer).
//   segment launches  any K, buffers that share an offset from a 16-byte boundary or none at all,
//                     shifted copies: head / vector body / tail segments cut by the planner.
//                     fold_segment_group_kernel (long vector bodies) / fold_kernel.
//   fold_tree_kernel  element-wise binomial tree for rank counts without a flat kernel.
//
// All are pure streaming kernels: HBM-bound, one 128-bit access per lane per buffer, no matrix
// instructions.  A wavefront's lanes read consecutive 16-byte vectors, so every load and store
// instruction covers one contiguous KiB, and a tile is 1 KiB per buffer.  The kernels for short
// launches run one wavefront per tile.  The group kernels run four wavefronts per workgroup on four
// tiles that lie 32 tiles apart and pass the tiles between the wavefronts through LDS, so that the
// accesses one wavefront issues together go to different tiles: on MI355X that sustains 80 - 85 %
// of the HBM peak where one wavefront per tile reaches 64 - 76 %, depending on where the caller's
// buffers happen to lie.
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "vrank_kernels.h"

namespace MegRay {
namespace vrank {
namespace detail {

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

// 128-bit accesses of single lanes at any byte address (gfx950 serves them; the pointer type tells the compiler
// not to assume more): buffers at any element offset go 16 bytes per lane.
typedef uint32_t u32x4_a1 __attribute__((ext_vector_type(4), aligned(1)));
__device__ __forceinline__ u32x4 load_vec(const char* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const u32x4_a1*>(p));
}
__device__ __forceinline__ void store_vec(char* p, u32x4 x) {
    __builtin_nontemporal_store(u32x4_a1(x), reinterpret_cast<u32x4_a1*>(p));
}

// One tile (1 KiB) of a buffer through buffer instructions with explicit cache policies: measured
// against plain non-temporal global accesses on MI355X (8 in + 8 out, fp32), non-temporal buffer
// loads plus "sc1 nt" buffer stores sustain about 5 % more HBM bandwidth.  Launches that write little
// (kKeepMaxBytes in vrank_types.h) store "sc1" without "nt", which leaves the data in the last-level cache;
// `keep` is uniform over the launch, so the choice is a scalar branch.
typedef int32_t i32x4 __attribute__((ext_vector_type(4)));
constexpr int kLoadPolicy = 2;        // nt
constexpr int kStorePolicy = 18;      // sc1 | nt
constexpr int kStoreKeepPolicy = 16;  // sc1
constexpr int kRsrcFlags = 0x00020000;  // raw 32-bit data format, no swizzle

__device__ __forceinline__ u32x4 load_tile_vec(const void* tile_base, uint32_t lane) {
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
            const_cast<void*>(tile_base), 0, int(kThreads * kVecBytes), kRsrcFlags);
    return __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, int(lane * kVecBytes), 0, kLoadPolicy));
}
__device__ __forceinline__ void store_tile_vec(void* tile_base, uint32_t lane, u32x4 x, bool keep) {
    __amdgpu_buffer_rsrc_t rsrc =
            __builtin_amdgcn_make_buffer_rsrc(tile_base, 0, int(kThreads * kVecBytes), kRsrcFlags);
    if (keep)
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, x), rsrc, int(lane * kVecBytes), 0, kStoreKeepPolicy);
    else
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(i32x4, x), rsrc, int(lane * kVecBytes), 0, kStorePolicy);
}

// The same for tiles that may start at any byte address (segments of 1- and 2-byte elements whose inputs are
// shifted against the outputs, or whose buffers lie at differing offsets): buffer instructions need a 4-byte
// boundary, so other tiles go lane by lane.  The test is uniform over the wavefront.
__device__ __forceinline__ u32x4 load_tile_any(const char* tile_base, uint32_t lane) {
    if ((reinterpret_cast<uintptr_t>(tile_base) & 3u) == 0) return load_tile_vec(tile_base, lane);
    return load_vec(tile_base + lane * kVecBytes);
}
__device__ __forceinline__ void store_tile_any(char* tile_base, uint32_t lane, u32x4 x, bool keep) {
    if ((reinterpret_cast<uintptr_t>(tile_base) & 3u) == 0) store_tile_vec(tile_base, lane, x, keep);
    else store_vec(tile_base + lane * kVecBytes, x);
}
// The same for tiles of elements of type T: buffers of 4- and 8-byte elements are element aligned wherever a kernel
// takes them a vector at a time, so their tiles always sit on 4-byte boundaries.  Leaving the other path out of those
// kernels matters beyond the test it saves: it is made of flat instructions, which complete out of order with the
// buffer instructions around them, and a kernel that contains both waits for everything outstanding wherever it
// waits at all - a wavefront's loads, and its stores to several ranks, then go one at a time.
template <typename T>
__device__ __forceinline__ u32x4 load_tile_of(const char* tile_base, uint32_t lane) {
    if constexpr (sizeof(T) >= 4) return load_tile_vec(tile_base, lane);
    else return load_tile_any(tile_base, lane);
}
template <typename T>
__device__ __forceinline__ void store_tile_of(char* tile_base, uint32_t lane, u32x4 x, bool keep) {
    if constexpr (sizeof(T) >= 4) store_tile_vec(tile_base, lane, x, keep);
    else store_tile_any(tile_base, lane, x, keep);
}

// One element at byte `offset` (a multiple of the element size, below 1 KiB) of a tile, with the tile stores' cache
// policy: written through, so that the kernel's end finds nothing to write back (a plain store leaves its line dirty
// in the L2, and a short launch then waits for the write-back).
template <typename T>
__device__ __forceinline__ void store_tile_element(char* tile_base, uint32_t offset, T value, bool keep) {
    if ((reinterpret_cast<uintptr_t>(tile_base) & 3u) != 0) {
        *reinterpret_cast<T*>(tile_base + offset) = value;
        return;
    }
    __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(tile_base, 0, int(kThreads * kVecBytes), kRsrcFlags);
    if constexpr (sizeof(T) == 1) {
        const auto bits = __builtin_bit_cast(uint8_t, value);
        if (keep) __builtin_amdgcn_raw_buffer_store_b8(bits, rsrc, int(offset), 0, kStoreKeepPolicy);
        else __builtin_amdgcn_raw_buffer_store_b8(bits, rsrc, int(offset), 0, kStorePolicy);
    } else if constexpr (sizeof(T) == 2) {
        const auto bits = __builtin_bit_cast(uint16_t, value);
        if (keep) __builtin_amdgcn_raw_buffer_store_b16(bits, rsrc, int(offset), 0, kStoreKeepPolicy);
        else __builtin_amdgcn_raw_buffer_store_b16(bits, rsrc, int(offset), 0, kStorePolicy);
    } else if constexpr (sizeof(T) == 4) {
        const auto bits = __builtin_bit_cast(uint32_t, value);
        if (keep) __builtin_amdgcn_raw_buffer_store_b32(bits, rsrc, int(offset), 0, kStoreKeepPolicy);
        else __builtin_amdgcn_raw_buffer_store_b32(bits, rsrc, int(offset), 0, kStorePolicy);
    } else {
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        const auto bits = __builtin_bit_cast(u32x2, value);
        if (keep) __builtin_amdgcn_raw_buffer_store_b64(bits, rsrc, int(offset), 0, kStoreKeepPolicy);
        else __builtin_amdgcn_raw_buffer_store_b64(bits, rsrc, int(offset), 0, kStorePolicy);
    }
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
    __device__ __forceinline__ void merge(const HalfAcc& other) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = combine<OP, float>(v[e], other.v[e], false);
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
    __device__ __forceinline__ void merge(const VecAcc& other) { raw = fold_vec<T, OP>(raw, other.raw, false); }
    __device__ __forceinline__ u32x4 finish() const { return raw; }
};

// int8 / uint8: the sixteen bytes of a vector are kept as 2 x 4 registers of packed 16-bit lanes
// (even bytes and odd bytes of each 32-bit word, sign- or zero-extended), so that one packed
// 16-bit add / max / min handles two elements.  SUM wraps mod 256 because only the low byte of
// each lane is kept at the end.
typedef int16_t i16x2 __attribute__((ext_vector_type(2)));
typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));

template <typename T, int OP>
struct ByteAcc {
    using Lanes = typename std::conditional<std::is_signed<T>::value, i16x2, u16x2>::type;
    Lanes even[4], odd[4];

    static __device__ __forceinline__ void split(uint32_t w, Lanes& ev, Lanes& od) {
        if constexpr (std::is_signed<T>::value) {
            const i16x2 lanes = __builtin_bit_cast(i16x2, w);
            ev = (lanes << 8) >> 8;  // arithmetic shift: sign-extends the low byte of each lane
            od = lanes >> 8;
        } else {
            ev = __builtin_bit_cast(u16x2, w & 0x00ff00ffu);
            od = __builtin_bit_cast(u16x2, (w >> 8) & 0x00ff00ffu);
        }
    }
    static __device__ __forceinline__ Lanes op(Lanes a, Lanes b) {
        if constexpr (OP == kSum) {
            return a + b;
        } else if constexpr (OP == kMax) {
            return __builtin_elementwise_max(a, b);
        } else {
            return __builtin_elementwise_min(a, b);
        }
    }
    __device__ __forceinline__ void seed(u32x4 raw) {
#pragma unroll
        for (int w = 0; w < 4; ++w) split(raw[w], even[w], odd[w]);
    }
    __device__ __forceinline__ void fold(u32x4 raw, bool) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            Lanes ev, od;
            split(raw[w], ev, od);
            even[w] = op(even[w], ev);
            odd[w] = op(odd[w], od);
        }
    }
    __device__ __forceinline__ void merge(const ByteAcc& other) {
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            even[w] = op(even[w], other.even[w]);
            odd[w] = op(odd[w], other.odd[w]);
        }
    }
    __device__ __forceinline__ u32x4 finish() const {
        u32x4 raw;
#pragma unroll
        for (int w = 0; w < 4; ++w)
            raw[w] = (__builtin_bit_cast(uint32_t, even[w]) & 0x00ff00ffu) |
                     ((__builtin_bit_cast(uint32_t, odd[w]) & 0x00ff00ffu) << 8);
        return raw;
    }
};

// int8 / uint8 SUM: four bytes per 32-bit register are added at once.  The low seven bits of every
// byte are added with the top bits masked off, so no carry crosses a byte border, and the top bits
// are put back with an exclusive or: exactly the byte-wise sum mod 256.
struct ByteSumAcc {
    u32x4 raw;
    static __device__ __forceinline__ u32x4 add(u32x4 a, u32x4 b) {
        const u32x4 low = (a & 0x7f7f7f7fu) + (b & 0x7f7f7f7fu);
        return low ^ ((a ^ b) & 0x80808080u);
    }
    __device__ __forceinline__ void seed(u32x4 r) { raw = r; }
    __device__ __forceinline__ void fold(u32x4 r, bool) { raw = add(raw, r); }
    __device__ __forceinline__ void merge(const ByteSumAcc& other) { raw = add(raw, other.raw); }
    __device__ __forceinline__ u32x4 finish() const { return raw; }
};

// Accumulator of a left fold: bytes in packed form (element by element they compile to several
// instructions per byte and spill), FLOAT16 in fp32, everything else element-wise in its own type.
template <typename T, int OP>
using ByteAccFor = typename std::conditional<
        OP == kSum, ByteSumAcc,
        typename std::conditional<OP == kMax || OP == kMin, ByteAcc<T, OP>, VecAcc<T, OP>>::type>::type;

template <typename T, int OP>
using AccFor = typename std::conditional<
        sizeof(T) == 1, ByteAccFor<T, OP>,
        typename std::conditional<std::is_same<T, _Float16>::value, HalfAcc<OP>, VecAcc<T, OP>>::type>::type;

template <typename T, int OP>
using TreeAccFor = AccFor<T, OP>;

// The segment a workgroup works in, found from its tile number: first_tile is ascending and padded
// with 0xffffffff, so the segment is the number of entries <= tile, minus one; eight entries per
// scalar load.
struct SegmentView {
    uint64_t in_begin, out_begin, count;
    uint32_t local_tile, start, out_first;
    int dir;
    bool vector, deal;
};
__device__ __forceinline__ SegmentView find_segment(const FoldLaunch& L, uint32_t tile) {
    uint32_t s = 0;
    for (uint32_t base = 0; base < L.nseg; base += 8) {
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) s += L.first_tile[base + i] <= tile ? 1u : 0u;
    }
    s -= 1;
    SegmentView sv;
    sv.in_begin = L.seg[s].in_begin;
    sv.out_begin = L.seg[s].out_begin;
    sv.count = L.seg[s].count;
    sv.local_tile = tile - L.first_tile[s];
    sv.start = L.seg[s].start;
    sv.dir = L.seg[s].dir;
    sv.out_first = L.seg[s].out_first;
    sv.vector = (L.seg[s].flags & kSegVector) != 0;
    sv.deal = (L.seg[s].flags & kSegDeal) != 0;
    return sv;
}

// Where a kernel finds its rank pointers.  ArgPtrs reads them from the launch descriptor as they are needed: a
// scalar load per pointer whose index is known only after the segment lookup, one more memory round trip before
// the first data load.  LanePtrs holds the tables in a register instead - lane l the descriptor's in[l], lane
// kMaxRanks + l its out[l], read by the whole wavefront at once when the kernel starts - and picks by readlane.
struct ArgPtrs {
    const FoldLaunch& L;
    __device__ __forceinline__ const char* in(uint32_t r) const { return static_cast<const char*>(L.in[r]); }
    __device__ __forceinline__ char* out(uint32_t r) const { return static_cast<char*>(L.out[r]); }
};
struct LanePtrs {
    uint32_t lo, hi;
    __device__ __forceinline__ char* pick(uint32_t lane) const {
        const uint64_t a = uint64_t(uint32_t(__builtin_amdgcn_readlane(int(lo), int(lane)))) |
                           uint64_t(uint32_t(__builtin_amdgcn_readlane(int(hi), int(lane)))) << 32;
        return reinterpret_cast<char*>(a);
    }
    __device__ __forceinline__ const char* in(uint32_t r) const { return pick(r); }
    __device__ __forceinline__ char* out(uint32_t r) const { return pick(kMaxRanks + r); }
};
static_assert(2 * kMaxRanks == kThreads, "one lane per entry of in[] and out[]");
static_assert(offsetof(FoldLaunch, out) == offsetof(FoldLaunch, in) + kMaxRanks * sizeof(void*), "out[] follows in[]");
static_assert(sizeof(FoldSegment) == 32 && kMaxSegments >= kThreads, "a lane reads one segment, two vectors");

// What a one-wavefront kernel reads of its launch descriptor before anything else, every lane its share, all four
// loads in flight together: lane l holds first_tile[l], seg[l] and one rank pointer.  The segment lookup is then a
// ballot and a handful of readlanes, and the rank pointers are at hand: one memory round trip between the kernel's
// start and its first data load, where the scalar lookup (find_segment, then seg[s], then in[r]) takes three.
struct LaneArgs {
    uint32_t first_tile;
    u32x4 seg_a, seg_b;
    LanePtrs ptrs;
};
__device__ __forceinline__ LaneArgs load_lane_args(uint32_t lane) {
    using Constant = const __attribute__((address_space(4))) char;
    Constant* base = (Constant*)__builtin_amdgcn_kernarg_segment_ptr();  // the descriptor is the only argument
    LaneArgs a;
    a.first_tile = *reinterpret_cast<const __attribute__((address_space(4))) uint32_t*>(
            base + offsetof(FoldLaunch, first_tile) + lane * sizeof(uint32_t));
    const auto* seg = reinterpret_cast<const __attribute__((address_space(4))) u32x4*>(
            base + offsetof(FoldLaunch, seg) + lane * sizeof(FoldSegment));
    a.seg_a = seg[0];
    a.seg_b = seg[1];
    const auto* ptr = reinterpret_cast<const __attribute__((address_space(4))) uint32_t*>(
            base + offsetof(FoldLaunch, in) + lane * sizeof(void*));
    a.ptrs.lo = ptr[0];
    a.ptrs.hi = ptr[1];
    return a;
}
// (launches of more than kThreads segments - 22 and more ranks off the vector grid - look the segment up the scalar way)
__device__ __forceinline__ SegmentView find_segment(const FoldLaunch& L, const LaneArgs& a, uint32_t tile) {
    if (L.nseg > kThreads) return find_segment(L, tile);
    const uint32_t s = uint32_t(__popcll(__ballot(a.first_tile <= tile))) - 1u;
    const auto pick = [&](uint32_t v) { return uint32_t(__builtin_amdgcn_readlane(int(v), int(s))); };
    SegmentView sv;
    sv.in_begin = uint64_t(pick(a.seg_a.x)) | uint64_t(pick(a.seg_a.y)) << 32;
    sv.out_begin = uint64_t(pick(a.seg_a.z)) | uint64_t(pick(a.seg_a.w)) << 32;
    sv.count = uint64_t(pick(a.seg_b.x)) | uint64_t(pick(a.seg_b.y)) << 32;
    sv.local_tile = tile - pick(a.first_tile);
    const uint32_t bytes = pick(a.seg_b.w);  // start, dir, out_first, flags
    sv.start = bytes & 0xffu;
    sv.dir = int(int8_t((bytes >> 8) & 0xffu));
    sv.out_first = (bytes >> 16) & 0xffu;
    sv.vector = ((bytes >> 24) & kSegVector) != 0;
    sv.deal = ((bytes >> 24) & kSegDeal) != 0;
    return sv;
}

// Element tiles: run heads / tails and buffers that are not 16-byte aligned.  A lane takes
// elems_per_lane(L) elements, a wavefront's lanes consecutive ones, four at a time; the loads of up to eight ranks
// are in flight together (one memory round trip for up to nine inputs, not one per input).
template <typename T, int OP, typename P>
__device__ __forceinline__ void fold_element_tile(const FoldLaunch& L, const P& ptrs, const SegmentView& sv, uint32_t nfold,
                                                  uint32_t local_tile, uint32_t tid) {
    using A = typename Wide<T>::type;
    constexpr uint32_t G = 4, B = 8;
    const uint64_t in_begin = sv.in_begin, out_begin = sv.out_begin, count = sv.count;
    const uint32_t start = sv.start, out_first = sv.out_first, nr = L.nranks, nout = L.nout;
    const int dir = sv.dir;
    const bool new_wins = L.new_wins_ties != 0;
    const uint32_t per_lane = elems_per_lane(L);
    const uint64_t ebase = uint64_t(local_tile) * (kThreads * per_lane);
    for (uint32_t g = 0; g < per_lane; g += G) {
        const uint64_t gbase = ebase + uint64_t(g) * kThreads;
        if (gbase >= count) break;
        const uint64_t left = count - gbase;
        const uint64_t ie = in_begin + gbase + tid;
        const uint64_t oe = out_begin + gbase + tid;
        bool have[G];
#pragma unroll
        for (uint32_t q = 0; q < G; ++q) have[q] = uint64_t(q) * kThreads + tid < left;
        A a[G];
        const T* seed = reinterpret_cast<const T*>(ptrs.in(start)) + ie;
#pragma unroll
        for (uint32_t q = 0; q < G; ++q) a[q] = have[q] ? static_cast<A>(seed[q * kThreads]) : A(0);
        for (uint32_t j0 = 1; j0 < nfold; j0 += B) {
            T x[B][G];
#pragma unroll
            for (uint32_t b = 0; b < B; ++b) {
                if (j0 + b < nfold) {
                    const T* src = reinterpret_cast<const T*>(ptrs.in(rotate_rank(start, dir, j0 + b, nr))) + ie;
#pragma unroll
                    for (uint32_t q = 0; q < G; ++q) x[b][q] = have[q] ? src[q * kThreads] : T(0);
                }
            }
#pragma unroll
            for (uint32_t b = 0; b < B; ++b) {
                if (j0 + b < nfold) {
#pragma unroll
                    for (uint32_t q = 0; q < G; ++q) a[q] = combine<OP, A>(a[q], static_cast<A>(x[b][q]), new_wins);
                }
            }
        }
        for (uint32_t m = 0; m < nout; ++m) {
            T* dst = reinterpret_cast<T*>(ptrs.out(rotate_rank(out_first, 1, m, nr))) + oe;
#pragma unroll
            for (uint32_t q = 0; q < G; ++q)
                if (have[q]) dst[q * kThreads] = static_cast<T>(a[q]);
        }
    }
}

// Up to kThreads vectors at vector index `vbase` of a segment, each lane folding one vector by itself
// with plain global accesses: the incomplete last group of a segment's vector body.
template <typename T, int OP, typename P>
__device__ __forceinline__ void fold_vector_remainder(const FoldLaunch& L, const P& ptrs, const SegmentView& sv, uint32_t nfold,
                                                      uint64_t vbase, uint64_t left, uint32_t tid) {
    if (tid >= left) return;
    const uint32_t nr = L.nranks;
    const bool new_wins = L.new_wins_ties != 0;
    const uint64_t in_off = sv.in_begin * sizeof(T) + (vbase + tid) * kVecBytes;
    const uint64_t out_off = sv.out_begin * sizeof(T) + (vbase + tid) * kVecBytes;
    AccFor<T, OP> a;
    // the loads of up to eight ranks in flight together, every batch size and the stores as straight-line code (see fold_tile)
    const auto batch = [&](auto count, uint32_t j0) {
        constexpr uint32_t C = decltype(count)::value;
        u32x4 x[C];
#pragma unroll
        for (uint32_t q = 0; q < C; ++q) x[q] = load_vec(ptrs.in(rotate_rank(sv.start, sv.dir, j0 + q, nr)) + in_off);
        if (j0 == 0) a.seed(x[0]);
        else a.fold(x[0], new_wins);
#pragma unroll
        for (uint32_t q = 1; q < C; ++q) a.fold(x[q], new_wins);
    };
    uint32_t j0 = 0;
    for (; j0 + 8 <= nfold; j0 += 8) batch(std::integral_constant<uint32_t, 8>{}, j0);
    switch (nfold - j0) {
        case 1: batch(std::integral_constant<uint32_t, 1>{}, j0); break;
        case 2: batch(std::integral_constant<uint32_t, 2>{}, j0); break;
        case 3: batch(std::integral_constant<uint32_t, 3>{}, j0); break;
        case 4: batch(std::integral_constant<uint32_t, 4>{}, j0); break;
        case 5: batch(std::integral_constant<uint32_t, 5>{}, j0); break;
        case 6: batch(std::integral_constant<uint32_t, 6>{}, j0); break;
        case 7: batch(std::integral_constant<uint32_t, 7>{}, j0); break;
        default: break;
    }
    const u32x4 r = a.finish();
    const auto put = [&](auto count, uint32_t m0) {
        constexpr uint32_t C = decltype(count)::value;
#pragma unroll
        for (uint32_t q = 0; q < C; ++q) store_vec(ptrs.out(rotate_rank(sv.out_first, 1, m0 + q, nr)) + out_off, r);
    };
    const uint32_t nout = L.nout;
    uint32_t m0 = 0;
    for (; m0 + 8 <= nout; m0 += 8) put(std::integral_constant<uint32_t, 8>{}, m0);
    switch (nout - m0) {
        case 1: put(std::integral_constant<uint32_t, 1>{}, m0); break;
        case 2: put(std::integral_constant<uint32_t, 2>{}, m0); break;
        case 3: put(std::integral_constant<uint32_t, 3>{}, m0); break;
        case 4: put(std::integral_constant<uint32_t, 4>{}, m0); break;
        case 5: put(std::integral_constant<uint32_t, 5>{}, m0); break;
        case 6: put(std::integral_constant<uint32_t, 6>{}, m0); break;
        case 7: put(std::integral_constant<uint32_t, 7>{}, m0); break;
        default: break;
    }
}

// Every lane polls the same word (one request per wavefront) until it reaches `target` or the time
// limit passes; each lane's acquire keeps its own loads behind the wait.  false: the group is poisoned
// (a wait gave up before, or this one does now) and the kernel must not store.
__device__ __forceinline__ bool hook_wait(const EdgeHooks& h, uint64_t target) {
    const uint64_t begin = wall_clock64();
    while (__hip_atomic_load(h.words, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < target) {
        if (__hip_atomic_load(h.words + 2, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT)) return false;
        if (wall_clock64() - begin > h.limit_ticks) {
            if (threadIdx.x == 0) {
                if (__hip_atomic_fetch_add(h.words + 2, uint64_t(1), __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == 0)
                    __hip_atomic_store(h.words + 4, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if (h.status) {
                    __hip_atomic_store(h.status + 1, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                    __hip_atomic_fetch_add(h.status, uint64_t(1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
                }
            }
            return false;
        }
        __builtin_amdgcn_s_sleep(1);
    }
    return __hip_atomic_load(h.words + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0;
}

// The poison of the group a launch belongs to (0 for launches outside a group).  Issued early, tested
// before the first store: the load rides along with the tile loads and costs the kernel no round trip.
__device__ __forceinline__ uint64_t hook_poison(const EdgeHooks& h) {
    return h.words ? __hip_atomic_load(h.words + 2, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : uint64_t(0);
}

// What the one-wavefront kernels do first: wait if the launch says so, and find out whether they may store.
__device__ __forceinline__ bool hook_enter(const EdgeHooks& h, uint64_t target) {
    if (target) return hook_wait(h, target);
    return hook_poison(h) == 0;
}

// After a one-wavefront workgroup's stores: count it, and let the last one publish the ticket.
// (Only short launches do this: the release fence writes the L2 back, once per workgroup; from a few
// hundred workgroups on that costs more than a separate notify kernel, and at 2560 workgroups it
// alone took ten times as long as the fold.)
__device__ __forceinline__ void hook_publish(const EdgeHooks& h, uint64_t ticket) {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // this wavefront's stores before its count
    if (threadIdx.x == 0) {
        const uint64_t before = __hip_atomic_fetch_add(h.words + 3, uint64_t(1), __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        if (before + 1 == gridDim.x) {
            __hip_atomic_store(h.words + 3, uint64_t(0), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            __hip_atomic_store(h.words + 1, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

// One wavefront per tile, for short launches.
// K > 0: fold count known at compile time, all K loads of a lane are issued before the first use.
// K == 0: fold count read from the launch, loads issued in groups of four.
template <typename T, int OP, int K>
__device__ __forceinline__ void fold_tile(const FoldLaunch& L, const LaneArgs& args) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    const SegmentView sv = find_segment(L, args, blockIdx.x);
    const LanePtrs& ptrs = args.ptrs;
    const uint32_t local_tile = sv.local_tile, start = sv.start, out_first = sv.out_first;
    const int dir = sv.dir;
    const uint32_t nr = L.nranks;
    const uint32_t nfold = K > 0 ? uint32_t(K) : L.nfold;
    const uint32_t nout = L.nout;
    const bool new_wins = L.new_wins_ties != 0;
    const uint32_t tid = threadIdx.x;

    if (sv.vector) {
        // A tile is kVecIters groups of kThreads vectors, taken one after the other: the segment
        // lookup above is paid once per tile while the registers of one group suffice.
        const uint64_t nvec = sv.count / EPV;
        const uint32_t iters = vec_iters(L);
        for (uint32_t it = 0; it < iters; ++it) {
            const uint64_t vbase = (uint64_t(local_tile) * iters + it) * kThreads;
            if (vbase >= nvec) break;
            const uint64_t left = nvec - vbase;  // vectors from this group's start to the segment's end
            if (left < kThreads) {
                fold_vector_remainder<T, OP>(L, ptrs, sv, nfold, vbase, left, tid);
                break;
            }
            const uint64_t in_off = sv.in_begin * sizeof(T) + vbase * kVecBytes;
            const uint64_t out_off = sv.out_begin * sizeof(T) + vbase * kVecBytes;
            AccFor<T, OP> acc;
            if constexpr (K > 0) {
                u32x4 x[K];
#pragma unroll
                for (int j = 0; j < K; ++j)
                    x[j] = load_tile_of<T>(ptrs.in(rotate_rank(start, dir, j, nr)) + in_off, tid);
                acc.seed(x[0]);
#pragma unroll
                for (int j = 1; j < K; ++j) acc.fold(x[j], new_wins);
            } else {
                // seven inputs at a time in flight, the seed among the first (eight cost twice the registers).  Every
                // batch size is straight-line code of its own: loads guarded one by one leave the compiler with values that
                // are defined on some paths only, which it copies at every join - after waiting for every load before it.
                const auto batch = [&](auto count, uint32_t j0) {
                    constexpr uint32_t C = decltype(count)::value;
                    u32x4 x[C];
#pragma unroll
                    for (uint32_t q = 0; q < C; ++q)
                        x[q] = load_tile_of<T>(ptrs.in(rotate_rank(start, dir, j0 + q, nr)) + in_off, tid);
                    if (j0 == 0) acc.seed(x[0]);
                    else acc.fold(x[0], new_wins);
#pragma unroll
                    for (uint32_t q = 1; q < C; ++q) acc.fold(x[q], new_wins);
                };
                uint32_t j0 = 0;
                for (; j0 + 7 <= nfold; j0 += 7) batch(std::integral_constant<uint32_t, 7>{}, j0);
                switch (nfold - j0) {
                    case 1: batch(std::integral_constant<uint32_t, 1>{}, j0); break;
                    case 2: batch(std::integral_constant<uint32_t, 2>{}, j0); break;
                    case 3: batch(std::integral_constant<uint32_t, 3>{}, j0); break;
                    case 4: batch(std::integral_constant<uint32_t, 4>{}, j0); break;
                    case 5: batch(std::integral_constant<uint32_t, 5>{}, j0); break;
                    case 6: batch(std::integral_constant<uint32_t, 6>{}, j0); break;
                    default: break;
                }
            }
            const u32x4 res = acc.finish();
            // the stores likewise, eight at a time and either policy on a path of its own: in a loop the compiler waits
            // for each store before it issues the next
            const auto put = [&](auto count, auto kept, uint32_t m0) {
                constexpr uint32_t C = decltype(count)::value;
#pragma unroll
                for (uint32_t q = 0; q < C; ++q)
                    store_tile_of<T>(ptrs.out(rotate_rank(out_first, 1, m0 + q, nr)) + out_off, tid, res, decltype(kept)::value);
            };
            const auto put_all = [&](auto kept) {
                uint32_t m0 = 0;
                for (; m0 + 8 <= nout; m0 += 8) put(std::integral_constant<uint32_t, 8>{}, kept, m0);
                switch (nout - m0) {
                    case 1: put(std::integral_constant<uint32_t, 1>{}, kept, m0); break;
                    case 2: put(std::integral_constant<uint32_t, 2>{}, kept, m0); break;
                    case 3: put(std::integral_constant<uint32_t, 3>{}, kept, m0); break;
                    case 4: put(std::integral_constant<uint32_t, 4>{}, kept, m0); break;
                    case 5: put(std::integral_constant<uint32_t, 5>{}, kept, m0); break;
                    case 6: put(std::integral_constant<uint32_t, 6>{}, kept, m0); break;
                    case 7: put(std::integral_constant<uint32_t, 7>{}, kept, m0); break;
                    default: break;
                }
            };
            if (L.keep != 0) put_all(std::true_type{});
            else put_all(std::false_type{});
        }
    } else {
        fold_element_tile<T, OP>(L, ptrs, sv, nfold, local_tile, tid);
    }
}

template <typename T, int OP, int K>
__global__ void __launch_bounds__(kThreads) fold_kernel(const FoldLaunch L) {
    const LaneArgs args = load_lane_args(threadIdx.x);  // issued first: nothing below depends on less
    if (!hook_enter(L.hooks, L.hook_target)) return;
    fold_tile<T, OP, K>(L, args);
    if (L.hook_ticket) hook_publish(L.hooks, L.hook_ticket);
}

// Group form of the segment fold for launches whose vector bodies are long (L.waves == kGroupWaves).
// A workgroup of kGroupWaves wavefronts owns kGroupWaves groups of kThreads vectors of one segment
// (1 KiB per buffer each) that lie kGroupStride such groups apart.  Wavefront w loads fold position
// j of group (w + j) % kGroupWaves, the groups are exchanged through LDS, wavefront w folds group
// w, and with several destinations the results are exchanged again so that wavefront w stores
// destination m of group (w + m) % kGroupWaves.  With the fold count read from the launch (K == 0)
// the inputs pass through LDS four at a time.  Element segments are the work of wavefront 0 alone.
template <typename T, int OP, int K>
__global__ void __launch_bounds__(kThreads * kGroupWaves) fold_segment_group_kernel(const FoldLaunch L) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t W = kGroupWaves;
    constexpr uint32_t SK = K > 0 ? uint32_t(K) : 4u;  // inputs staged at a time
    constexpr uint32_t kGroupBytes = kThreads * kVecBytes;
    __shared__ u32x4 stage[W][SK][kThreads];
    __shared__ u32x4 result[W][kThreads];
    __shared__ uint32_t folded[W];
    const SegmentView sv = find_segment(L, blockIdx.x);
    const uint32_t tid = threadIdx.x % kThreads;
    const uint32_t wave = uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x / kThreads)));
    const uint32_t nr = L.nranks;
    const uint32_t nfold = K > 0 ? uint32_t(K) : L.nfold;
    const uint32_t nout = L.nout;
    const bool new_wins = L.new_wins_ties != 0;
    // A launch of a communicator group stores nothing once the group is poisoned (the test masks stores only: the
    // wavefronts of a workgroup may see the poison rise at different moments and must all reach the barriers).
    const bool live = hook_poison(L.hooks) == 0;
    if (!sv.vector) {
        if (wave == 0 && live) fold_element_tile<T, OP>(L, ArgPtrs{L}, sv, nfold, sv.local_tile, tid);
        return;
    }
    const uint64_t nvec = sv.count / EPV;
    const uint64_t whole_groups = nvec / kThreads;  // groups of kThreads vectors that are complete
    // Consecutive workgroups run on different XCDs, each with an L2 of its own.  Where the tiles do not sit on the
    // cache lines of every buffer (inputs shifted against the outputs), neighbouring tiles share a line, so the
    // workgroups of eight runs of kGroupStride (one run = 4 * kGroupStride consecutive tiles) are dealt out such
    // that a whole run goes to one XCD and the shared lines are fetched into one L2 only (reduce_scatter of 8 x
    // 32 MiB fp32 with an odd receive length: 74 -> 83 % of the HBM peak).  Tiles on line boundaries keep the
    // plain order, which serves them 1 - 4 points better.
    uint32_t local = sv.local_tile;
    if (sv.deal) {
        constexpr uint32_t kXcds = 8, kDeal = kXcds * kGroupStride;
        const uint32_t wgs = uint32_t((nvec + kThreads - 1) / kThreads + W * kGroupStride - 1) / (W * kGroupStride) * kGroupStride;
        if (local < wgs / kDeal * kDeal) {
            const uint32_t w = local % kDeal;
            local = local - w + (w % kXcds) * kGroupStride + w / kXcds;
        }
    }
    const uint64_t first = uint64_t(local / kGroupStride) * (W * kGroupStride) + local % kGroupStride;
    const uint64_t mine = first + wave * kGroupStride;
    const bool have = mine < whole_groups;
    const uint64_t in_base = sv.in_begin * sizeof(T), out_base = sv.out_begin * sizeof(T);

    AccFor<T, OP> acc;
    if constexpr (K == 1) {
        // a copy: nothing to skew on the load side
        if (have) acc.seed(load_tile_of<T>(static_cast<const char*>(L.in[sv.start]) + in_base + mine * kGroupBytes, tid));
    } else {
        // Long launches keep two loads per wavefront in flight instead of all SK (L.paced, as in the flat group
        // kernel): load q + 2 is issued when load q has arrived.
        const bool paced = L.paced != 0;
        constexpr uint32_t D = SK < kGroupLoadsInFlight ? SK : kGroupLoadsInFlight;
        for (uint32_t j0 = 0; j0 < nfold; j0 += SK) {
            const auto load_input = [&](uint32_t q, uint32_t lane) -> u32x4 {
                const uint64_t group = first + ((wave + q) % W) * kGroupStride;
                if (j0 + q < nfold && group < whole_groups)
                    return load_tile_of<T>(static_cast<const char*>(L.in[rotate_rank(sv.start, sv.dir, j0 + q, nr)]) +
                                                 in_base + group * kGroupBytes,
                                         lane);
                return u32x4{0u, 0u, 0u, 0u};
            };
            u32x4 x[SK];
#pragma unroll
            for (uint32_t q = 0; q < D; ++q) x[q] = load_input(q, tid);
            if (!paced) {
#pragma unroll
                for (uint32_t q = D; q < SK; ++q) x[q] = load_input(q, tid);
            }
            if (K == 0 && j0) __syncthreads();  // the previous four have been folded by everyone
#pragma unroll
            for (uint32_t q = 0; q < SK; ++q) {
                if (paced && q + D < SK) {
                    uint32_t lane = tid;
                    asm volatile("" : "+v"(lane) : "v"(x[q]));  // the next load's address waits for x[q]
                    x[q + D] = load_input(q + D, lane);
                }
                stage[(wave + q) % W][q][tid] = x[q];
            }
            __syncthreads();
            if (have) {
#pragma unroll
                for (uint32_t q = 0; q < SK; ++q) {
                    if (j0 + q >= nfold) break;
                    if (j0 + q == 0)
                        acc.seed(stage[wave][q][tid]);
                    else
                        acc.fold(stage[wave][q][tid], new_wins);
                }
            }
        }
    }
    // the segment's incomplete last group of vectors belongs to whoever owns its index
    if (mine == whole_groups && nvec % kThreads && live)
        fold_vector_remainder<T, OP>(L, ArgPtrs{L}, sv, nfold, mine * kThreads, nvec % kThreads, tid);

    if (nout == 1) {
        if (have && live)
            store_tile_of<T>(static_cast<char*>(L.out[sv.out_first]) + out_base + mine * kGroupBytes, tid, acc.finish(), L.keep != 0);
        return;
    }
    if (have) result[wave][tid] = acc.finish();
    if (tid == 0) folded[wave] = have ? 1u : 0u;
    __syncthreads();
    for (uint32_t m = 0; m < nout; ++m) {
        const uint32_t k = (wave + m) % W;
        if (folded[k] && live)
            store_tile_of<T>(static_cast<char*>(L.out[rotate_rank(sv.out_first, 1, m, nr)]) + out_base +
                                   (first + uint64_t(k) * kGroupStride) * kGroupBytes,
                           tid, result[k][tid], L.keep != 0);
        if (L.paced && (m + 1) % kGroupStoresInFlight == 0 && m + 1 < nout) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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

// Binomial tree towards virtual rank 0 = actual rank ROOT (src/ucx/reduce.cpp:56-80): in round
// `bit`, virtual rank v (a multiple of 2*bit) takes in v + bit as reduce(incoming, own), which
// keeps its own value on a MAX/MIN tie.
template <typename T, int OP, int K, int ROOT>
__device__ __forceinline__ u32x4 tree_static(const u32x4 (&x)[K]) {
    TreeAccFor<T, OP> a[K];
#pragma unroll
    for (int v = 0; v < K; ++v) a[v].seed(x[(v + ROOT) % K]);
#pragma unroll
    for (int bit = 1; bit < K; bit <<= 1) {
#pragma unroll
        for (int v = 0; v + bit < K; v += 2 * bit) a[v].merge(a[v + bit]);
    }
    return a[0].finish();
}

template <typename T, int OP, int K, int S = 0>
__device__ __forceinline__ u32x4 tree_from(const u32x4 (&x)[K], uint32_t root) {
    if constexpr (S == K - 1) {
        return tree_static<T, OP, K, S>(x);
    } else {
        if (root == S) return tree_static<T, OP, K, S>(x);
        return tree_from<T, OP, K, S + 1>(x, root);
    }
}

// The same tree on one element.  N > 0: rank count known at compile time (registers only);
// N == 0: read from `n` (the element-wise kernel for arbitrary rank counts).
template <typename T, int OP, int N, typename Launch>
__device__ __forceinline__ T tree_element(const Launch& L, uint32_t n, uint32_t root, uint64_t el) {
    using A = typename Wide<T>::type;
    constexpr uint32_t CAP = N > 0 ? uint32_t(N) : kMaxRanks;
    const uint32_t count = N > 0 ? uint32_t(N) : n;
    A a[CAP];
#pragma unroll
    for (uint32_t v = 0; v < CAP; ++v)
        if (v < count) a[v] = static_cast<A>(static_cast<const T*>(L.in[rotate_rank(root, 1, v, count)])[el]);
#pragma unroll
    for (uint32_t bit = 1; bit < CAP; bit <<= 1) {
#pragma unroll
        for (uint32_t v = 0; v + bit < CAP; v += 2 * bit)
            if (v + bit < count) a[v] = combine<OP, A>(a[v], a[v + bit], false);
    }
    return static_cast<T>(a[0]);
}

// The same tree on the 16-byte vector at byte offset `off` of up to kMaxRanks buffers.  The subtree of SPAN virtual
// ranks from v0 is its left half combined with its right half, if there is one: that is the expression the rounds of
// the element-wise form build.  It is evaluated eight leaves at a time: the loads of a batch are straight-line code for
// every batch size and all in flight together, the subtree of a batch is fixed at compile time, and the up to four
// batch values are combined by the same rule.  (The plain recursive walk, tree_walk below, tests the rank count at every
// node; that leaves the compiler with loads on some paths only, and it waits for each before it issues the next, so
// that a wavefront has two or three loads in flight.  Long launches of few ranks and 4- or 8-byte elements whose
// stores stream are served best that way, and keep it: TreeLaunch::batch.)
// TILE: `off` is the byte offset of a whole tile, loaded with one buffer instruction per rank (lane `tid`
// takes its vector of it); otherwise `off` is the lane's own vector.
template <typename T, int OP, uint32_t SPAN, uint32_t C>
__device__ __forceinline__ TreeAccFor<T, OP> tree_of_batch(const u32x4* x) {  // C of the SPAN leaves exist, 1 <= C <= SPAN
    if constexpr (SPAN == 1) {
        TreeAccFor<T, OP> a;
        a.seed(x[0]);
        return a;
    } else {
        constexpr uint32_t H = SPAN / 2;
        TreeAccFor<T, OP> left = tree_of_batch<T, OP, H, (C < H ? C : H)>(x);
        if constexpr (C > H) left.merge(tree_of_batch<T, OP, H, C - H>(x + H));
        return left;
    }
}
// (the rank pointers come out of a register that holds the descriptor's in[], lane l entry l: see LanePtrs)
struct TreeRanks {
    LanePtrs ptrs;
    uint32_t root, nranks, batch;
};
__device__ __forceinline__ TreeRanks load_tree_ranks(const TreeLaunch& L, uint32_t lane) {
    using Constant = const __attribute__((address_space(4))) char;
    Constant* base = (Constant*)__builtin_amdgcn_kernarg_segment_ptr();  // the descriptor is the only argument
    const auto* ptr = reinterpret_cast<const __attribute__((address_space(4))) uint32_t*>(
            base + offsetof(TreeLaunch, in) + (lane % kMaxRanks) * sizeof(void*));
    TreeRanks r;
    r.ptrs.lo = ptr[0];
    r.ptrs.hi = ptr[1];
    r.root = L.root;
    r.nranks = L.nranks;
    r.batch = L.batch;
    return r;
}
template <typename T, int OP, bool TILE, uint32_t B, uint32_t C>
__device__ __forceinline__ TreeAccFor<T, OP> tree_batch(const TreeRanks& L, uint64_t off, uint32_t v0, uint32_t tid) {
    u32x4 x[C];
#pragma unroll
    for (uint32_t q = 0; q < C; ++q) {
        const char* base = L.ptrs.in(rotate_rank(L.root, 1, v0 + q, L.nranks)) + off;
        if constexpr (TILE) x[q] = load_tile_of<T>(base, tid);
        else x[q] = load_vec(base);
    }
    return tree_of_batch<T, OP, B, C>(x);
}
template <typename T, int OP, bool TILE, uint32_t B>
__device__ __forceinline__ TreeAccFor<T, OP> tree_batch_of(const TreeRanks& L, uint64_t off, uint32_t v0, uint32_t tid) {
    const uint32_t left = L.nranks - v0;  // leaves from v0 on: a whole batch, or what is left
    if constexpr (B >= 8) {
        switch (left) {
            case 7: return tree_batch<T, OP, TILE, B, 7>(L, off, v0, tid);
            case 6: return tree_batch<T, OP, TILE, B, 6>(L, off, v0, tid);
            case 5: return tree_batch<T, OP, TILE, B, 5>(L, off, v0, tid);
            case 4: return tree_batch<T, OP, TILE, B, 4>(L, off, v0, tid);
            default: break;
        }
    }
    if constexpr (B >= 4) {
        switch (left) {
            case 3: return tree_batch<T, OP, TILE, B, 3>(L, off, v0, tid);
            case 2: return tree_batch<T, OP, TILE, B, 2>(L, off, v0, tid);
            default: break;
        }
    }
    if (left == 1) return tree_batch<T, OP, TILE, B, 1>(L, off, v0, tid);
    return tree_batch<T, OP, TILE, B, B>(L, off, v0, tid);
}
// the batch values of SPAN batches from batch b0, combined by the same rule
template <typename T, int OP, bool TILE, uint32_t B, uint32_t SPAN>
__device__ __forceinline__ TreeAccFor<T, OP> tree_top(const TreeRanks& L, uint64_t off, uint32_t b0, uint32_t tid) {
    if constexpr (SPAN == 1) {
        return tree_batch_of<T, OP, TILE, B>(L, off, b0 * B, tid);
    } else {
        TreeAccFor<T, OP> left = tree_top<T, OP, TILE, B, SPAN / 2>(L, off, b0, tid);
        if ((b0 + SPAN / 2) * B < L.nranks) left.merge(tree_top<T, OP, TILE, B, SPAN / 2>(L, off, b0 + SPAN / 2, tid));
        return left;
    }
}
// The plain recursive walk, one leaf at a time, rank pointers read from the descriptor as they are needed (see above).
template <typename T, int OP, uint32_t SPAN, bool TILE>
__device__ __forceinline__ TreeAccFor<T, OP> tree_walk(const TreeLaunch& L, uint64_t off, uint32_t v0, uint32_t tid) {
    if constexpr (SPAN == 1) {
        TreeAccFor<T, OP> a;
        const char* base = static_cast<const char*>(L.in[rotate_rank(L.root, 1, v0, L.nranks)]) + off;
        if constexpr (TILE) a.seed(load_tile_of<T>(base, tid));
        else a.seed(load_vec(base));
        return a;
    } else {
        TreeAccFor<T, OP> left = tree_walk<T, OP, SPAN / 2, TILE>(L, off, v0, tid);
        if (v0 + SPAN / 2 < L.nranks) left.merge(tree_walk<T, OP, SPAN / 2, TILE>(L, off, v0 + SPAN / 2, tid));
        return left;
    }
}
template <typename T, int OP, bool TILE>
__device__ __forceinline__ TreeAccFor<T, OP> tree_node(const TreeRanks& L, uint64_t off, uint32_t tid) {
    return tree_top<T, OP, TILE, 8, kMaxRanks / 8>(L, off, 0, tid);
}

template <typename T, int OP>
__device__ __forceinline__ u32x4 tree_vector(const TreeRanks& L, uint64_t off) {
    return tree_node<T, OP, false>(L, off, 0).finish();
}

template <typename T, int OP>
__device__ __forceinline__ void tree_tile(const TreeLaunch& L, const TreeRanks& ranks) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    const uint64_t lane = uint64_t(blockIdx.x) * kThreads + threadIdx.x;
    if (!L.vector) {
        if (lane < L.count) static_cast<T*>(L.out)[lane] = tree_element<T, OP, 0>(L, L.nranks, L.root, lane);
        return;
    }
    const uint64_t nvec = L.count / EPV;
    const uint64_t tile_off = uint64_t(blockIdx.x) * kThreads * kVecBytes;
    if ((uint64_t(blockIdx.x) + 1) * kThreads <= nvec) {
        // a whole tile: buffer instructions with the streaming cache policies
        const u32x4 r = L.batch == 1 ? tree_walk<T, OP, kMaxRanks, true>(L, tile_off, 0, threadIdx.x).finish()
                                     : tree_node<T, OP, true>(ranks, tile_off, threadIdx.x).finish();
        store_tile_of<T>(static_cast<char*>(L.out) + tile_off, threadIdx.x, r, L.keep != 0);
    } else if (lane < nvec) {
        store_vec(static_cast<char*>(L.out) + lane * kVecBytes, tree_vector<T, OP>(ranks, lane * kVecBytes));
    }
    // the elements behind the last whole vector: the first lanes of the last workgroup
    if (blockIdx.x == gridDim.x - 1 && threadIdx.x < L.count % EPV) {
        const uint64_t el = nvec * EPV + threadIdx.x;
        static_cast<T*>(L.out)[el] = tree_element<T, OP, 0>(L, L.nranks, L.root, el);
    }
}

template <typename T, int OP>
__global__ void __launch_bounds__(kThreads) fold_tree_kernel(const TreeLaunch L) {
    const TreeRanks ranks = load_tree_ranks(L, threadIdx.x);  // issued first
    if (!hook_enter(L.hooks, L.hook_target)) return;
    tree_tile<T, OP>(L, ranks);
    if (L.hook_ticket) hook_publish(L.hooks, L.hook_ticket);
}

// The run tables of a flat launch are kernel arguments read through scalar loads.  Written naively
// (short-circuit conditions, one field at a time) every entry becomes a load of its own that the next
// compare waits for, sixteen and more in a row; the helpers below fetch eight runs with a few wide
// loads that are all in flight together, and only the tables the launch needs.
struct RunBatch {
    uint64_t begin0;    // where the first run of the batch begins
    uint64_t end[8];
    uint32_t meta[8];
    uint64_t shift[8];
    __device__ __forceinline__ uint64_t begin(uint32_t i) const { return i ? end[i - 1] : begin0; }
};

__device__ __forceinline__ RunBatch load_batch(const FlatLaunch& L, uint32_t base) {
    RunBatch b;
    b.begin0 = base ? L.end[base - 1] : 0;
    __builtin_memcpy(b.end, &L.end[base], sizeof(b.end));
    __builtin_memcpy(b.meta, &L.meta[base], sizeof(b.meta));
    if (L.unshifted) {
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) b.shift[i] = 0;
    } else {
        __builtin_memcpy(b.shift, &L.shift[base], sizeof(b.shift));
    }
    return b;
}
__device__ __forceinline__ uint32_t meta_start(uint32_t meta) { return meta & 0xffu; }
__device__ __forceinline__ int meta_dir(uint32_t meta) { return int(int8_t((meta >> 8) & 0xffu)); }
__device__ __forceinline__ uint32_t meta_out_first(uint32_t meta) { return (meta >> 16) & 0xffu; }

// The run that holds all of a tile, if there is one (everything here is uniform: scalar registers).
struct TileRun {
    bool covered = false;
    uint32_t meta = 1u << 8;
    uint64_t shift = 0;
};
__device__ __forceinline__ void uniform_scan(const RunBatch& b, uint64_t e_lo, uint64_t e_hi, TileRun& tr) {
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
        const bool covers = (b.begin(i) <= e_lo) & (e_hi <= b.end[i]);  // unused entries end at 0
        tr.covered = tr.covered | covers;
        tr.meta = covers ? b.meta[i] : tr.meta;
        tr.shift = covers ? b.shift[i] : tr.shift;
    }
}

// What a lane knows about the run its own 16-byte vector lies in.
struct LaneRun {
    bool inside = false;  // the vector lies wholly inside one run (whose order and destinations follow)
    bool cut = false;     // the vector is cut by a run border
    uint32_t meta = 1u << 8;
    uint32_t shift_lo = 0, shift_hi = 0;  // the run's out_shift: a whole number of vectors in a flat launch
};

// Eight runs against the lanes of tile `tile`, without branches (unused entries end at 0 and match
// nothing).  A run's borders are clamped to the tile on the scalar side, so the per-lane part is 32-bit.
template <typename T>
__device__ __forceinline__ void lane_scan(const RunBatch& w, uint32_t tile, uint32_t tid, LaneRun& lr) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;
    const uint64_t e_lo = uint64_t(tile) * TILE;
    const uint32_t lane_off = tid * EPV;  // the lane's vector, in elements from the tile's start
#pragma unroll
    for (uint32_t i = 0; i < 8; ++i) {
        const uint64_t b64 = w.begin(i) > e_lo ? w.begin(i) - e_lo : 0;
        const uint64_t e64 = w.end[i] > e_lo ? w.end[i] - e_lo : 0;
        const uint32_t b = uint32_t(b64 < TILE ? b64 : TILE), e = uint32_t(e64 < TILE ? e64 : TILE);
        const bool holds = (lane_off >= b) & (lane_off + EPV <= e);
        lr.cut = lr.cut | (!holds & (lane_off < e) & (lane_off + EPV > b));
        lr.inside = lr.inside | holds;
        lr.meta = holds ? w.meta[i] : lr.meta;
        lr.shift_lo = holds ? uint32_t(w.shift[i]) : lr.shift_lo;
        lr.shift_hi = holds ? uint32_t(w.shift[i] >> 32) : lr.shift_hi;
    }
}

// A tile that lies inside the buffers but straddles run borders, its K input vectors staged in LDS as
// staged[r][lane].  Every lane has looked up the run its own vector lies in (LaneRun); the lanes whose vector lies
// wholly inside one run fold it in that run's order, fetching the inputs from LDS by rank: one straight pass
// whatever the number of runs in the tile, which is what the smallest messages consist of (8 ranks x 4 KiB: every
// tile holds two chunks).  Returns the folded vector (of those lanes); `store`: also stores it to the run's outputs.
// Lanes whose vector a run border cuts are left to flat_tile_ragged.
template <typename T, int OP, int K, bool TREE>
__device__ __forceinline__ u32x4 flat_tile_whole_vectors(const FlatLaunch& L, uint32_t tile, uint32_t tid,
                                                         const u32x4 (*staged)[kThreads], const LaneRun& lr, bool store) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;
    u32x4 res = {0u, 0u, 0u, 0u};
    if (!lr.inside) return res;
    const bool new_wins = L.new_wins_ties != 0;
    const uint32_t start = meta_start(lr.meta), out_first = meta_out_first(lr.meta);
    const int dir = meta_dir(lr.meta);
    if constexpr (TREE) {
        u32x4 x[K];
#pragma unroll
        for (int r = 0; r < K; ++r) x[r] = staged[r][tid];
        res = tree_from<T, OP, K>(x, start);
    } else {
        AccFor<T, OP> acc;
        acc.seed(staged[start][tid]);
#pragma unroll
        for (uint32_t j = 1; j < uint32_t(K); ++j) acc.fold(staged[rotate_rank(start, dir, j, K)][tid], new_wins);
        res = acc.finish();
    }
    if (store) {
        const uint64_t shift = uint64_t(lr.shift_lo) | (uint64_t(lr.shift_hi) << 32);
        const uint64_t out_el = uint64_t(tile) * TILE + uint64_t(tid) * EPV - shift;
#pragma unroll 1
        for (uint32_t m = 0; m < L.nout; ++m)
            store_vec(reinterpret_cast<char*>(static_cast<T*>(L.out[rotate_rank(out_first, 1, m, K)]) + out_el), res);
    }
    return res;
}

// The buffers' last tile, which their end cuts: x[r] = this lane's vector of input r, lane by lane (nothing may be
// read beyond the end), zero where the buffers have ended.  The vector that the end cuts is put together in LDS:
// the elements that exist are loaded one per lane (all of them in flight together) and written where they belong in
// a vector of zeros, which the lane that owns it then reads back.  `cut` is LDS of the workgroup that only the one
// wavefront holding this tile touches (a wavefront's LDS instructions execute in order).
template <typename T, int K>
__device__ __forceinline__ void load_tile_at_the_end(const FlatLaunch& L, uint32_t tile, uint32_t tid, u32x4 (&x)[K],
                                                     u32x4* cut) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;
    const uint64_t e_lo = uint64_t(tile) * TILE;
    const uint32_t nvalid = uint32_t(L.count - e_lo);  // below TILE
    const uint32_t nfull = nvalid / EPV, ntail = nvalid % EPV;
    T last[K];
#pragma unroll
    for (int r = 0; r < K; ++r) {
        const T* p = static_cast<const T*>(L.in[r]) + e_lo;
        x[r] = u32x4{0u, 0u, 0u, 0u};
        if (tid < nfull) x[r] = load_vec(reinterpret_cast<const char*>(p + tid * EPV));
        last[r] = T(0);
        if (tid < ntail) last[r] = __builtin_nontemporal_load(p + nfull * EPV + tid);
    }
    if (!ntail) return;
    if (tid < uint32_t(K)) cut[tid] = u32x4{0u, 0u, 0u, 0u};
    __builtin_amdgcn_wave_barrier();
    if (tid < ntail) {
#pragma unroll
        for (int r = 0; r < K; ++r) reinterpret_cast<T*>(&cut[r])[tid] = last[r];
    }
    __builtin_amdgcn_wave_barrier();
    if (tid == nfull) {
#pragma unroll
        for (int r = 0; r < K; ++r) x[r] = cut[r];
    }
}

// One tile of a flat launch that no single run covers, or that the buffers' end cuts.  staged[r][lane] (LDS) is the lane's
// vector of input r (zero where the buffers have ended); `pending` lanes have not stored their vector yet.  Run by run (uniform;
// the runs that reach into the tile are found with eight runs per round of scalar loads, they are in order and none
// is empty): the whole wavefront folds its vectors in that run's order, and every pending lane stores what of its
// vector lies in the run - the whole vector if all of it does, else element by element (chunk lengths need not be
// multiples of a vector, so a border may cut one, and so may the buffers' end).  No second pass over memory.
template <typename T, int OP, int K, bool TREE, bool MERGE>
__device__ __forceinline__ void flat_tile_ragged(const FlatLaunch& L, uint32_t tile, uint32_t tid,
                                                 const u32x4 (*staged)[kThreads], bool pending, u32x4& merged) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;
    const uint64_t e_lo = uint64_t(tile) * TILE;
    const uint64_t e_hi = e_lo + TILE < L.count ? e_lo + TILE : L.count;
    const uint32_t lane_off = tid * EPV;  // the lane's vector, in elements from the tile's start
    const bool new_wins = L.new_wins_ties != 0;
    const bool keep = (L.exchange & kFlatKeep) != 0;
    const uint32_t nout = L.nout;
    uint32_t first_run = L.nruns, last_run = 0;
    for (uint32_t base = 0; base < L.nruns; base += 8) {
        const RunBatch w = load_batch(L, base);
        if (w.begin0 >= e_hi) break;
#pragma unroll
        for (uint32_t i = 0; i < 8; ++i) {
            const bool reaches = (w.begin(i) < e_hi) & (w.end[i] > e_lo);  // unused entries end at 0
            first_run = reaches && base + i < first_run ? base + i : first_run;
            last_run = reaches ? base + i : last_run;
        }
    }
    // one run at a time (not unrolled: one copy of the fold, whose seed rank and direction are uniform)
#pragma unroll 1
    for (uint32_t i = first_run; i <= last_run && i < L.nruns; ++i) {
        const uint64_t run_begin = i ? L.end[i - 1] : 0, run_end = L.end[i];
        const uint32_t b = uint32_t((run_begin > e_lo ? run_begin : e_lo) - e_lo);
        const uint32_t e = uint32_t((run_end < e_hi ? run_end : e_hi) - e_lo);
        const uint32_t meta = L.meta[i];
        const uint32_t start = meta_start(meta), out_first = meta_out_first(meta);
        const int dir = meta_dir(meta);
        const uint64_t shift = L.unshifted ? 0 : L.shift[i];
        // the inputs come from LDS by rank, in the run's order: no copy of the fold per seed rank, no registers held
        u32x4 res;
        if constexpr (TREE) {
            u32x4 y[K];
#pragma unroll
            for (int v = 0; v < K; ++v) y[v] = staged[rotate_rank(start, 1, uint32_t(v), K)][tid];
            res = tree_static<T, OP, K, 0>(y);
        } else {
            AccFor<T, OP> acc;
            acc.seed(staged[start][tid]);
#pragma unroll
            for (uint32_t j = 1; j < uint32_t(K); ++j) acc.fold(staged[rotate_rank(start, dir, j, K)][tid], new_wins);
            res = acc.finish();
        }
        const uint32_t lo = lane_off > b ? lane_off : b;
        const uint32_t hi = lane_off + EPV < e ? lane_off + EPV : e;
        if (!pending || lo >= hi) continue;
        VecOf<T> v;
        v.raw = res;
        if constexpr (MERGE) {
            // every rank receives the whole tile at the inputs' offsets: the lane collects its vector, the caller stores it
            VecOf<T> sum;
            sum.raw = merged;
#pragma unroll
            for (uint32_t k = 0; k < EPV; ++k)
                if (lane_off + k >= lo && lane_off + k < hi) sum.v[k] = v.v[k];
            merged = sum.raw;
        } else {
            const uint64_t tile_out = (e_lo - shift) * sizeof(T);  // where the tile begins in the outputs, in bytes
            const bool whole_vector = hi - lo == EPV;
            for (uint32_t m = 0; m < nout; ++m) {
                char* out_tile = static_cast<char*>(L.out[rotate_rank(out_first, 1, m, K)]) + tile_out;
                if (whole_vector) {
                    store_tile_of<T>(out_tile, tid, res, keep);
                } else {
                    T* out = reinterpret_cast<T*>(out_tile) + lane_off;
#pragma unroll
                    for (uint32_t k = 0; k < EPV; ++k)
                        if (lane_off + k >= lo && lane_off + k < hi) out[k] = v.v[k];
                }
            }
        }
    }
}

// A tile of a flat launch that no single run covers (or that the buffers' end cuts, `whole` false), from the lane's
// vectors x[r]; `staged` is LDS of K x 64 vectors that this wavefront may use, and holds them already if `parked`.
// Where every rank receives the whole tile at the inputs' offsets (all_reduce) each lane collects its vector of
// results, whatever runs it spans, and the tile is stored like any other: whole cache lines, once.  Otherwise the
// pieces go to their runs' outputs as they are folded.
template <typename T, int OP, int K, bool TREE>
__device__ __forceinline__ void flat_tile_uncovered(const FlatLaunch& L, uint32_t tile, uint32_t tid, u32x4 (&x)[K],
                                                    u32x4 (*staged)[kThreads], bool parked, bool whole, const RunBatch& first) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;
    const bool merge = L.nout == uint32_t(K) && L.unshifted;
    const bool keep = (L.exchange & kFlatKeep) != 0;
    const uint64_t tile_off = uint64_t(tile) * (kThreads * kVecBytes);
    u32x4 merged = {0u, 0u, 0u, 0u};
    if (whole) {
        if (!parked) {
            // each lane parks its vectors in LDS, where its own run's fold order can index them
#pragma unroll
            for (int r = 0; r < K; ++r) staged[r][tid] = x[r];
        }
        LaneRun lr;
        lane_scan<T>(first, tile, tid, lr);
        for (uint32_t base = 8; base < L.nruns; base += 8) lane_scan<T>(load_batch(L, base), tile, tid, lr);
        merged = flat_tile_whole_vectors<T, OP, K, TREE>(L, tile, tid, staged, lr, !merge);
        if (__builtin_amdgcn_ballot_w64(lr.cut)) {
            if (merge) flat_tile_ragged<T, OP, K, TREE, true>(L, tile, tid, staged, lr.cut, merged);
            else flat_tile_ragged<T, OP, K, TREE, false>(L, tile, tid, staged, lr.cut, merged);
        }
        if (merge) {
#pragma unroll
            for (int m = 0; m < K; ++m) store_tile_vec(static_cast<char*>(L.out[m]) + tile_off, tid, merged, keep);
        }
        return;
    }
    // the buffers' last tile
    load_tile_at_the_end<T, K>(L, tile, tid, x, &staged[0][0]);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < K; ++r) staged[r][tid] = x[r];
    if (!merge) {
        flat_tile_ragged<T, OP, K, TREE, false>(L, tile, tid, staged, true, merged);
        return;
    }
    flat_tile_ragged<T, OP, K, TREE, true>(L, tile, tid, staged, true, merged);
    const uint32_t nvalid = uint32_t(L.count - uint64_t(tile) * TILE);
    const uint32_t nfull = nvalid / EPV, ntail = nvalid % EPV;
    VecOf<T> v;
    v.raw = merged;
#pragma unroll
    for (int m = 0; m < K; ++m) {
        char* out_tile = static_cast<char*>(L.out[m]) + tile_off;
        if (tid < nfull) {
            store_tile_of<T>(out_tile, tid, merged, keep);
        } else if (tid == nfull) {  // the elements behind the last whole vector
            T* out = reinterpret_cast<T*>(out_tile) + tid * EPV;
#pragma unroll
            for (uint32_t k = 0; k < EPV; ++k)
                if (k < ntail) out[k] = v.v[k];
        }
    }
}

// One tile of a flat launch by one wavefront.
template <typename T, int OP, int K, bool TREE>
__device__ __forceinline__ void flat_tile(const FlatLaunch& L, uint32_t tile, uint32_t tid) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;  // elements per tile
    const uint64_t tile_off = uint64_t(tile) * (kThreads * kVecBytes);  // byte offset of the tile
    const bool whole = (uint64_t(tile) + 1) * TILE <= L.count;  // tile lies inside the buffer

    u32x4 x[K];
    if (whole) {
#pragma unroll
        for (int r = 0; r < K; ++r) x[r] = load_tile_vec(static_cast<const char*>(L.in[r]) + tile_off, tid);
    }

    // Which run holds this tile?  Eight runs per round of scalar loads (one round for up to eight
    // runs, which is every all_reduce of up to eight ranks in the ring order).
    const uint64_t e_lo = uint64_t(tile) * TILE, e_hi = e_lo + TILE;
    const RunBatch first = load_batch(L, 0);
    TileRun tr;
    uniform_scan(first, e_lo, e_hi, tr);
    for (uint32_t base = 8; base < L.nruns && !tr.covered; base += 8) uniform_scan(load_batch(L, base), e_lo, e_hi, tr);
    const bool covered = tr.covered;
    const uint32_t meta = tr.meta;
    const uint64_t shift = tr.shift;
    const bool new_wins = L.new_wins_ties != 0;
    const uint32_t nout = L.nout;

    if (covered && whole) {
        // the whole tile shares one fold order (and lies inside the buffer)
        const uint32_t start = meta_start(meta);
        const int dir = meta_dir(meta);
        const uint32_t out_first = meta_out_first(meta);
        const uint64_t out_off = tile_off - shift * sizeof(T);
        u32x4 res;
        if constexpr (TREE) {
            res = tree_from<T, OP, K>(x, start);
        } else {
            res = fold_from<T, OP, K>(x, start, dir, new_wins);
        }
        if (nout == uint32_t(K)) {
#pragma unroll
            for (int m = 0; m < K; ++m) store_tile_vec(static_cast<char*>(L.out[m]) + out_off, tid, res, (L.exchange & kFlatKeep) != 0);
        } else {
            for (uint32_t m = 0; m < nout; ++m)
                store_tile_vec(static_cast<char*>(L.out[rotate_rank(out_first, 1, m, K)]) + out_off, tid, res, (L.exchange & kFlatKeep) != 0);
        }
        return;
    }

    __shared__ u32x4 parked[K][kThreads];
    flat_tile_uncovered<T, OP, K, TREE>(L, tile, tid, x, parked, false, whole, first);
}

// TREE selects the binomial-tree combination; it is a template parameter, not a run-time branch,
// so that the tree's K live accumulators do not cost the left fold any registers.
template <typename T, int OP, int K, bool TREE>
__global__ void __launch_bounds__(kThreads) fold_flat_kernel(const FlatLaunch L) {
    if ((L.hook_target != 0) | ((L.exchange & kFlatGuarded) != 0)) {
        if (!hook_enter(L.hooks, L.hook_target)) return;
    }
    flat_tile<T, OP, K, TREE>(L, blockIdx.x, threadIdx.x);
    if (L.hook_ticket) hook_publish(L.hooks, L.hook_ticket);
}

// Group form of the flat fold for launches of many tiles.  A workgroup of kGroupWaves wavefronts
// owns kGroupWaves tiles that lie kGroupStride tiles apart.  Wavefront w loads input r of tile
// (w + r) % kGroupWaves, so the K loads it issues together go to different tiles; the tiles are
// exchanged through LDS and wavefront w folds tile w.  Where every rank is an output at the inputs'
// offsets (all_reduce, L.exchange) the results are exchanged again and wavefront w stores output m
// of tile (w + m) % kGroupWaves; otherwise wavefront w stores its own tile.  Measured on MI355X,
// fp32, over several buffer sizes and placements, against one wavefront per tile on the same
// device: 8 in + 8 out 83 % of the HBM peak against 70 - 76 %, 8 in + 1 out 85 % against 75 - 79 %;
// strides of 32 and 64 tiles are the good ones, 16 and 128 lose most of the gain.
template <typename T, int OP, int K, bool TREE>
__global__ void __launch_bounds__(kThreads * kGroupWaves) fold_group_kernel(const FlatLaunch L) {
    constexpr uint32_t EPV = kVecBytes / sizeof(T);
    constexpr uint32_t TILE = kThreads * EPV;
    constexpr uint32_t W = kGroupWaves;
    __shared__ u32x4 stage[W][K][kThreads];
    __shared__ u32x4 result[W][kThreads];
    __shared__ uint32_t folded[W];
    const uint32_t tid = threadIdx.x % kThreads;
    // wavefront index, made known to be uniform so that it selects pointers in scalar registers
    const uint32_t wave = uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x / kThreads)));
    uint32_t block = blockIdx.x;
    if (L.exchange & 2u) {  // deal whole runs of kGroupStride workgroups to one XCD each
        constexpr uint32_t kXcds = 8, kDeal = kXcds * kGroupStride;
        if (block < gridDim.x / kDeal * kDeal) {
            const uint32_t w = block % kDeal;
            block = block - w + (w % kXcds) * kGroupStride + w / kXcds;
        }
    }
    const uint32_t first = (block / kGroupStride) * (W * kGroupStride) + block % kGroupStride;
    const uint32_t mine = first + wave * kGroupStride;
    const bool exchange = (L.exchange & 1u) != 0;

    // tile k of the group is first + k * kGroupStride; it is loaded if it lies inside the buffers.
    // A wavefront keeps kGroupLoadsInFlight loads in flight: load r + 2 is issued when load r has arrived (its
    // address is made to depend on it).  The memory system serves a workgroup's accesses better spread over time
    // than all at once, the more so the worse the caller's buffers lie relative to each other (see kGroupLoadsInFlight).
    constexpr int D = K < int(kGroupLoadsInFlight) ? K : int(kGroupLoadsInFlight);
    const auto load_input = [&](int r, uint32_t lane) -> u32x4 {
        const uint64_t tile = uint64_t(first) + ((wave + r) % W) * kGroupStride;
        if ((tile + 1) * TILE <= L.count)
            return load_tile_vec(static_cast<const char*>(L.in[r]) + tile * (kThreads * kVecBytes), lane);
        return u32x4{0u, 0u, 0u, 0u};  // never folded: such a tile goes element by element
    };
    const bool paced = (L.exchange & kFlatPaced) != 0;
    u32x4 x[K];
#pragma unroll
    for (int r = 0; r < D; ++r) x[r] = load_input(r, tid);
    if (!paced) {  // short launches: everything at once, their time is latency
#pragma unroll
        for (int r = D; r < K; ++r) x[r] = load_input(r, tid);
    }
    // A launch of a communicator group stores nothing once the group is poisoned.  The wavefronts of a workgroup
    // may see the poison rise at different moments, so it only ever masks stores and never skips a barrier.
    const bool live = (L.exchange & kFlatGuarded) == 0 || hook_poison(L.hooks) == 0;
    // while the loads are in flight: which run does this wavefront's own tile lie in?
    TileRun tr;
    {
        const uint64_t e_lo = uint64_t(mine) * TILE;
        for (uint32_t base = 0; base < L.nruns && !tr.covered; base += 8) uniform_scan(load_batch(L, base), e_lo, e_lo + TILE, tr);
    }
    const int run = tr.covered ? 0 : -1;
    const uint32_t start = meta_start(tr.meta), out_first = meta_out_first(tr.meta);
    const int dir = meta_dir(tr.meta);
    const uint64_t out_shift = tr.shift;
#pragma unroll
    for (int r = 0; r < K; ++r) {
        if (paced && r + D < K) {
            uint32_t lane = tid;
            asm volatile("" : "+v"(lane) : "v"(x[r]));  // the next load's address waits for x[r]
            x[r + D] = load_input(r + D, lane);
        }
        stage[(wave + r) % W][r][tid] = x[r];
    }
    __syncthreads();

    if (run >= 0) {
        // the whole tile shares one fold order (and lies inside the buffers)
#pragma unroll
        for (int r = 0; r < K; ++r) x[r] = stage[wave][r][tid];
        u32x4 res;
        if constexpr (TREE) {
            res = tree_from<T, OP, K>(x, start);
        } else {
            res = fold_from<T, OP, K>(x, start, dir, L.new_wins_ties != 0);
        }
        if (exchange) {
            result[wave][tid] = res;
        } else if (live) {
            const uint64_t out_off = uint64_t(mine) * (kThreads * kVecBytes) - out_shift * sizeof(T);
            for (uint32_t m = 0; m < L.nout; ++m)
                store_tile_vec(static_cast<char*>(L.out[rotate_rank(out_first, 1, m, K)]) + out_off, tid, res, (L.exchange & kFlatKeep) != 0);
        }
    } else if (!live) {
        // nothing is stored
    } else if (mine < L.total_tiles) {
        // across run borders (from the staged vectors), or the buffers' last, partial tile (which nobody has loaded);
        // stored by this wavefront
        const bool whole = (uint64_t(mine) + 1) * TILE <= L.count;
        flat_tile_uncovered<T, OP, K, TREE>(L, mine, tid, x, stage[wave], whole, whole, load_batch(L, 0));
    }
    if (exchange) {
        if (tid == 0) folded[wave] = run >= 0 ? 1u : 0u;
        __syncthreads();
#pragma unroll
        for (int m = 0; m < K; ++m) {
            const uint32_t k = (wave + m) % W;
            if (folded[k] && live) {
                const uint64_t tile = uint64_t(first) + k * kGroupStride;
                store_tile_vec(static_cast<char*>(L.out[m]) + tile * (kThreads * kVecBytes), tid, result[k][tid], (L.exchange & kFlatKeep) != 0);
            }
            // ... and kGroupStoresInFlight stores in flight
            if (paced && (m + 1) % int(kGroupStoresInFlight) == 0 && m + 1 < K) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }
}

// ---------------------------------------------------------------------------------------------
// Launchers for one element type.  `op` is kSum / kMax / kMin; SUM exists for the unsigned and the
// floating types only (a signed integer SUM runs on its unsigned twin: two's-complement wrap).

using FoldFn = void (*)(const FoldLaunch);
using FlatFn = void (*)(const FlatLaunch);
using TreeFn = void (*)(const TreeLaunch);

template <typename T>
constexpr bool has_sum() {
    return !(std::is_integral<T>::value && std::is_signed<T>::value);
}

template <typename T, int OP>
FoldFn pick_fold_group(uint32_t nfold) {
    switch (nfold) {
        case 1: return fold_segment_group_kernel<T, OP, 1>;
        case 2: return fold_segment_group_kernel<T, OP, 2>;
        case 3: return fold_segment_group_kernel<T, OP, 3>;
        case 4: return fold_segment_group_kernel<T, OP, 4>;
        case 8: return fold_segment_group_kernel<T, OP, 8>;
        default: return fold_segment_group_kernel<T, OP, 0>;
    }
}

template <typename T, int OP>
FoldFn pick_fold(uint32_t nfold) {
    switch (nfold) {
        case 2: return fold_kernel<T, OP, 2>;
        case 3: return fold_kernel<T, OP, 3>;
        case 4: return fold_kernel<T, OP, 4>;
        case 8: return fold_kernel<T, OP, 8>;
        default: return fold_kernel<T, OP, 0>;
    }
}

template <typename T, int OP, bool TREE>
FlatFn pick_flat_k(uint32_t nranks) {
    switch (nranks) {
        case 2: return fold_flat_kernel<T, OP, 2, TREE>;
        case 3: return fold_flat_kernel<T, OP, 3, TREE>;
        case 4: return fold_flat_kernel<T, OP, 4, TREE>;
        case 8: return fold_flat_kernel<T, OP, 8, TREE>;
        default: return nullptr;
    }
}

template <typename T, int OP, bool TREE>
FlatFn pick_group_k(uint32_t nranks) {
    switch (nranks) {
        case 2: return fold_group_kernel<T, OP, 2, TREE>;
        case 3: return fold_group_kernel<T, OP, 3, TREE>;
        case 4: return fold_group_kernel<T, OP, 4, TREE>;
        case 8: return fold_group_kernel<T, OP, 8, TREE>;
        default: return nullptr;
    }
}

template <typename T, int OP>
FlatFn pick_flat(const FlatLaunch& L) {
    if (L.waves == kGroupWaves) return L.tree ? pick_group_k<T, OP, true>(L.nranks) : pick_group_k<T, OP, false>(L.nranks);
    return L.tree ? pick_flat_k<T, OP, true>(L.nranks) : pick_flat_k<T, OP, false>(L.nranks);
}

// The kernel (as a host-side function address) that carries out `op` on element type T for a
// launch descriptor; nullptr if there is none.
template <typename T>
const void* fold_kernel_t(const FoldLaunch& L, int op) {
    FoldFn fn = nullptr;
    const bool group = L.waves == kGroupWaves;
    if (op == kMax) fn = group ? pick_fold_group<T, kMax>(L.nfold) : pick_fold<T, kMax>(L.nfold);
    if (op == kMin) fn = group ? pick_fold_group<T, kMin>(L.nfold) : pick_fold<T, kMin>(L.nfold);
    if constexpr (has_sum<T>()) {
        if (op == kSum) fn = group ? pick_fold_group<T, kSum>(L.nfold) : pick_fold<T, kSum>(L.nfold);
    }
    return reinterpret_cast<const void*>(fn);
}

template <typename T>
const void* flat_kernel_t(const FlatLaunch& L, int op) {
    FlatFn fn = nullptr;
    if (op == kMax) fn = pick_flat<T, kMax>(L);
    if (op == kMin) fn = pick_flat<T, kMin>(L);
    if constexpr (has_sum<T>()) {
        if (op == kSum) fn = pick_flat<T, kSum>(L);
    }
    return reinterpret_cast<const void*>(fn);
}

template <typename T>
const void* tree_kernel_t(int op) {
    TreeFn fn = nullptr;
    if (op == kMax) fn = fold_tree_kernel<T, kMax>;
    if (op == kMin) fn = fold_tree_kernel<T, kMin>;
    if constexpr (has_sum<T>()) {
        if (op == kSum) fn = fold_tree_kernel<T, kSum>;
    }
    return reinterpret_cast<const void*>(fn);
}

// Defines the three kernel tables of element type T in the including translation unit.
#define MEGRAY_VRANK_INSTANTIATE(T)                                    \
    template const void* fold_kernel_t<T>(const FoldLaunch&, int);     \
    template const void* flat_kernel_t<T>(const FlatLaunch&, int);     \
    template const void* tree_kernel_t<T>(int);

}  // namespace detail
}  // namespace vrank
}  // namespace MegRay
