// Dispatch of the virtual-rank launches to the per-type fold kernels, plus the type-agnostic
// kernels: pack_kernel (equally sized block copies between rank buffers for all_to_all / scatter /
// gather, replacing the per-peer send/recv pairs of src/ucx/all_to_all.cpp:30-41,
// src/ucx/scatter.cpp:30-44 and src/ucx/gather.cpp:30-44) and the plain copies of the fold kernel.
#include "vrank_fold_impl.hpp"

#include <cstring>
#include <mutex>
#include <unordered_map>

#include "megray/debug.h"

namespace MegRay {
namespace vrank {

namespace detail {
// instantiated in vrank_fold_<type>.hip
#define MEGRAY_VRANK_EXTERN(T)                                                \
    extern template const void* fold_kernel_t<T>(const FoldLaunch&, int);     \
    extern template const void* flat_kernel_t<T>(const FlatLaunch&, int);     \
    extern template const void* tree_kernel_t<T>(int);
MEGRAY_VRANK_EXTERN(int8_t)
MEGRAY_VRANK_EXTERN(uint8_t)
MEGRAY_VRANK_EXTERN(int32_t)
MEGRAY_VRANK_EXTERN(uint32_t)
MEGRAY_VRANK_EXTERN(int64_t)
MEGRAY_VRANK_EXTERN(uint64_t)
MEGRAY_VRANK_EXTERN(_Float16)
MEGRAY_VRANK_EXTERN(float)
MEGRAY_VRANK_EXTERN(double)
}  // namespace detail

namespace {

using namespace detail;

template <typename W>
__device__ __forceinline__ W load_w(const char* p) {
    return __builtin_nontemporal_load(reinterpret_cast<const W*>(p));
}
template <typename W>
__device__ __forceinline__ void store_w(char* p, W x) {
    __builtin_nontemporal_store(x, reinterpret_cast<W*>(p));
}

// Decodes copy `copy` of a pack launch into its endpoints.
struct PackEnds {
    uint32_t src_rank, src_block, dst_rank, dst_block, ndst;
};
__device__ __forceinline__ PackEnds pack_ends(const PackLaunch& L, uint32_t copy) {
    const uint32_t n = L.nranks;
    if (L.mode == kPackAllToAll) return {copy / n, copy % n, copy % n, copy / n, 1};
    if (L.mode == kPackScatter) return {L.root, copy, copy, 0, 1};
    if (L.mode == kPackGather) return {copy, 0, L.root, copy, 1};
    if (L.mode == kPackBroadcast) return {L.root, 0, 0, 0, n};
    return {copy, 0, 0, copy, n};  // kPackAllGather: read once, write the block into every rank's buffer
}

// Where the 16-byte vectors of one block copy lie.  They start at the (first) destination's first 16-byte boundary,
// `head` bytes into the block; `nvec` whole vectors follow, then `tail` bytes (both below 16, and 0 for blocks on
// 16-byte boundaries).  Lane `tid` of tile `t` takes vector t * kThreads + tid - pad, where `pad` (below kThreads)
// is chosen so that tile 1 starts on a 1 KiB boundary of the destination: whole tiles then store whole cache lines
// whatever the block's offset.
struct PackVectors {
    uint32_t head, tail, pad;
    uint64_t nvec;
};
__device__ __forceinline__ PackVectors pack_vectors(const PackLaunch& L, const PackEnds& e, uint64_t dst_off) {
    constexpr uint64_t kTileBytes = uint64_t(kThreads) * kVecBytes;
    const uintptr_t dst = reinterpret_cast<uintptr_t>(L.out[e.dst_rank]) + dst_off;
    uint64_t head = (0 - dst) & (kVecBytes - 1);
    if (head > L.block_bytes) head = L.block_bytes;
    const uint64_t nvec = (L.block_bytes - head) / kVecBytes;
    const uint64_t before = ((0 - (dst + head)) & (kTileBytes - 1)) / kVecBytes;  // vectors in front of the 1 KiB boundary
    const uint32_t pad = uint32_t((kThreads - before) % kThreads);
    return {uint32_t(head), uint32_t(L.block_bytes - head - nvec * kVecBytes), pad, nvec};
}

// The bytes in front of the first and behind the last vector of a block copy, in units of the blocks' common
// alignment (4 bytes at most): at most 30 lanes of one wavefront.
template <typename U>
__device__ __forceinline__ void pack_edge_units(const PackLaunch& L, const PackEnds& e, const PackVectors& pv,
                                                const char* src, uint64_t dst_off, uint32_t tid) {
    const uint32_t hu = pv.head / sizeof(U), tu = pv.tail / sizeof(U);
    if (tid >= hu + tu) return;
    const uint64_t off = tid < hu ? uint64_t(tid) * sizeof(U)
                                  : pv.head + pv.nvec * kVecBytes + uint64_t(tid - hu) * sizeof(U);
    const U x = load_w<U>(src + off);
    for (uint32_t m = 0; m < e.ndst; ++m) store_w<U>(static_cast<char*>(L.out[e.dst_rank + m]) + dst_off + off, x);
}
__device__ __forceinline__ void pack_edges(const PackLaunch& L, const PackEnds& e, const PackVectors& pv,
                                           const char* src, uint64_t dst_off, uint32_t tid) {
    if (L.width >= 4) pack_edge_units<uint32_t>(L, e, pv, src, dst_off, tid);
    else if (L.width == 2) pack_edge_units<uint16_t>(L, e, pv, src, dst_off, tid);
    else pack_edge_units<uint8_t>(L, e, pv, src, dst_off, tid);
}

// Tile `tile` of a block copy, by one wavefront: whole tiles through buffer instructions, the partial ones at the
// block's ends lane by lane.  `src` and `dst_off` address the block's first byte.
__device__ __forceinline__ void pack_vector_tile(const PackLaunch& L, const PackEnds& e, const PackVectors& pv,
                                                 const char* src, uint64_t dst_off, uint64_t tile, uint32_t tid) {
    const uint64_t t0 = tile * kThreads;  // this tile's lanes take vectors [t0 - pad, t0 - pad + kThreads)
    if (t0 >= pv.pad && t0 - pv.pad + kThreads <= pv.nvec) {
        const uint64_t off = pv.head + (t0 - pv.pad) * kVecBytes;
        const u32x4 x = load_tile_any(src + off, tid);
        for (uint32_t m = 0; m < e.ndst; ++m)
            store_tile_any(static_cast<char*>(L.out[e.dst_rank + m]) + dst_off + off, tid, x, L.keep != 0);
    } else if (t0 + tid >= pv.pad && t0 + tid - pv.pad < pv.nvec) {
        const uint64_t off = pv.head + (t0 + tid - pv.pad) * kVecBytes;
        const u32x4 x = load_vec(src + off);
        for (uint32_t m = 0; m < e.ndst; ++m)
            store_vec(static_cast<char*>(L.out[e.dst_rank + m]) + dst_off + off, x);
    }
}

// One wavefront per tile: short block copies.
__global__ void __launch_bounds__(kThreads) pack_kernel(const PackLaunch L) {
    if (!hook_enter(L.hooks, L.hook_target)) return;
    const uint32_t copy = blockIdx.x / L.tiles_per_copy;
    const uint64_t tile = L.first_tile + (blockIdx.x - copy * L.tiles_per_copy);
    const PackEnds e = pack_ends(L, copy);
    const uint32_t tid = threadIdx.x;
    const char* src = static_cast<const char*>(L.in[e.src_rank]) + e.src_block * L.block_bytes;
    const uint64_t dst_off = e.dst_block * L.block_bytes;
    const PackVectors pv = pack_vectors(L, e, dst_off);
    pack_vector_tile(L, e, pv, src, dst_off, tile, tid);
    if (tile == 0) pack_edges(L, e, pv, src, dst_off, tid);
    if (L.hook_ticket) hook_publish(L.hooks, L.hook_ticket);
}

// Group form of the pack kernel for long blocks: a workgroup of kGroupWaves
// wavefronts owns kGroupWaves tiles of one block copy, kGroupStride tiles apart; wavefront w loads
// tile w.  With one destination it stores that tile; with N destinations (all_gather) the tiles are
// exchanged through LDS and wavefront w stores destination m of tile (w + m) % kGroupWaves, so the
// N stores it issues together go to different tiles.  Measured on MI355X (1 GiB and 128 MiB
// buffers): 1 -> 8 copies 82 % of the HBM peak against 65 - 69 % with one wavefront per tile,
// 1 -> 1 copies 84 - 87 % against 83 - 84 %.
__global__ void __launch_bounds__(kThreads * kGroupWaves) pack_group_kernel(const PackLaunch L) {
    constexpr uint32_t W = kGroupWaves;
    __shared__ u32x4 stage[W][kThreads];
    __shared__ uint32_t staged[W];
    const uint32_t tid = threadIdx.x % kThreads;
    const uint32_t wave = uint32_t(__builtin_amdgcn_readfirstlane(int(threadIdx.x / kThreads)));
    const uint32_t copy = blockIdx.x / L.groups_per_copy;
    uint32_t group = blockIdx.x - copy * L.groups_per_copy;
    const PackEnds e = pack_ends(L, copy);
    const char* src = static_cast<const char*>(L.in[e.src_rank]) + e.src_block * L.block_bytes;
    const uint64_t dst_off = e.dst_block * L.block_bytes;
    const PackVectors pv = pack_vectors(L, e, dst_off);
    // The tiles sit on the destination's cache lines.  If the source lies differently, neighbouring tiles share
    // source lines: consecutive workgroups run on different XCDs, each with an L2 of its own, so whole runs of
    // kGroupStride workgroups (4 * kGroupStride consecutive tiles) are dealt to one XCD each.
    if ((reinterpret_cast<uintptr_t>(src) - (reinterpret_cast<uintptr_t>(L.out[e.dst_rank]) + dst_off)) & 127u) {
        constexpr uint32_t kXcds = 8, kDeal = kXcds * kGroupStride;
        if (group < L.groups_per_copy / kDeal * kDeal) {
            const uint32_t w = group % kDeal;
            group = group - w + (w % kXcds) * kGroupStride + w / kXcds;
        }
    }
    const uint64_t first = L.first_tile + uint64_t(group / kGroupStride) * (W * kGroupStride) + group % kGroupStride;
    // A launch of a communicator group stores nothing once the group is poisoned (stores are masked, barriers kept).
    const bool live = hook_poison(L.hooks) == 0;
    if (first == 0 && wave == 0 && live) pack_edges(L, e, pv, src, dst_off, tid);

    // tile t holds vectors [t * kThreads - pad, ...): whole if all of them exist
    const uint64_t mine = first + wave * kGroupStride;
    const auto whole_tile = [&](uint64_t t) { return t * kThreads >= pv.pad && t * kThreads - pv.pad + kThreads <= pv.nvec; };
    const auto tile_off = [&](uint64_t t) { return pv.head + (t * kThreads - pv.pad) * kVecBytes; };  // whole tiles only
    const bool whole = whole_tile(mine);
    u32x4 x = {0u, 0u, 0u, 0u};
    if (whole)
        x = load_tile_any(src + tile_off(mine), tid);
    else if (live)
        pack_vector_tile(L, e, pv, src, dst_off, mine, tid);  // a partial tile at either end: copied to every destination here
    if (e.ndst == 1) {
        if (whole && live) store_tile_any(static_cast<char*>(L.out[e.dst_rank]) + dst_off + tile_off(mine), tid, x, L.keep != 0);
        return;
    }
    stage[wave][tid] = x;
    if (tid == 0) staged[wave] = whole ? 1u : 0u;
    __syncthreads();
    for (uint32_t m = 0; m < e.ndst; ++m) {
        const uint32_t k = (wave + m) % W;
        if (staged[k] && live)
            store_tile_any(static_cast<char*>(L.out[e.dst_rank + m]) + dst_off + tile_off(first + uint64_t(k) * kGroupStride),
                            tid, stage[k][tid], L.keep != 0);
        if (L.paced) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // one store in flight per wavefront
    }
}

FoldFn pick_copy_group(uint32_t elem_size) {
    switch (elem_size) {
        case 1: return fold_segment_group_kernel<uint8_t, kCopy, 1>;
        case 2: return fold_segment_group_kernel<uint16_t, kCopy, 1>;
        case 4: return fold_segment_group_kernel<uint32_t, kCopy, 1>;
        default: return fold_segment_group_kernel<uint64_t, kCopy, 1>;
    }
}

FoldFn pick_copy(uint32_t elem_size) {
    switch (elem_size) {
        case 1: return fold_kernel<uint8_t, kCopy, 1>;
        case 2: return fold_kernel<uint16_t, kCopy, 1>;
        case 4: return fold_kernel<uint32_t, kCopy, 1>;
        default: return fold_kernel<uint64_t, kCopy, 1>;
    }
}

// Calls `call(T{}, k)` for the element type that carries out `op` on `dtype`: integer SUM wraps,
// so both signs share the unsigned kernel.
template <typename F>
const void* with_type(DType dtype, ReduceOp op, F&& call) {
    int k;
    switch (op) {
        case MEGRAY_SUM: k = kSum; break;
        case MEGRAY_MAX: k = kMax; break;
        case MEGRAY_MIN: k = kMin; break;
        default: return nullptr;
    }
    const bool sum = k == kSum;
    switch (dtype) {
        case MEGRAY_INT8: return sum ? call(uint8_t{}, k) : call(int8_t{}, k);
        case MEGRAY_UINT8: return call(uint8_t{}, k);
        case MEGRAY_INT32: return sum ? call(uint32_t{}, k) : call(int32_t{}, k);
        case MEGRAY_UINT32: return call(uint32_t{}, k);
        case MEGRAY_INT64: return sum ? call(uint64_t{}, k) : call(int64_t{}, k);
        case MEGRAY_UINT64: return call(uint64_t{}, k);
        case MEGRAY_FLOAT16: return call(_Float16{}, k);
        case MEGRAY_FLOAT32: return call(float{}, k);
        case MEGRAY_FLOAT64: return call(double{}, k);
        default: return nullptr;
    }
}

}  // namespace

const void* fold_kernel_for(const FoldLaunch& L, DType dtype, ReduceOp op) {
    if (L.nfold == 1)
        return reinterpret_cast<const void*>(L.waves == kGroupWaves ? pick_copy_group(L.elem_size) : pick_copy(L.elem_size));
    return with_type(dtype, op, [&](auto tag, int k) { return fold_kernel_t<decltype(tag)>(L, k); });
}

const void* flat_kernel_for(const FlatLaunch& L, DType dtype, ReduceOp op) {
    return with_type(dtype, op, [&](auto tag, int k) { return flat_kernel_t<decltype(tag)>(L, k); });
}

const void* tree_kernel_for(const TreeLaunch&, DType dtype, ReduceOp op) {
    return with_type(dtype, op, [&](auto tag, int k) { return tree_kernel_t<decltype(tag)>(k); });
}

const void* pack_kernel_for(const PackLaunch& L) {
    return L.waves == kGroupWaves ? reinterpret_cast<const void*>(&pack_group_kernel)
                                  : reinterpret_cast<const void*>(&pack_kernel);
}

namespace {

// What the occupancy caps assume of the device in use, asked of the runtime once per device: the LDS a CU
// holds, and whether the device is the part the caps were measured on (gfx950).  On any other part the
// caps are left out (a launch at full occupancy is always correct, the cap is a tuning of MI355X).
struct DeviceTraits {
    bool known = false;
    bool tuned = false;      // gfx950: the measured occupancy tables apply
    uint32_t lds_per_cu = 0;
};

DeviceTraits device_traits() {
    constexpr int kMaxDevices = 64;
    static std::mutex mutex;
    static DeviceTraits traits[kMaxDevices];
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) {
        (void)hipGetLastError();
        return {};
    }
    std::lock_guard<std::mutex> lock(mutex);
    DeviceTraits& t = traits[device];
    if (!t.known) {
        hipDeviceProp_t prop;
        int lds = 0;
        if (hipGetDeviceProperties(&prop, device) != hipSuccess ||
            hipDeviceGetAttribute(&lds, hipDeviceAttributeMaxSharedMemoryPerMultiprocessor, device) != hipSuccess) {
            (void)hipGetLastError();
            return {};
        }
        t.known = true;
        t.tuned = std::strncmp(prop.gcnArchName, "gfx950", 6) == 0;
        t.lds_per_cu = lds > 0 ? uint32_t(lds) : 0;
        if (!t.tuned)
            MEGRAY_WARN("device %d is %s, not gfx950: launches keep their full occupancy (the caps were measured on MI355X)",
                        device, prop.gcnArchName);
    }
    return t;
}

}  // namespace

uint32_t lds_for_waves_per_cu(const void* kernel, uint32_t waves_per_cu) {
    if (!kernel || !waves_per_cu) return 0;
    const DeviceTraits traits = device_traits();
    if (!traits.known || !traits.tuned || !traits.lds_per_cu) return 0;
    // what the kernel declares itself, asked of the runtime once per kernel
    static std::mutex mutex;
    static std::unordered_map<const void*, uint32_t> declared;
    static bool complained = false;
    uint32_t own = 0;
    {
        std::lock_guard<std::mutex> lock(mutex);
        auto it = declared.find(kernel);
        if (it == declared.end()) {
            hipFuncAttributes attr;
            const hipError_t err = hipFuncGetAttributes(&attr, kernel);
            if (err != hipSuccess) {
                (void)hipGetLastError();
                if (!complained) {
                    complained = true;
                    MEGRAY_WARN("hipFuncGetAttributes failed (%s): large one-output folds run at full occupancy, "
                                "a few points of the HBM peak slower", hipGetErrorString(err));
                }
                return 0;
            }
            it = declared.emplace(kernel, uint32_t(attr.sharedSizeBytes)).first;
        }
        own = it->second;
    }
    // The hardware hands LDS out in 128 units per CU (1280 bytes each on MI355X; measured: four workgroups of 40960
    // bytes share a CU, of 40976 three; three of 53760, of 53776 two), so a workgroup gets 128 / waves_per_cu whole units.
    const uint32_t unit = traits.lds_per_cu / 128;
    const uint32_t each = 128 / waves_per_cu * unit;
    return each > own ? each - own : 0;
}

hipError_t enqueue(const void* kernel, uint32_t grid, uint32_t block, const void* launch, hipStream_t stream,
                   uint32_t lds) {
    if (!kernel) return hipErrorInvalidValue;
    if (!grid) return hipSuccess;
    void* args[] = {const_cast<void*>(launch)};
    return hipLaunchKernel(kernel, dim3(grid), dim3(block), args, lds, stream);
}

}  // namespace vrank
}  // namespace MegRay
