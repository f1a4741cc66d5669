#include "vrank_edges.h"

#include <hip/hip_runtime.h>

#include <mutex>

namespace MegRay {
namespace vrank {

// The counter blocks of groups that must not allocate.  In host code this name stands for the
// variable, it is not a device address: the address of the current device's copy comes from
// hipGetSymbolAddress (edge_static_words below) and is what kernels, clears and copies are given.
static __device__ __align__(256) uint64_t scratch[kStaticEdgeSlots * (sizeof(EdgeWords) / sizeof(uint64_t))];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
uint64_t* g_scratch_base[kMaxDevices] = {};  // per device: where its copy of `scratch` lies

__global__ void __launch_bounds__(64) edge_arrive_kernel(uint64_t* arrived) {
    if (threadIdx.x == 0) __hip_atomic_fetch_add(arrived, uint64_t(1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// Nothing is published for a poisoned group: the streams that wait for it find the poison themselves.
__global__ void __launch_bounds__(64) edge_notify_kernel(uint64_t* done, uint64_t ticket, const uint64_t* poison) {
    if (threadIdx.x != 0) return;
    if (__hip_atomic_load(poison, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT)) return;
    __hip_atomic_store(done, ticket, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

// One lane polls `word` until it reaches `target` or `limit_ticks` of the constant-rate wall clock
// have passed; the wavefront sleeps between polls.  A wait of a poisoned group returns at once; a wait
// that gives up poisons its group (edge_words[2], the group's `timeouts`) and tells the host.
__global__ void __launch_bounds__(64) edge_wait_kernel(const uint64_t* word, uint64_t target, uint64_t limit_ticks,
                                                       uint64_t* group_words, uint64_t* status) {
    if (threadIdx.x != 0) return;
    uint64_t* timeouts = group_words + 2;
    const uint64_t begin = wall_clock64();
    while (__hip_atomic_load(word, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) < target) {
        if (__hip_atomic_load(timeouts, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT)) return;
        if (wall_clock64() - begin > limit_ticks) {
            if (__hip_atomic_fetch_add(timeouts, uint64_t(1), __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT) == 0)
                __hip_atomic_store(group_words + 4, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (status) {
                __hip_atomic_store(status + 1, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
                __hip_atomic_fetch_add(status, uint64_t(1), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
            }
            return;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

}  // namespace

hipError_t edge_static_words(uint32_t slot, EdgeWords** words) {
    if (!words || slot >= kStaticEdgeSlots) return hipErrorInvalidValue;
    *words = nullptr;
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return err;
    if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_base[device]) {
        void* base = nullptr;
        err = hipGetSymbolAddress(&base, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return err;
        g_scratch_base[device] = static_cast<uint64_t*>(base);
    }
    *words = reinterpret_cast<EdgeWords*>(g_scratch_base[device]) + slot;
    return hipSuccess;
}

hipError_t edge_arrive(EdgeWords* words, hipStream_t stream) {
    hipLaunchKernelGGL(edge_arrive_kernel, dim3(1), dim3(64), 0, stream, &words->arrived);
    return hipGetLastError();
}

hipError_t edge_notify(EdgeWords* words, EdgeWords* group, uint64_t ticket, hipStream_t stream) {
    hipLaunchKernelGGL(edge_notify_kernel, dim3(1), dim3(64), 0, stream, &words->done, ticket, &group->timeouts);
    return hipGetLastError();
}

hipError_t edge_wait_arrived(EdgeWords* words, EdgeWords* group, uint64_t target, uint64_t limit_ticks,
                             uint64_t* status, hipStream_t stream) {
    hipLaunchKernelGGL(edge_wait_kernel, dim3(1), dim3(64), 0, stream, &words->arrived, target, limit_ticks,
                       reinterpret_cast<uint64_t*>(group), status);
    return hipGetLastError();
}

hipError_t edge_wait_done(EdgeWords* words, EdgeWords* group, uint64_t ticket, uint64_t limit_ticks,
                          uint64_t* status, hipStream_t stream) {
    hipLaunchKernelGGL(edge_wait_kernel, dim3(1), dim3(64), 0, stream, &words->done, ticket, limit_ticks,
                       reinterpret_cast<uint64_t*>(group), status);
    return hipGetLastError();
}

hipError_t edge_read_timeouts(const EdgeWords* words, hipStream_t stream, uint64_t* timeouts, uint64_t* gave_up_at) {
    EdgeWords copy;
    hipError_t err = hipMemcpyAsync(&copy, words, sizeof(copy), hipMemcpyDeviceToHost, stream);
    if (err == hipSuccess) err = hipStreamSynchronize(stream);
    if (err != hipSuccess) return err;
    *timeouts = copy.timeouts;
    *gave_up_at = copy.gave_up_at;
    return hipSuccess;
}

}  // namespace vrank
}  // namespace MegRay
