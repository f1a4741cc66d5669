// The virtual-rank collectives as plain functions over N rank buffers in one GPU's memory.
// Both faces of the library sit on these: the C ABI (vrank_capi.cpp) calls them directly, the
// MegRay::Communicator backend (vrank_communicator.cpp) calls them once all ranks have arrived.
//
// Contract violations throw MegRay::Exception like the reference does (unknown dtype / op:
// src/ucx/kernel.cu:55-56,95-96); planner and HIP failures come back as a Status.
#pragma once

#include <hip/hip_runtime_api.h>

#include <vector>

#include "megray/common.h"
#include "vrank_plan.h"

namespace MegRay {
namespace vrank {

// Element size of a dtype a reduce kernel exists for; throws "unknown dtype" for MEGRAY_CHAR and
// out-of-range values.  FLOAT16 is accepted (fp32 accumulation, one rounding).
uint32_t reduce_elem_size(DType dtype);
// Throws "unknown reduce op" outside SUM / MAX / MIN.
void check_reduce_op(ReduceOp op);

// One kernel launch of a plan, ready for hipLaunchKernel or a graph node.  `launch` points into
// the Plan it was resolved from.
struct KernelCall {
    const void* kernel;
    uint32_t grid;
    uint32_t block;  // threads per workgroup
    const void* launch;
    uint32_t lds = 0;  // LDS bytes reserved per workgroup on top of the kernel's own (sets the occupancy)
};

// Which collective a plan is for (the values of the C ABI's MRV_* selectors).
enum CollectiveKind : int {
    kCollAllReduce = 0,
    kCollReduceScatter = 1,
    kCollAllGather = 2,
    kCollAllToAll = 3,
    kCollScatter = 4,
    kCollGather = 5,
    kCollBroadcast = 6,
    kCollReduce2 = 7,
    kCollReduce = 8,
};

inline bool is_reduction(int kind) {
    return kind == kCollAllReduce || kind == kCollReduceScatter || kind == kCollReduce || kind == kCollReduce2;
}

// Plans collective `kind` over the N rank buffers.  Contract violations (unknown dtype / op / order /
// schedule / collective, root out of range) throw MegRay::Exception like the reference; shapes a
// single pass cannot honour come back as MEGRAY_INVALID_ARGUMENT with plan_error() set.
Status plan_collective(Plan& plan, int kind, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                       size_t count, DType dtype, int order, int schedule, uint32_t root);

// Enqueue every launch of `plan` on `stream`.
Status execute(const Plan& plan, DType dtype, ReduceOp op, hipStream_t stream);
// The same launches, resolved but not enqueued.
Status resolve(const Plan& plan, DType dtype, ReduceOp op, std::vector<KernelCall>& calls);

// Plans collective `kind` (or finds the plan among the calling thread's last few: same arguments, same buffer
// addresses) and enqueues it.  The flat entry points below all end here.
Status run_collective(int kind, const void* const* send, void* const* recv, uint32_t nranks, size_t count, DType dtype,
                      ReduceOp op, int order, int schedule, uint32_t root, hipStream_t stream);

Status reduce2(const void* i0, const void* i1, void* o, size_t len, DType dtype, ReduceOp op,
               hipStream_t stream);
Status all_reduce(const void* const* send, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                  ReduceOp op, FoldOrder order, Schedule sched, hipStream_t stream);
Status reduce_scatter(const void* const* send, void* const* recv, uint32_t nranks, size_t recvlen,
                      DType dtype, ReduceOp op, FoldOrder order, hipStream_t stream);
Status reduce_to_root(const void* const* send, void* recv_root, uint32_t nranks, size_t len, DType dtype,
                      ReduceOp op, FoldOrder order, uint32_t root, hipStream_t stream);
Status all_gather(const void* const* send, void* const* recv, uint32_t nranks, size_t sendlen, DType dtype,
                  hipStream_t stream);
Status all_to_all(const void* const* send, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                  hipStream_t stream);
Status scatter(const void* send_root, void* const* recv, uint32_t nranks, size_t recvlen, DType dtype,
               uint32_t root, hipStream_t stream);
Status gather(const void* const* send, void* recv_root, uint32_t nranks, size_t sendlen, DType dtype,
              uint32_t root, hipStream_t stream);
Status broadcast(const void* send_root, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                 uint32_t root, hipStream_t stream);

}  // namespace vrank
}  // namespace MegRay
