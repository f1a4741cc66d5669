#include "vrank_engine.h"

#include "megray/hip_context.h"
#include "vrank_kernels.h"

namespace MegRay {
namespace vrank {

uint32_t reduce_elem_size(DType dtype) {
    switch (dtype) {
        case MEGRAY_INT8:
        case MEGRAY_UINT8:
            return 1;
        case MEGRAY_FLOAT16:
            return 2;
        case MEGRAY_INT32:
        case MEGRAY_UINT32:
        case MEGRAY_FLOAT32:
            return 4;
        case MEGRAY_INT64:
        case MEGRAY_UINT64:
        case MEGRAY_FLOAT64:
            return 8;
        default:
            MEGRAY_THROW("unknown dtype");
    }
}

void check_reduce_op(ReduceOp op) {
    if (op != MEGRAY_SUM && op != MEGRAY_MAX && op != MEGRAY_MIN) MEGRAY_THROW("unknown reduce op");
}

namespace {
FoldOrder as_order(int order) {
    if (order < 0 || order >= kOrderCount) MEGRAY_THROW("unknown fold order");
    return static_cast<FoldOrder>(order);
}
Schedule as_schedule(int schedule) {
    if (schedule < 0 || schedule >= kSchedCount) MEGRAY_THROW("unknown schedule");
    return static_cast<Schedule>(schedule);
}
}  // namespace

Status plan_collective(Plan& plan, int kind, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                       size_t count, DType dt, int order, int schedule, uint32_t root) {
    switch (kind) {
        case kCollAllReduce:
            // a ring hop stores its partial result in the element type: FLOAT16 would round N-1 times
            if (as_schedule(schedule) == kSchedRing && dt == MEGRAY_FLOAT16)
                MEGRAY_THROW("the ring schedule is not offered for FLOAT16 (it would round at every hop)");
            return plan_all_reduce(plan, sendbuffs, recvbuffs, nranks, count, reduce_elem_size(dt), as_order(order),
                                   as_schedule(schedule));
        case kCollReduceScatter:
            return plan_reduce_scatter(plan, sendbuffs, recvbuffs, nranks, count, reduce_elem_size(dt),
                                       as_order(order), as_schedule(schedule));
        case kCollAllGather:
            return plan_all_gather(plan, sendbuffs, recvbuffs, nranks, count, uint32_t(get_dtype_size(dt)));
        case kCollAllToAll:
            return plan_all_to_all(plan, sendbuffs, recvbuffs, nranks, count, uint32_t(get_dtype_size(dt)));
        case kCollScatter:
            if (root >= nranks) MEGRAY_THROW("root out of range");
            return plan_scatter(plan, sendbuffs[root], recvbuffs, nranks, count, uint32_t(get_dtype_size(dt)), root);
        case kCollGather:
            if (root >= nranks) MEGRAY_THROW("root out of range");
            return plan_gather(plan, sendbuffs, recvbuffs[root], nranks, count, uint32_t(get_dtype_size(dt)), root);
        case kCollBroadcast:
            if (root >= nranks) MEGRAY_THROW("root out of range");
            return plan_broadcast(plan, sendbuffs[root], recvbuffs, nranks, count, uint32_t(get_dtype_size(dt)),
                                  root);
        case kCollReduce:
            if (root >= nranks) MEGRAY_THROW("root out of range");
            return plan_reduce(plan, sendbuffs, recvbuffs[root], nranks, count, reduce_elem_size(dt), as_order(order),
                               root);
        case kCollReduce2:
            return plan_reduce2(plan, sendbuffs[0], sendbuffs[1], recvbuffs[0], count, reduce_elem_size(dt));
        default:
            MEGRAY_THROW("unknown collective");
    }
}

Status resolve(const Plan& plan, DType dtype, ReduceOp op, std::vector<KernelCall>& calls) {
    calls.clear();
    calls.reserve(plan.steps.size());
    for (const Step& step : plan.steps) {
        KernelCall call{nullptr, 0, kThreads, nullptr};
        switch (step.kind) {
            case Step::kFold:
                call = {fold_kernel_for(step.fold, dtype, op), step.fold.total_tiles, kThreads * step.fold.waves,
                        &step.fold};
                break;
            case Step::kFlat:
                if (step.flat.waves == kGroupWaves)
                    call = {flat_kernel_for(step.flat, dtype, op), group_grid(step.flat.total_tiles),
                            kThreads * kGroupWaves, &step.flat};
                else {
                    call = {flat_kernel_for(step.flat, dtype, op), step.flat.total_tiles, kThreads, &step.flat};
                    // the planner leaves a launch this large at one wavefront per tile only to have it run at a
                    // reduced occupancy (flat_one_out)
                    if (step.flat.total_tiles >= kFlatOneOutMinTiles)
                        call.lds = lds_for_waves_per_cu(call.kernel, flat_one_out_waves_per_cu(step.flat.nranks));
                }
                break;
            case Step::kTree:
                call = {tree_kernel_for(step.tree, dtype, op), step.tree.total_tiles, kThreads, &step.tree};
                if (step.tree.vector && step.tree.elem_size >= 4 && step.tree.total_tiles >= kTreeCapMinTiles)
                    call.lds = lds_for_waves_per_cu(call.kernel, kTreeCapWavesPerCu);
                break;
            case Step::kPack:
                if (step.pack.waves == kGroupWaves)
                    call = {pack_kernel_for(step.pack), step.pack.ncopies * step.pack.groups_per_copy,
                            kThreads * kGroupWaves, &step.pack};
                else
                    call = {pack_kernel_for(step.pack), step.pack.ncopies * step.pack.tiles_per_copy, kThreads,
                            &step.pack};
                break;
        }
        if (!call.kernel) {
            MEGRAY_ERROR("no kernel for dtype %d / op %d", int(dtype), int(op));
            return MEGRAY_INVALID_ARGUMENT;
        }
        calls.push_back(call);
    }
    return MEGRAY_OK;
}

Status execute(const Plan& plan, DType dtype, ReduceOp op, hipStream_t stream) {
    std::vector<KernelCall> calls;
    const Status st = resolve(plan, dtype, op, calls);
    if (st != MEGRAY_OK) return st;
    for (const KernelCall& call : calls) HIP_CHECK(enqueue(call.kernel, call.grid, call.block, call.launch, stream, call.lds));
    return MEGRAY_OK;
}

Status reduce2(const void* i0, const void* i1, void* o, size_t len, DType dtype, ReduceOp op,
               hipStream_t stream) {
    const uint32_t size = reduce_elem_size(dtype);
    check_reduce_op(op);
    Plan plan;
    Status st = plan_reduce2(plan, i0, i1, o, len, size);
    return st == MEGRAY_OK ? execute(plan, dtype, op, stream) : st;
}

Status all_reduce(const void* const* send, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                  ReduceOp op, FoldOrder order, Schedule sched, hipStream_t stream) {
    const uint32_t size = reduce_elem_size(dtype);
    check_reduce_op(op);
    // a ring hop stores its partial result in the element type: FLOAT16 would round N-1 times
    if (sched == kSchedRing && dtype == MEGRAY_FLOAT16)
        MEGRAY_THROW("the ring schedule is not offered for FLOAT16 (it would round at every hop)");
    Plan plan;
    Status st = plan_all_reduce(plan, send, recv, nranks, len, size, order, sched);
    return st == MEGRAY_OK ? execute(plan, dtype, op, stream) : st;
}

Status reduce_scatter(const void* const* send, void* const* recv, uint32_t nranks, size_t recvlen,
                      DType dtype, ReduceOp op, FoldOrder order, hipStream_t stream) {
    const uint32_t size = reduce_elem_size(dtype);
    check_reduce_op(op);
    Plan plan;
    Status st = plan_reduce_scatter(plan, send, recv, nranks, recvlen, size, order, kSchedFused);
    return st == MEGRAY_OK ? execute(plan, dtype, op, stream) : st;
}

Status reduce_to_root(const void* const* send, void* recv_root, uint32_t nranks, size_t len, DType dtype,
                      ReduceOp op, FoldOrder order, uint32_t root, hipStream_t stream) {
    const uint32_t size = reduce_elem_size(dtype);
    check_reduce_op(op);
    Plan plan;
    Status st = plan_reduce(plan, send, recv_root, nranks, len, size, order, root);
    return st == MEGRAY_OK ? execute(plan, dtype, op, stream) : st;
}

Status all_gather(const void* const* send, void* const* recv, uint32_t nranks, size_t sendlen, DType dtype,
                  hipStream_t stream) {
    Plan plan;
    Status st = plan_all_gather(plan, send, recv, nranks, sendlen, uint32_t(get_dtype_size(dtype)));
    return st == MEGRAY_OK ? execute(plan, dtype, MEGRAY_SUM, stream) : st;
}

Status all_to_all(const void* const* send, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                  hipStream_t stream) {
    Plan plan;
    Status st = plan_all_to_all(plan, send, recv, nranks, len, uint32_t(get_dtype_size(dtype)));
    return st == MEGRAY_OK ? execute(plan, dtype, MEGRAY_SUM, stream) : st;
}

Status scatter(const void* send_root, void* const* recv, uint32_t nranks, size_t recvlen, DType dtype,
               uint32_t root, hipStream_t stream) {
    Plan plan;
    Status st = plan_scatter(plan, send_root, recv, nranks, recvlen, uint32_t(get_dtype_size(dtype)), root);
    return st == MEGRAY_OK ? execute(plan, dtype, MEGRAY_SUM, stream) : st;
}

Status gather(const void* const* send, void* recv_root, uint32_t nranks, size_t sendlen, DType dtype,
              uint32_t root, hipStream_t stream) {
    Plan plan;
    Status st = plan_gather(plan, send, recv_root, nranks, sendlen, uint32_t(get_dtype_size(dtype)), root);
    return st == MEGRAY_OK ? execute(plan, dtype, MEGRAY_SUM, stream) : st;
}

Status broadcast(const void* send_root, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                 uint32_t root, hipStream_t stream) {
    Plan plan;
    Status st = plan_broadcast(plan, send_root, recv, nranks, len, uint32_t(get_dtype_size(dtype)), root);
    return st == MEGRAY_OK ? execute(plan, dtype, MEGRAY_SUM, stream) : st;
}

}  // namespace vrank
}  // namespace MegRay
