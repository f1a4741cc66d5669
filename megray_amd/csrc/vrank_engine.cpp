#include "vrank_engine.h"

#include <cstdlib>
#include <cstring>
#include <memory>

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

namespace {
Status plan_steps(Plan& plan, int kind, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
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
}  // namespace

Status plan_collective(Plan& plan, int kind, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                       size_t count, DType dt, int order, int schedule, uint32_t root) {
    const Status st = plan_steps(plan, kind, sendbuffs, recvbuffs, nranks, count, dt, order, schedule, root);
    if (st == MEGRAY_OK) set_store_policy(plan);
    return st;
}

namespace {
// Workgroups per CU for the group form of the general fold kernel with a run-time fold width (5, 6, 7 and 9 - 32
// inputs, staged through LDS four at a time; its LDS allows 7), 0 = as many as fit.  Measured on MI355X, fp32, placed
// buffers, % of the HBM peak, interleaved in one process, as the LDS allows -> capped:
//   all_reduce shapes (every rank an output), accesses at once, 256 MiB per rank -> 4 per CU:
//     6 / 7 / 10 / 12 / 16 ranks 81.3 -> 82.3 / 81.5 -> 82.0 / 80.5 -> 82.5 / 80.3 -> 81.8 / 80.9 -> 81.6
//     (3 per CU: 78 / 80 / 81.3 / 82.2 / 82.1; 5 per CU: 82.4 / 82.3 / 81.6 / 81.0 / 81.9); 64 MiB per rank, 6 / 7 / 12 ranks:
//     78.9 -> 79.7 / 78.7 -> 80.8 / 78.6 -> 80.8; 16 / 32 MiB per rank, 6 / 7 / 10 / 12 / 16 ranks: 77.8 -> 78.8 / 75.7 -> 78.3 / 71.7 -> 72.9 /
//     71.7 -> 73.9 / 72.7 -> 75.7 and 74.9 -> 75.2 / 76.1 -> 78.1 / 75.5 -> 77.2 / 76.3 -> 78.4 / 77.3 -> 79.5; at 8 MiB + 1 to - 1;
//     5 ranks gain nothing at any occupancy
//   folds into one output that pace their accesses (reduce_scatter from 1 GiB over all buffers) -> 6 per CU:
//     6 / 7 / 10 / 12 / 16 ranks x 256 MiB 80.1 -> 84.0 / 80.9 -> 83.6 / 81.7 -> 83.7 / 82.0 -> 84.2 / 84.3 -> 85.4 (5 ranks 82.8 -> 82.3;
//     at 7 per CU, reserved the same way, nothing changes; 5 per CU loses 1 - 7 points)
// The same for the group form of the flat fold: long launches that issue a wavefront's accesses at once run at fewer
// workgroups per CU than their LDS allows - the all_reduce shapes (tables at group_cap_per_cu in vrank_types.h), and
// the fold of two inputs into one output, which is the reference's own kernel shape (mrv_reduce) and the reduce_scatter
// of two ranks: 1 GiB per buffer 86.3 -> 87.4 % of the HBM peak at 5 per CU (6: 86.8, 4: 83.4, 3: 71.2), reduce_scatter of
// 2 x 512 MiB 84.8 -> 86.0; at 128 MiB per buffer the cap costs a point (87.9 -> 86.9) and is not applied.
uint32_t flat_group_per_cu(const FlatLaunch& L) {
    if (L.exchange & kFlatPaced) return 0;
    const uint64_t bytes = L.count * L.elem_size;
    if (L.exchange & 1u) return bytes >= (L.nranks >= 8 ? kGroupCapMinBytes8 : kGroupCapMinBytes) ? group_cap_per_cu(L.nranks) : 0;
    if (L.nranks == 2 && L.nout == 1) return bytes >= (uint64_t(512) << 20) ? 5u : 0u;
    return 0;
}

uint32_t general_group_per_cu(const FoldLaunch& L) {
    if (L.nfold < 6 || L.nfold == 8) return 0;  // 1, 2, 3, 4 and 8 inputs run kernels of their own
    if (L.nout == 1) return L.paced ? 6u : 0u;
    const bool long_launch = L.total_tiles >= 4096;  // 16 MiB per buffer: a workgroup takes 4 KiB of each
    return L.nout == L.nranks && !L.paced && long_launch ? 4u : 0u;
}
}  // namespace

Status resolve(const Plan& plan, DType dtype, ReduceOp op, std::vector<KernelCall>& calls) {
    calls.clear();
    calls.reserve(plan.steps.size());
    // MEGRAY_VRANK_GROUP_PER_CU=n in the environment runs every group-form fold at n workgroups per CU instead of
    // what the tables say (for measurements; 0 or unset: the tables)
    const char* forced_text = std::getenv("MEGRAY_VRANK_GROUP_PER_CU");
    const uint32_t forced = forced_text ? uint32_t(std::strtoul(forced_text, nullptr, 10)) : 0;
    for (const Step& step : plan.steps) {
        KernelCall call{nullptr, 0, kThreads, nullptr};
        switch (step.kind) {
            case Step::kFold:
                call = {fold_kernel_for(step.fold, dtype, op), step.fold.total_tiles, kThreads * step.fold.waves,
                        &step.fold};
                if (step.fold.waves == kGroupWaves) {
                    const uint32_t per_cu = forced ? forced : general_group_per_cu(step.fold);
                    if (per_cu) call.lds = lds_for_waves_per_cu(call.kernel, per_cu);
                }
                break;
            case Step::kFlat:
                if (step.flat.waves == kGroupWaves) {
                    call = {flat_kernel_for(step.flat, dtype, op), group_grid(step.flat.total_tiles),
                            kThreads * kGroupWaves, &step.flat};
                    const uint32_t per_cu = forced ? forced : flat_group_per_cu(step.flat);
                    if (per_cu) call.lds = lds_for_waves_per_cu(call.kernel, per_cu);
                } else {
                    call = {flat_kernel_for(step.flat, dtype, op), step.flat.total_tiles, kThreads, &step.flat};
                    // the planner leaves a launch this large at one wavefront per tile only to have it run at an
                    // occupancy of its own (flat_one_out_waves_per_cu)
                    if (step.flat.total_tiles >= kFlatOneOutMinTiles) {
                        const bool keep = (step.flat.exchange & kFlatKeep) != 0;
                        const uint32_t per_cu = flat_one_out_waves_per_cu(step.flat.nranks, step.flat.total_tiles, keep, step.flat.elem_size);
                        if (per_cu) call.lds = lds_for_waves_per_cu(call.kernel, per_cu);
                    }
                }
                break;
            case Step::kTree:
                call = {tree_kernel_for(step.tree, dtype, op), step.tree.total_tiles, kThreads, &step.tree};
                if (step.tree.vector) {
                    const uint32_t per_cu = tree_waves_per_cu(step.tree.nranks, step.tree.total_tiles, step.tree.keep != 0, step.tree.elem_size);
                    if (per_cu) call.lds = lds_for_waves_per_cu(call.kernel, per_cu);
                }
                break;
            case Step::kPack:
                if (step.pack.waves == kGroupWaves) {
                    call = {pack_kernel_for(step.pack), step.pack.ncopies * step.pack.groups_per_copy,
                            kThreads * kGroupWaves, &step.pack};
                    if (forced) call.lds = lds_for_waves_per_cu(call.kernel, forced);
                } else
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

namespace {

// The flat entry points plan on every call, and planning a small collective costs as much as launching it (the
// reference re-derives its chunking per call as well, src/ucx/all_reduce.cpp:33-51).  Callers repeat their
// collectives on the same buffers, so each thread keeps the last few plans, found by everything a plan depends on:
// the collective, its arguments and the buffer addresses.  (The communicator keeps such a cache per group, and
// mrv_plan_* lets a caller hold a plan explicitly.)
struct FlatKey {
    int kind, order, sched, pace;
    uint32_t nranks, root;
    size_t count;
    DType dtype;
    ReduceOp op;
    int device;
    const void* send[kMaxRanks];
    void* recv[kMaxRanks];
};

struct FlatEntry {
    FlatKey key;
    uint64_t signature = 0;  // a mix of the key's words: compared first
    uint64_t last_used = 0;
    Plan plan;
    std::vector<KernelCall> calls;  // point into `plan`
};

constexpr size_t kFlatCacheSlots = 16;

bool same_key(const FlatKey& a, const FlatKey& b) {
    return a.kind == b.kind && a.order == b.order && a.sched == b.sched && a.pace == b.pace && a.nranks == b.nranks &&
           a.root == b.root && a.count == b.count && a.dtype == b.dtype && a.op == b.op && a.device == b.device &&
           std::memcmp(a.send, b.send, sizeof(a.send)) == 0 && std::memcmp(a.recv, b.recv, sizeof(a.recv)) == 0;
}

uint64_t key_signature(const FlatKey& key) {
    static_assert(sizeof(FlatKey) % sizeof(uint64_t) == 0, "the key is hashed word by word");
    uint64_t words[sizeof(FlatKey) / sizeof(uint64_t)];
    std::memcpy(words, &key, sizeof(key));
    uint64_t h = 0x9e3779b97f4a7c15ull;
    for (uint64_t w : words) {
        h ^= w + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
        h *= 0xff51afd7ed558ccdull;
    }
    return h ^ (h >> 32);
}

}  // namespace

Status run_collective(int kind, const void* const* send, void* const* recv, uint32_t nranks, size_t count, DType dtype,
                      ReduceOp op, int order, int schedule, uint32_t root, hipStream_t stream) {
    if (nranks < 1 || nranks > kMaxRanks) {  // the planner says so; nothing to remember
        Plan plan;
        const Status st = plan_collective(plan, kind, send, recv, nranks, count, dtype, order, schedule, root);
        return st == MEGRAY_OK ? execute(plan, dtype, is_reduction(kind) ? op : MEGRAY_SUM, stream) : st;
    }
    thread_local std::vector<std::unique_ptr<FlatEntry>> cache;
    thread_local uint64_t clock = 0;
    FlatKey key;
    std::memset(&key, 0, sizeof(key));
    key.kind = kind, key.order = order, key.sched = schedule, key.pace = plan_overrides();  // the planner reads the environment: part of what a plan depends on
    key.nranks = nranks, key.root = root, key.count = count, key.dtype = dtype, key.op = is_reduction(kind) ? op : MEGRAY_SUM;
    if (hipGetDevice(&key.device) != hipSuccess) {
        (void)hipGetLastError();
        key.device = -1;
    }
    // which pointers a collective looks at: the rooted ones only their root's on one side
    const bool send_root_only = kind == kCollScatter || kind == kCollBroadcast;
    const bool recv_root_only = kind == kCollGather || kind == kCollReduce;
    const uint32_t nsend = kind == kCollReduce2 ? 2 : nranks, nrecv = kind == kCollReduce2 ? 1 : nranks;
    for (uint32_t r = 0; r < nsend; ++r)
        if (!send_root_only || r == root) key.send[r] = send[r];
    for (uint32_t r = 0; r < nrecv; ++r)
        if (!recv_root_only || r == root) key.recv[r] = recv[r];
    const uint64_t signature = key_signature(key);
    FlatEntry* hit = nullptr;
    for (auto& e : cache)
        if (e->signature == signature && same_key(e->key, key)) hit = e.get();
    if (!hit) {
        auto fresh = std::make_unique<FlatEntry>();
        fresh->key = key;
        fresh->signature = signature;
        Status st = plan_collective(fresh->plan, kind, send, recv, nranks, count, dtype, order, schedule, root);
        if (st == MEGRAY_OK) st = resolve(fresh->plan, dtype, key.op, fresh->calls);
        if (st != MEGRAY_OK) return st;
        if (cache.size() < kFlatCacheSlots) {
            cache.push_back(std::move(fresh));
            hit = cache.back().get();
        } else {
            size_t oldest = 0;
            for (size_t i = 1; i < cache.size(); ++i)
                if (cache[i]->last_used < cache[oldest]->last_used) oldest = i;
            cache[oldest] = std::move(fresh);
            hit = cache[oldest].get();
        }
    }
    hit->last_used = ++clock;
    for (const KernelCall& call : hit->calls) HIP_CHECK(enqueue(call.kernel, call.grid, call.block, call.launch, stream, call.lds));
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
    (void)reduce_elem_size(dtype);
    check_reduce_op(op);
    const void* send[2] = {i0, i1};
    void* recv[1] = {o};
    return run_collective(kCollReduce2, send, recv, 2, len, dtype, op, kOrderUcx, kSchedFused, 0, stream);
}

Status all_reduce(const void* const* send, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                  ReduceOp op, FoldOrder order, Schedule sched, hipStream_t stream) {
    (void)reduce_elem_size(dtype);
    check_reduce_op(op);
    return run_collective(kCollAllReduce, send, recv, nranks, len, dtype, op, order, sched, 0, stream);
}

Status reduce_scatter(const void* const* send, void* const* recv, uint32_t nranks, size_t recvlen,
                      DType dtype, ReduceOp op, FoldOrder order, hipStream_t stream) {
    (void)reduce_elem_size(dtype);
    check_reduce_op(op);
    return run_collective(kCollReduceScatter, send, recv, nranks, recvlen, dtype, op, order, kSchedFused, 0, stream);
}

namespace {
// The rooted collectives' one-sided argument as a per-rank table with the root's entry set.
struct RootTable {
    const void* send[kMaxRanks] = {};
    void* recv[kMaxRanks] = {};
};
void check_root(uint32_t nranks, uint32_t root) {
    if (nranks < 1 || nranks > kMaxRanks) MEGRAY_THROW("nranks must be in [1, 32]");
    if (root >= nranks) MEGRAY_THROW("root out of range");
}
}  // namespace

Status reduce_to_root(const void* const* send, void* recv_root, uint32_t nranks, size_t len, DType dtype,
                      ReduceOp op, FoldOrder order, uint32_t root, hipStream_t stream) {
    (void)reduce_elem_size(dtype);
    check_reduce_op(op);
    check_root(nranks, root);
    RootTable t;
    t.recv[root] = recv_root;
    return run_collective(kCollReduce, send, t.recv, nranks, len, dtype, op, order, kSchedFused, root, stream);
}

Status all_gather(const void* const* send, void* const* recv, uint32_t nranks, size_t sendlen, DType dtype,
                  hipStream_t stream) {
    return run_collective(kCollAllGather, send, recv, nranks, sendlen, dtype, MEGRAY_SUM, kOrderUcx, kSchedFused, 0, stream);
}

Status all_to_all(const void* const* send, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                  hipStream_t stream) {
    return run_collective(kCollAllToAll, send, recv, nranks, len, dtype, MEGRAY_SUM, kOrderUcx, kSchedFused, 0, stream);
}

Status scatter(const void* send_root, void* const* recv, uint32_t nranks, size_t recvlen, DType dtype,
               uint32_t root, hipStream_t stream) {
    (void)get_dtype_size(dtype);
    check_root(nranks, root);
    RootTable t;
    t.send[root] = send_root;
    return run_collective(kCollScatter, t.send, recv, nranks, recvlen, dtype, MEGRAY_SUM, kOrderUcx, kSchedFused, root, stream);
}

Status gather(const void* const* send, void* recv_root, uint32_t nranks, size_t sendlen, DType dtype,
              uint32_t root, hipStream_t stream) {
    (void)get_dtype_size(dtype);
    check_root(nranks, root);
    RootTable t;
    t.recv[root] = recv_root;
    return run_collective(kCollGather, send, t.recv, nranks, sendlen, dtype, MEGRAY_SUM, kOrderUcx, kSchedFused, root, stream);
}

Status broadcast(const void* send_root, void* const* recv, uint32_t nranks, size_t len, DType dtype,
                 uint32_t root, hipStream_t stream) {
    (void)get_dtype_size(dtype);
    check_root(nranks, root);
    RootTable t;
    t.send[root] = send_root;
    return run_collective(kCollBroadcast, t.send, recv, nranks, len, dtype, MEGRAY_SUM, kOrderUcx, kSchedFused, root, stream);
}

}  // namespace vrank
}  // namespace MegRay
