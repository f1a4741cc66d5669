// MEGRAY_VRANK: the MegRay::Communicator backend whose N ranks are virtual ranks inside one
// process, with all their buffers in one GPU's memory.
//
// It takes the place the reference's UcxCommunicator (src/ucx/communicator.h:28-88) and
// ShmCommunicator (src/shm/communicator.h:84-196) have behind the same abstract class: one object
// per rank, each driven from its own thread, every rank calling the same collective in the same
// order.  A collective call deposits this rank's buffers and stream with the group and waits for
// the other ranks; the last rank to arrive plans the whole collective and enqueues it, after which
// every rank's stream is ordered behind the result.  Calls return once the work is enqueued
// (stream-asynchronous, like the reference's NCCL backend, src/nccl/communicator.cpp:175-186).
#pragma once

#include <memory>
#include <vector>

#include "megray/communicator.h"
#include "vrank_plan.h"

namespace MegRay {

namespace vrank {
class Group;
struct PendingP2P;
}  // namespace vrank

class VRankCommunicator final : public Communicator {
public:
    VRankCommunicator(uint32_t nranks, uint32_t rank);
    ~VRankCommunicator();

    // the Communicator interface (buffer sizes as documented there; `src` / `dst` are this rank's)
    Status do_init() override;
    Status do_init(BcastCallback broadcast_fn) override;
    Status scatter(const void* src, void* dst, size_t per_rank, DType dtype, uint32_t root, ContextPtr ctx) override;
    Status gather(const void* src, void* dst, size_t per_rank, DType dtype, uint32_t root, ContextPtr ctx) override;
    Status all_to_all(const void* src, void* dst, size_t per_pair, DType dtype, ContextPtr ctx) override;
    Status all_gather(const void* src, void* dst, size_t per_rank, DType dtype, ContextPtr ctx) override;
    Status all_reduce(const void* src, void* dst, size_t count, DType dtype, ReduceOp op, ContextPtr ctx) override;
    Status reduce_scatter(const void* src, void* dst, size_t per_rank, DType dtype, ReduceOp op, ContextPtr ctx) override;
    Status broadcast(const void* src, void* dst, size_t count, DType dtype, uint32_t root, ContextPtr ctx) override;
    Status reduce(const void* src, void* dst, size_t count, DType dtype, ReduceOp op, uint32_t root,
                  ContextPtr ctx) override;
    Status group_start() override;
    Status group_end() override;

    // Not part of the reference API: all_reduce for callers that may not allocate device memory
    // (harnesses that forbid it, tight serving loops).  Same result as all_reduce(); the counters that
    // order the ranks' streams are a block of the library's static device array instead of an
    // allocation made at the group's first collective, and there is no fallback to events.  At most
    // vrank::kStaticEdgeSlots groups per process can use it at a time; every rank of a group must make
    // the same call.
    Status all_reduce_no_alloc(const void* src, void* dst, size_t count, DType dtype, ReduceOp op, ContextPtr ctx);

    // Not part of the reference API: has a stream wait of this rank's group given up?  Synchronous: waits for the
    // context's stream, reads the group's counters back, and returns MEGRAY_UNEXPECTED_ERR (for good) if one
    // has.  Collectives report the same on their own - the call after the one that gave up, or, for a group
    // that only ever used all_reduce_no_alloc (which has no host-visible word to report to), within one and a
    // half wait limits; this asks now.
    Status check(ContextPtr ctx);

    // Not part of the reference API: counts kept by this rank's group since it was formed, for benchmarks and
    // diagnosis.  collectives: collectives launched; plans_built: of those, how many had to be planned (the others
    // found their plan in the group's cache); sleeps: times a rank that was waiting for the others gave up polling
    // and went to sleep on a condition variable (a wake-up costs tens of microseconds).
    struct Stats {
        uint64_t collectives, plans_built, sleeps;
    };
    Stats stats() const;

    // Not part of the reference API: which reference loop's combination order all_reduce /
    // reduce_scatter / reduce reproduce (default: the ucx ring), and how all_reduce is laid out in
    // launches (default: fused).  Every rank of a group must choose the same.
    void set_fold_order(vrank::FoldOrder order) { m_order = order; }
    void set_schedule(vrank::Schedule sched) { m_sched = sched; }

protected:
    Status _send(const void* src, size_t bytes, uint32_t peer, ContextPtr ctx) override;
    Status _recv(void* dst, size_t bytes, uint32_t peer, ContextPtr ctx) override;

private:
    Status join(const uint64_t id[2]);
    Status p2p(bool is_send, const void* src, void* dst, size_t bytes, uint32_t peer, ContextPtr ctx);

    std::shared_ptr<vrank::Group> m_group;
    vrank::FoldOrder m_order = vrank::kOrderUcx;
    vrank::Schedule m_sched = vrank::kSchedFused;
    bool m_grouping = false;
    std::vector<std::shared_ptr<vrank::PendingP2P>> m_pending;
};

}  // namespace MegRay
