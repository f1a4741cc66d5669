#include "vrank_communicator.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <map>
#include <mutex>
#include <random>

#include <unistd.h>

#include "megray/hip_context.h"
#include "vrank_engine.h"

namespace MegRay {
namespace vrank {

namespace {

enum class Kind : int { kScatter, kGather, kAllToAll, kAllGather, kAllReduce, kReduceScatter, kBroadcast, kReduce };

// What one rank brings to a collective.
struct Call {
    Kind kind;
    size_t len;
    DType dtype;
    ReduceOp op;
    uint32_t root;
    FoldOrder order;
    Schedule sched;
    const void* send;
    void* recv;
    hipStream_t stream;
    int device;
    bool arrived_recorded = false;  // the rank marked its stream's position itself (see Group::collective)
};

bool same_collective(const Call& a, const Call& b) {
    return a.kind == b.kind && a.len == b.len && a.dtype == b.dtype && a.op == b.op && a.root == b.root &&
           a.order == b.order && a.sched == b.sched && a.device == b.device;
}

}  // namespace

// One posted send or receive.
struct PendingP2P {
    bool is_send;
    const void* src;
    void* dst;
    size_t size;
    hipStream_t stream;
    int device;
    bool done;
    Status status;
};

// The process-local meeting point of the N rank objects of one communicator group.
class Group {
public:
    explicit Group(uint32_t nranks)
            : m_nranks(nranks), m_slots(nranks), m_arrive(nranks, nullptr), m_mail(size_t(nranks) * nranks) {}

    ~Group() {
        for (hipEvent_t ev : m_events) (void)hipEventDestroy(ev);
        for (hipEvent_t ev : m_arrive)
            if (ev) (void)hipEventDestroy(ev);
        if (m_done) (void)hipEventDestroy(m_done);
        for (uint64_t* c : m_counters) (void)hipFree(c);
    }

    // Groups are found by the 128-bit id rank 0 drew and the bootstrap broadcast.
    static std::shared_ptr<Group> join(const uint64_t id[2], uint32_t nranks) {
        static std::mutex registry_mutex;
        static std::map<std::pair<uint64_t, uint64_t>, std::weak_ptr<Group>> registry;
        std::lock_guard<std::mutex> lock(registry_mutex);
        for (auto it = registry.begin(); it != registry.end();)
            it = it->second.expired() ? registry.erase(it) : std::next(it);
        auto key = std::make_pair(id[0], id[1]);
        std::shared_ptr<Group> group = registry[key].lock();
        if (!group) {
            group = std::make_shared<Group>(nranks);
            registry[key] = group;
        }
        return group->m_nranks == nranks ? group : nullptr;
    }

    // Deposit `call` for `rank` and wait until every rank of the group has done the same; the last
    // to arrive enqueues the collective for all.  Every rank returns the same Status.
    Status collective(uint32_t rank, const Call& in_call) {
        Call call = in_call;
        // Every rank marks, on its own stream and from its own thread, the point its buffers are
        // ready at; the N records run in parallel instead of one after the other in the leader.
        // A rank whose stream is the one every rank shared last time skips the record: if all ranks
        // share a stream again nobody needs it (no cross-stream edge exists), and if not, the leader
        // records it on the rank's behalf before it waits on it.
        const bool shared = m_shared_valid.load(std::memory_order_acquire) &&
                            m_shared_stream.load(std::memory_order_relaxed) == static_cast<void*>(call.stream);
        const uint64_t ticket = m_generation.load(std::memory_order_acquire) + 1;  // stable until this rank arrives
        if (!shared) {
            MEGRAY_CHECK(mark(rank, call.stream, ticket));
            call.arrived_recorded = true;
        }

        std::unique_lock<std::mutex> lock(m_mutex);
        m_slots[rank] = call;
        const uint64_t gen = m_generation.load(std::memory_order_relaxed);
        if (++m_arrived == m_nranks) {
            Status st;
            try {
                st = launch(rank);
            } catch (const MegRay::Exception& e) {
                MEGRAY_ERROR("collective failed: %s", e.what());
                st = MEGRAY_INVALID_ARGUMENT;
            }
            m_result[gen & 1] = st;
            m_lead_stream[gen & 1] = call.stream;
            m_arrived = 0;
            m_generation.store(gen + 1, std::memory_order_release);
            lock.unlock();
            m_cv.notify_all();
            return st;
        }
        lock.unlock();
        // The other ranks are usually a few microseconds away: poll the generation for a while before
        // going to sleep on the condition variable (a sleeping thread costs tens of microseconds to wake).
        bool released = false;
        for (int spin = 0; spin < kSpinPolls && !released; ++spin) {
            released = m_generation.load(std::memory_order_acquire) != gen;
            if (!released) __builtin_ia32_pause();
        }
        if (!released) {
            lock.lock();
            m_cv.wait(lock, [&] { return m_generation.load(std::memory_order_acquire) != gen; });
            lock.unlock();
        }
        // ... and orders its own stream behind the result.  The done mark is not set again before
        // every rank has passed this point: the next collective needs all of them to arrive first.
        const Status st = m_result[gen & 1];
        if (st == MEGRAY_OK && call.stream != m_lead_stream[gen & 1]) MEGRAY_CHECK(await(m_nranks, call.stream, gen + 1));
        return st;
    }

    // Post one side of a point-to-point transfer; the side that finds its counterpart already
    // posted enqueues the copy.  Matching is first come, first served per (source, destination).
    void post(uint32_t src_rank, uint32_t dst_rank, const std::shared_ptr<PendingP2P>& op) {
        std::lock_guard<std::mutex> lock(m_mutex);
        Mailbox& box = m_mail[size_t(src_rank) * m_nranks + dst_rank];
        auto& mine = op->is_send ? box.sends : box.recvs;
        auto& theirs = op->is_send ? box.recvs : box.sends;
        if (theirs.empty()) {
            mine.push_back(op);
            return;
        }
        std::shared_ptr<PendingP2P> other = theirs.front();
        theirs.pop_front();
        PendingP2P& s = op->is_send ? *op : *other;
        PendingP2P& r = op->is_send ? *other : *op;
        Status st = transfer(s, r);
        s.status = r.status = st;
        s.done = r.done = true;
        m_cv.notify_all();
    }

    Status wait(const std::shared_ptr<PendingP2P>& op) {
        std::unique_lock<std::mutex> lock(m_mutex);
        m_cv.wait(lock, [&] { return op->done; });
        return op->status;
    }

private:
    struct Mailbox {
        std::deque<std::shared_ptr<PendingP2P>> sends, recvs;
    };

    hipEvent_t event(size_t index) {
        while (m_events.size() <= index) {
            hipEvent_t ev;
            HIP_ASSERT(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
            m_events.push_back(ev);
        }
        return m_events[index];
    }

    // Cross-stream ordering, "stream B goes on after what stream A holds now", is a mark on A and an
    // await on B.  Where the runtime has stream memory operations, a mark writes a ticket (the
    // collective's number) into a 64-bit counter in signal memory and an await polls it for
    // ">= ticket"; measured on MI355X with 8 threads each doing one mark and one cross-stream await,
    // that costs 27 us a round against 71 us with event record / stream-wait-event, which is the
    // fallback.  Slot r < nranks: rank r has arrived; slot nranks: the collective is enqueued.
    void prepare_edges(hipStream_t probe) {
        std::call_once(m_edges_once, [&] {
            // MEGRAY_VRANK_EDGES=events in the environment keeps to events
            const char* choice = std::getenv("MEGRAY_VRANK_EDGES");
            if (choice && std::strcmp(choice, "events") == 0) return;
            // hipStreamWaitValue64 polls "signal memory" only (an 8-byte allocation of its own kind per
            // counter), and a device says whether it can
            int device = 0, can_wait = 0;
            if (hipGetDevice(&device) != hipSuccess ||
                hipDeviceGetAttribute(&can_wait, hipDeviceAttributeCanUseStreamWaitValue, device) != hipSuccess ||
                !can_wait) {
                (void)hipGetLastError();
                return;
            }
            std::vector<uint64_t*> counters(m_nranks + 1, nullptr);
            bool ok = true;
            for (uint64_t*& c : counters) {
                ok = ok && hipExtMallocWithFlags(reinterpret_cast<void**>(&c), sizeof(uint64_t), hipMallocSignalMemory) ==
                                   hipSuccess;
                ok = ok && hipStreamWriteValue64(probe, c, 0, 0) == hipSuccess;
            }
            ok = ok && hipStreamSynchronize(probe) == hipSuccess;
            if (!ok) {
                (void)hipGetLastError();
                for (uint64_t* c : counters)
                    if (c) (void)hipFree(c);
                return;
            }
            m_counters = counters;
        });
    }

    Status mark(uint32_t slot, hipStream_t stream, uint64_t ticket) {
        prepare_edges(stream);
        if (!m_counters.empty()) {
            HIP_CHECK(hipStreamWriteValue64(stream, m_counters[slot], ticket, 0));
            return MEGRAY_OK;
        }
        hipEvent_t& ev = slot < m_nranks ? m_arrive[slot] : m_done;
        if (!ev) HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        HIP_CHECK(hipEventRecord(ev, stream));
        return MEGRAY_OK;
    }

    Status await(uint32_t slot, hipStream_t stream, uint64_t ticket) {
        if (!m_counters.empty()) {
            HIP_CHECK(hipStreamWaitValue64(stream, m_counters[slot], ticket, hipStreamWaitValueGte, ~uint64_t(0)));
            return MEGRAY_OK;
        }
        HIP_CHECK(hipStreamWaitEvent(stream, slot < m_nranks ? m_arrive[slot] : m_done, 0));
        return MEGRAY_OK;
    }

    // Called with the mutex held by the last rank to arrive.
    Status launch(uint32_t leader) {
        const Call& lead = m_slots[leader];
        for (uint32_t r = 0; r < m_nranks; ++r) {
            if (!same_collective(lead, m_slots[r])) {
                MEGRAY_ERROR("rank %u and rank %u called different collectives (or with different arguments)",
                             leader, r);
                return MEGRAY_INVALID_USAGE;
            }
        }
        const void* send[kMaxRanks] = {};
        void* recv[kMaxRanks] = {};
        for (uint32_t r = 0; r < m_nranks; ++r) {
            send[r] = m_slots[r].send;
            recv[r] = m_slots[r].recv;
        }
        // order the leader's stream behind everything already enqueued on the other ranks' streams
        hipStream_t stream = lead.stream;
        bool one_stream = true;
        for (uint32_t r = 0; r < m_nranks; ++r) {
            if (m_slots[r].stream == stream) continue;
            one_stream = false;
            const uint64_t ticket = m_generation.load(std::memory_order_relaxed) + 1;
            // a rank that expected everyone on its stream did not mark it; it is parked in collective(),
            // so its stream's tail is still the point it arrived at
            if (!m_slots[r].arrived_recorded) MEGRAY_CHECK(mark(r, m_slots[r].stream, ticket));
            MEGRAY_CHECK(await(r, stream, ticket));
        }
        m_shared_stream.store(static_cast<void*>(stream), std::memory_order_relaxed);
        m_shared_valid.store(one_stream, std::memory_order_release);
        Status st = MEGRAY_OK;
        const uint32_t n = m_nranks;
        switch (lead.kind) {
            case Kind::kAllReduce:
                st = all_reduce(send, recv, n, lead.len, lead.dtype, lead.op, lead.order, lead.sched, stream);
                break;
            case Kind::kReduceScatter:
                st = reduce_scatter(send, recv, n, lead.len, lead.dtype, lead.op, lead.order, stream);
                break;
            case Kind::kAllGather:
                st = all_gather(send, recv, n, lead.len, lead.dtype, stream);
                break;
            case Kind::kAllToAll:
                st = all_to_all(send, recv, n, lead.len, lead.dtype, stream);
                break;
            case Kind::kScatter:
                st = scatter(send[lead.root], recv, n, lead.len, lead.dtype, lead.root, stream);
                break;
            case Kind::kGather:
                st = gather(send, recv[lead.root], n, lead.len, lead.dtype, lead.root, stream);
                break;
            case Kind::kBroadcast:
                st = broadcast(send[lead.root], recv, n, lead.len, lead.dtype, lead.root, stream);
                break;
            case Kind::kReduce:
                st = reduce_to_root(send, recv[lead.root], n, lead.len, lead.dtype, lead.op, lead.order, lead.root,
                                    stream);
                break;
        }
        if (st == MEGRAY_INVALID_ARGUMENT) MEGRAY_ERROR("collective rejected: %s", plan_error());
        // the other ranks order their streams behind this point themselves (none has to if all share the stream)
        if (!one_stream) MEGRAY_CHECK(mark(m_nranks, stream, m_generation.load(std::memory_order_relaxed) + 1));
        return st;
    }

    // Enqueue the copy of a matched send / receive pair: on the receiver's stream, after the
    // sender's stream has reached the send, and before the sender's stream goes on.
    Status transfer(const PendingP2P& s, const PendingP2P& r) {
        if (s.size != r.size || s.device != r.device) {
            MEGRAY_ERROR("send of %zu bytes met a receive of %zu bytes", s.size, r.size);
            return MEGRAY_INVALID_USAGE;
        }
        if (!s.size) return MEGRAY_OK;
        const size_t base = 0;
        if (s.stream != r.stream) {
            HIP_CHECK(hipEventRecord(event(base), s.stream));
            HIP_CHECK(hipStreamWaitEvent(r.stream, event(base), 0));
        }
        HIP_CHECK(hipMemcpyAsync(r.dst, s.src, s.size, hipMemcpyDeviceToDevice, r.stream));
        if (s.stream != r.stream) {
            HIP_CHECK(hipEventRecord(event(base + 1), r.stream));
            HIP_CHECK(hipStreamWaitEvent(s.stream, event(base + 1), 0));
        }
        return MEGRAY_OK;
    }

    const uint32_t m_nranks;
    std::mutex m_mutex;
    std::condition_variable m_cv;
    std::vector<Call> m_slots;
    uint32_t m_arrived = 0;
    std::atomic<uint64_t> m_generation{0};
    static constexpr int kSpinPolls = 20000;
    Status m_result[2] = {MEGRAY_OK, MEGRAY_OK};
    hipStream_t m_lead_stream[2] = {nullptr, nullptr};
    std::atomic<void*> m_shared_stream{nullptr};  // the stream of the last collective, ...
    std::atomic<bool> m_shared_valid{false};      // ... if every rank passed that same one
    std::once_flag m_edges_once;
    std::vector<uint64_t*> m_counters;  // signal memory, one per slot; empty: the events below are used instead
    std::vector<hipEvent_t> m_arrive;  // per rank: "my buffers are ready", recorded by the rank itself
    hipEvent_t m_done = nullptr;       // recorded by the leader behind the collective
    std::vector<hipEvent_t> m_events;  // point-to-point transfers
    std::vector<Mailbox> m_mail;
};

}  // namespace vrank

using namespace vrank;

namespace {

hipStream_t stream_of(const std::shared_ptr<Context>& ctx) {
    // the reference asserts the context type first thing in every collective
    // (src/ucx/all_reduce.cpp:27-28); this backend takes HIP streams
    MEGRAY_ASSERT(ctx && ctx->type() == MEGRAY_CTX_HIP, "only hip context supported");
    return static_cast<HipContext*>(ctx.get())->get_stream();
}

int current_device() {
    int device = 0;
    HIP_ASSERT(hipGetDevice(&device));
    return device;
}

void draw_group_id(uint64_t id[2]) {
    static std::atomic<uint64_t> counter{0};
    std::random_device rd;
    id[0] = (uint64_t(rd()) << 32) ^ rd() ^ uint64_t(getpid());
    id[1] = (uint64_t(std::chrono::steady_clock::now().time_since_epoch().count()) << 16) ^ ++counter;
}

}  // namespace

VRankCommunicator::VRankCommunicator(uint32_t nranks, uint32_t rank) : Communicator(nranks, rank) {
    MEGRAY_ASSERT(nranks >= 1 && nranks <= kMaxRanks, "the vrank backend takes 1 to %u ranks", kMaxRanks);
    MEGRAY_ASSERT(rank < nranks, "rank %u out of range", rank);
}

VRankCommunicator::~VRankCommunicator() = default;

Status VRankCommunicator::join(const uint64_t id[2]) {
    m_group = Group::join(id, m_nranks);
    if (!m_group) {
        MEGRAY_ERROR("ranks of one group disagree on the number of ranks");
        return MEGRAY_INVALID_USAGE;
    }
    return MEGRAY_OK;
}

// Rank 0 draws the group id and the bootstrap client broadcasts it, the way the reference hands
// out its NCCL unique id (src/nccl/communicator.cpp:42-52).  All ranks must live in one process.
Status VRankCommunicator::do_init() {
    uint64_t id[2] = {0, 0};
    if (m_rank == 0) draw_group_id(id);
    MEGRAY_CHECK(m_client->broadcast(id, id, sizeof(id), 0));
    std::vector<int64_t> pids(m_nranks);
    const int64_t pid = getpid();
    MEGRAY_CHECK(m_client->allgather(&pid, pids.data(), sizeof(pid)));
    for (int64_t p : pids) {
        if (p != pid) {
            MEGRAY_ERROR("MEGRAY_VRANK needs every rank of the group in one process");
            return MEGRAY_INVALID_USAGE;
        }
    }
    return join(id);
}

// Same with a caller-supplied broadcast (src/nccl/communicator.cpp:54-64).
Status VRankCommunicator::do_init(BcastCallback cb) {
    uint64_t id[2] = {0, 0};
    if (m_rank == 0) draw_group_id(id);
    cb(reinterpret_cast<char*>(id), sizeof(id));
    return join(id);
}

#define VRANK_COLLECTIVE(KIND, LEN, DTYPE, OP, ROOT)                                        \
    do {                                                                                    \
        MEGRAY_ASSERT(m_group != nullptr, "communicator used before init()");               \
        Call call{KIND, LEN, DTYPE, OP, ROOT, m_order, m_sched, sendbuff, recvbuff, stream_of(ctx), \
                  current_device()};                                                        \
        return m_group->collective(m_rank, call);                                           \
    } while (0)

Status VRankCommunicator::scatter(const void* sendbuff, void* recvbuff, size_t recvlen, DType dtype, uint32_t root,
                                  std::shared_ptr<Context> ctx) {
    get_dtype_size(dtype);  // throws "unknown dtype" on this rank's own thread
    MEGRAY_ASSERT(root < m_nranks, "root %u out of range", root);
    VRANK_COLLECTIVE(Kind::kScatter, recvlen, dtype, MEGRAY_SUM, root);
}

Status VRankCommunicator::gather(const void* sendbuff, void* recvbuff, size_t sendlen, DType dtype, uint32_t root,
                                 std::shared_ptr<Context> ctx) {
    get_dtype_size(dtype);
    MEGRAY_ASSERT(root < m_nranks, "root %u out of range", root);
    VRANK_COLLECTIVE(Kind::kGather, sendlen, dtype, MEGRAY_SUM, root);
}

Status VRankCommunicator::all_to_all(const void* sendbuff, void* recvbuff, size_t len, DType dtype,
                                     std::shared_ptr<Context> ctx) {
    get_dtype_size(dtype);
    VRANK_COLLECTIVE(Kind::kAllToAll, len, dtype, MEGRAY_SUM, 0);
}

Status VRankCommunicator::all_gather(const void* sendbuff, void* recvbuff, size_t sendlen, DType dtype,
                                     std::shared_ptr<Context> ctx) {
    get_dtype_size(dtype);
    VRANK_COLLECTIVE(Kind::kAllGather, sendlen, dtype, MEGRAY_SUM, 0);
}

Status VRankCommunicator::all_reduce(const void* sendbuff, void* recvbuff, size_t len, DType dtype, ReduceOp op,
                                     std::shared_ptr<Context> ctx) {
    reduce_elem_size(dtype);  // "unknown dtype", src/ucx/kernel.cu:95-96
    check_reduce_op(op);      // "unknown reduce op", src/ucx/kernel.cu:55-56
    VRANK_COLLECTIVE(Kind::kAllReduce, len, dtype, op, 0);
}

Status VRankCommunicator::reduce_scatter(const void* sendbuff, void* recvbuff, size_t recvlen, DType dtype,
                                         ReduceOp op, std::shared_ptr<Context> ctx) {
    reduce_elem_size(dtype);
    check_reduce_op(op);
    VRANK_COLLECTIVE(Kind::kReduceScatter, recvlen, dtype, op, 0);
}

Status VRankCommunicator::broadcast(const void* sendbuff, void* recvbuff, size_t len, DType dtype, uint32_t root,
                                    std::shared_ptr<Context> ctx) {
    get_dtype_size(dtype);
    MEGRAY_ASSERT(root < m_nranks, "root %u out of range", root);
    VRANK_COLLECTIVE(Kind::kBroadcast, len, dtype, MEGRAY_SUM, root);
}

Status VRankCommunicator::reduce(const void* sendbuff, void* recvbuff, size_t len, DType dtype, ReduceOp op,
                                 uint32_t root, std::shared_ptr<Context> ctx) {
    reduce_elem_size(dtype);
    check_reduce_op(op);
    MEGRAY_ASSERT(root < m_nranks, "root %u out of range", root);
    if (m_rank != root) recvbuff = nullptr;  // only the root's pointer means anything (test/test_opr.cpp:501-505)
    VRANK_COLLECTIVE(Kind::kReduce, len, dtype, op, root);
}

// Between group_start() and group_end() sends and receives are only collected; group_end() posts
// them all and then waits for all, so that two ranks may each send to the other first.
Status VRankCommunicator::group_start() {
    m_grouping = true;
    return MEGRAY_OK;
}

Status VRankCommunicator::group_end() {
    m_grouping = false;
    Status result = MEGRAY_OK;
    for (auto& op : m_pending) {
        Status st = m_group->wait(op);
        if (st != MEGRAY_OK) result = st;
    }
    m_pending.clear();
    return result;
}

Status VRankCommunicator::p2p(bool is_send, const void* sendbuff, void* recvbuff, size_t size, uint32_t peer,
                              std::shared_ptr<Context> ctx) {
    MEGRAY_ASSERT(m_group != nullptr, "communicator used before init()");
    MEGRAY_ASSERT(peer < m_nranks && peer != m_rank, "invalid peer rank %u", peer);
    auto op = std::make_shared<PendingP2P>(
            PendingP2P{is_send, sendbuff, recvbuff, size, stream_of(ctx), current_device(), false, MEGRAY_OK});
    if (is_send) {
        m_group->post(m_rank, peer, op);
    } else {
        m_group->post(peer, m_rank, op);
    }
    if (m_grouping) {
        m_pending.push_back(op);
        return MEGRAY_OK;
    }
    return m_group->wait(op);
}

Status VRankCommunicator::_send(const void* sendbuff, size_t size, uint32_t rank, std::shared_ptr<Context> ctx) {
    return p2p(true, sendbuff, nullptr, size, rank, ctx);
}

Status VRankCommunicator::_recv(void* recvbuf, size_t size, uint32_t rank, std::shared_ptr<Context> ctx) {
    return p2p(false, nullptr, recvbuf, size, rank, ctx);
}

}  // namespace MegRay
