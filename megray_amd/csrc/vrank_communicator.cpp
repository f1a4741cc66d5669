#include "vrank_communicator.h"

#include <atomic>
#include <cstdlib>
#include <cstring>
#include <chrono>
#include <condition_variable>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <random>

#include <unistd.h>

#include "megray/hip_context.h"
#include "vrank_edges.h"
#include "vrank_engine.h"
#include "vrank_kernels.h"

namespace MegRay {
namespace vrank {

namespace {

// What one rank brings to a collective.
struct Call {
    int kind;  // CollectiveKind
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
    bool marked = false;    // the rank put a mark on its stream: everything enqueued before the call precedes it
    bool poisoned = false;  // the rank's own arguments were rejected; it does not take part
    bool fixed = false;     // allocation-free call: the edge counters are a block of the library's static device array
};

bool same_collective(const Call& a, const Call& b) {
    return a.kind == b.kind && a.len == b.len && a.dtype == b.dtype && a.op == b.op && a.root == b.root &&
           a.order == b.order && a.sched == b.sched && a.device == b.device && a.fixed == b.fixed;
}

// Slots of the static counter array, handed out process-wide (a group keeps its slot while it lives).
std::mutex g_slot_mutex;
bool g_slot_taken[kStaticEdgeSlots] = {};

int take_static_slot() {
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    for (uint32_t i = 0; i < kStaticEdgeSlots; ++i) {
        if (!g_slot_taken[i]) {
            g_slot_taken[i] = true;
            return int(i);
        }
    }
    return -1;
}

void give_back_static_slot(int slot) {
    std::lock_guard<std::mutex> lock(g_slot_mutex);
    if (slot >= 0) g_slot_taken[slot] = false;
}

// A planned collective kept for the next call with the same arguments and buffers: training loops
// and benchmarks repeat their collectives, and planning costs more than the launch itself.
struct CachedPlan {
    Call key;
    const void* send[kMaxRanks];
    void* recv[kMaxRanks];
    uint64_t signature;  // plan_signature() of the three above: compared first
    uint64_t last_used;  // the group's collective count when the plan was last launched
    Plan plan;
    std::vector<KernelCall> calls;  // point into `plan`
};

// A 64-bit mix of what identifies a planned collective, so that a look-up among many plans compares
// one word per plan before it compares arguments and addresses.
uint64_t plan_signature(const Call& c, const void* const* send, void* const* recv) {
    uint64_t h = 0x9e3779b97f4a7c15ull;
    const auto mix = [&h](uint64_t v) {
        h ^= v + 0x9e3779b97f4a7c15ull + (h << 6) + (h >> 2);
        h *= 0xff51afd7ed558ccdull;
        h ^= h >> 32;
    };
    mix(uint64_t(c.kind) | uint64_t(c.dtype) << 8 | uint64_t(c.op) << 16 | uint64_t(c.root) << 24 |
        uint64_t(c.order) << 32 | uint64_t(c.sched) << 40 | uint64_t(c.fixed) << 48);
    mix(c.len);
    for (uint32_t r = 0; r < kMaxRanks; ++r) {
        mix(reinterpret_cast<uintptr_t>(send[r]));
        mix(reinterpret_cast<uintptr_t>(recv[r]));
    }
    return h;
}

// The same for the copy of a point-to-point transfer.
struct CachedCopy {
    const void* src;
    void* dst;
    size_t size;
    Plan plan;
    std::vector<KernelCall> calls;  // point into `plan`
};

// Zeroes counters in device memory and returns when they ARE zero.  (hipMemset on device memory may return before
// the fill has run, and streams created non-blocking are not ordered behind the null stream it runs on: a rank's
// first arrive kernel could otherwise be wiped out by the clear that was meant to precede it.)
hipError_t clear_words(void* words, size_t bytes) {
    hipError_t err = hipMemsetAsync(words, 0, bytes, nullptr);
    if (err == hipSuccess) err = hipStreamSynchronize(nullptr);
    return err;
}

uint64_t env_u64(const char* name, uint64_t fallback) {
    const char* text = std::getenv(name);
    if (!text || !*text) return fallback;
    char* end = nullptr;
    const unsigned long long v = std::strtoull(text, &end, 10);
    return end == text ? fallback : uint64_t(v);
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
            : m_nranks(nranks), m_slots(nranks), m_entered(nranks, 0), m_arrive(nranks, nullptr),
              m_mail(size_t(nranks) * nranks) {}

    ~Group() {
        // The counters belong to the device the group worked on, which need not be the one current in the thread
        // that lets go of the last rank object (a finaliser thread, interpreter shutdown): switch to it for the
        // synchronisation and the frees, and back afterwards.
        int before = -1;
        const bool switched = m_device >= 0 && hipGetDevice(&before) == hipSuccess && before != m_device &&
                              hipSetDevice(m_device) == hipSuccess;
        bool drained = true;
        // wait kernels of the last collectives may still be polling the counters
        if (m_edges[0].words || m_edges[1].words) drained = hipDeviceSynchronize() == hipSuccess;
        if (drained && m_edges[1].words && !m_dead.load(std::memory_order_relaxed)) {
            uint64_t timeouts = 0, at = 0;
            if (edge_read_timeouts(m_edges[1].words, nullptr, &timeouts, &at) == hipSuccess && timeouts)
                MEGRAY_ERROR("a communicator group is torn down whose stream waits gave up (%llu of them, the first "
                             "waiting for %llu): results after that point were not written",
                             static_cast<unsigned long long>(timeouts), static_cast<unsigned long long>(at));
        }
        for (hipEvent_t ev : m_events) (void)hipEventDestroy(ev);
        for (hipEvent_t ev : m_arrive)
            if (ev) (void)hipEventDestroy(ev);
        if (m_done) (void)hipEventDestroy(m_done);
        if (m_edges[0].words) (void)hipFree(m_edges[0].words);
        if (m_p2p_words) (void)hipFree(m_p2p_words);
        if (m_edges[0].status) (void)hipHostFree(m_edges[0].status);
        // a block some kernel may still be polling is not handed to another group
        if (drained) give_back_static_slot(m_fixed_slot);
        (void)hipGetLastError();
        if (switched) (void)hipSetDevice(before);
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
    // to arrive enqueues the collective for all.  Every rank returns the same Status (and finds the
    // same text in plan_error()).
    Status collective(uint32_t rank, const Call& in_call) {
        Call call = in_call;
        await_release(rank);
        // Every rank marks, on its own stream and from its own thread, the point its buffers are
        // ready at; the marks are enqueued in parallel instead of one after the other by the leader.
        // No mark is needed from a rank whose stream is the one every rank shared last time (if all
        // share a stream again no cross-stream edge exists; if not, the leader marks it on the rank's
        // behalf, the rank being parked here) or from the rank that sees all others arrived already (it
        // is going to launch on its own stream).  (Asking the runtime whether a stream is idle, to
        // skip the mark, costs as much as the mark itself when the stream is busy.)
        const bool shared = m_shared_valid.load(std::memory_order_acquire) &&
                            m_shared_stream.load(std::memory_order_relaxed) == static_cast<void*>(call.stream);
        const bool last = m_arrived.load(std::memory_order_acquire) == m_nranks - 1;
        if (!shared && !last) {
            const Status st = mark(rank, call.stream, call.fixed);
            if (st != MEGRAY_OK)
                return withdraw(rank, call.fixed && !m_edges[1].words ? m_fixed_error : "a stream mark could not be enqueued", st);
            call.marked = true;
        }
        return arrive(rank, call, true);
    }

    // A rank whose own arguments were rejected tells the group and leaves at once (its caller gets
    // the exception); the other ranks' calls come back with MEGRAY_INVALID_USAGE instead of waiting
    // for a rank that will never arrive.
    void poison(uint32_t rank, const char* why) {
        // still counted as withdrawn from a collective the other ranks have not finished: nothing to add
        if (m_generation.load(std::memory_order_acquire) < m_entered[rank]) return;
        (void)withdraw(rank, why, MEGRAY_INVALID_USAGE);
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
        Status st = check_alive(m_edges[0], r.stream);
        if (st == MEGRAY_OK) st = transfer(s, r, size_t(src_rank) * m_nranks + dst_rank);
        s.status = r.status = st;
        s.done = r.done = true;
        m_cv.notify_all();
    }

    Status wait(const std::shared_ptr<PendingP2P>& op) {
        std::unique_lock<std::mutex> lock(m_mutex);
        m_cv.wait(lock, [&] { return op->done; });
        return op->status;
    }

    void stats(uint64_t out[3]) const {
        out[0] = m_stat_collectives.load(std::memory_order_relaxed);
        out[1] = m_stat_plans.load(std::memory_order_relaxed);
        out[2] = m_stat_sleeps.load(std::memory_order_relaxed);
    }

    // Reads the counters back now (after `stream` has drained): has any stream wait of the group given up?
    Status check(hipStream_t stream) {
        for (EdgeSet& set : m_edges) {
            if (m_dead.load(std::memory_order_acquire) || !set.words) continue;
            uint64_t gave_up = 0, at = 0;
            HIP_CHECK(edge_read_timeouts(set.words, stream, &gave_up, &at));
            if (gave_up) declare_dead(at);
        }
        if (!m_dead.load(std::memory_order_acquire)) return MEGRAY_OK;
        set_plan_error(m_dead_text);
        return MEGRAY_UNEXPECTED_ERR;
    }

private:
    // Counters of the edge kernels.  [0]: allocated at the first collective (null: the events below are
    // used instead).  [1]: a block of the library's static device array, for the allocation-free entry point.
    struct EdgeSet {
        EdgeWords* words = nullptr;
        uint64_t* status = nullptr;  // pinned host memory: [0] waits that gave up, [1] what the last one waited for
        std::atomic<uint64_t> marks{0};  // arrive kernels enqueued so far = value `arrived` reaches when all have run
    };
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

    // A rank that left a collective early (poison) comes back only when that collective is over.
    void await_release(uint32_t rank) {
        const uint64_t need = m_entered[rank];
        if (m_generation.load(std::memory_order_acquire) >= need) return;
        sleep_until_past(need);
    }

    Status withdraw(uint32_t rank, const char* why, Status st) {
        Call call{};
        call.poisoned = true;
        char text[200];
        std::snprintf(text, sizeof(text), "rank %u left the collective: %s", rank, why ? why : "");
        {
            std::lock_guard<std::mutex> lock(m_poison_mutex);
            if (!m_poison_text[0]) std::snprintf(m_poison_text, sizeof(m_poison_text), "%s", text);
        }
        (void)arrive(rank, call, false);
        set_plan_error(text);
        return st;
    }

    // Deposit and, for the last rank, launch; `park`: wait for the release and order the own stream
    // behind the result.  Arrival is one atomic increment (eight threads meeting at a mutex spend
    // more time in its wait queue than the launch takes); the rank whose increment completes the
    // count reads every slot and launches, the others poll the generation.
    Status arrive(uint32_t rank, const Call& call, bool park) {
        m_slots[rank].call = call;
        if (call.marked) m_edges[call.fixed].marks.fetch_add(1, std::memory_order_relaxed);
        const uint64_t gen = m_generation.load(std::memory_order_relaxed);  // cannot move on before this rank arrives
        m_entered[rank] = gen + 1;
        if (m_arrived.fetch_add(1, std::memory_order_acq_rel) + 1 == m_nranks) {
            Status st;
            try {
                st = launch(rank);
            } catch (const MegRay::Exception& e) {
                set_plan_error(e.what());
                st = MEGRAY_INVALID_ARGUMENT;
            } catch (const std::exception& e) {
                set_plan_error(e.what());
                st = MEGRAY_UNEXPECTED_ERR;
            } catch (...) {
                set_plan_error("unknown failure while launching the collective");
                st = MEGRAY_UNEXPECTED_ERR;
            }
            if (st != MEGRAY_OK) {
                MEGRAY_ERROR("collective failed: %s", plan_error());
                std::snprintf(m_error[gen & 1], sizeof(m_error[0]), "%s", plan_error());
            }
            m_result[gen & 1] = st;
            m_lead_stream[gen & 1] = call.stream;
            {
                std::lock_guard<std::mutex> lock(m_poison_mutex);
                m_poison_text[0] = 0;
            }
            m_arrived.store(0, std::memory_order_relaxed);
            m_generation.store(gen + 1, std::memory_order_seq_cst);
            if (m_sleepers.load(std::memory_order_seq_cst)) {
                { std::lock_guard<std::mutex> lock(m_mutex); }  // a sleeper is either waiting or has not yet checked
                m_cv.notify_all();
            }
            return st;
        }
        if (!park) return MEGRAY_OK;
        // The other ranks are usually a few microseconds away: poll the generation for a while before
        // going to sleep on the condition variable (a sleeping thread costs tens of microseconds to wake).
        bool released = false;
        for (int spin = 0; spin < kSpinPolls && !released; ++spin) {
            released = m_generation.load(std::memory_order_acquire) != gen;
            if (!released) __builtin_ia32_pause();
        }
        if (!released) sleep_until_past(gen + 1);
        // ... and orders its own stream behind the result.  The done mark is not set again before
        // every rank has passed this point: the next collective needs all of them to arrive first.
        const Status st = m_result[gen & 1];
        if (st != MEGRAY_OK) {
            set_plan_error(m_error[gen & 1]);
            return st;
        }
        if (call.stream != m_lead_stream[gen & 1]) MEGRAY_CHECK(await_done(call.stream, gen + 1, call.fixed));
        return st;
    }

    void sleep_until_past(uint64_t need) {
        m_stat_sleeps.fetch_add(1, std::memory_order_relaxed);
        std::unique_lock<std::mutex> lock(m_mutex);
        m_sleepers.fetch_add(1, std::memory_order_seq_cst);
        m_cv.wait(lock, [&] { return m_generation.load(std::memory_order_seq_cst) >= need; });
        m_sleepers.fetch_sub(1, std::memory_order_seq_cst);
    }

    // Cross-stream ordering, "stream B goes on after what stream A holds now", is a mark on A and a
    // wait on B.  Default: the one-wavefront kernels of vrank_edges.h on counters in device memory
    // (kernel launches from several threads run in parallel in the runtime; its stream memory
    // operations and event calls are serialised across threads and cost 3 - 5 times as much on
    // MI355X).  MEGRAY_VRANK_EDGES=events in the environment keeps to event record / stream-wait-event,
    // which is also the fallback when the counters cannot be allocated.
    bool wait_limit() {
        int device = 0, khz = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device) != hipSuccess || khz <= 0) {
            (void)hipGetLastError();
            return false;
        }
        // a wait gives up after this long (wall-clock ticks): long enough for any stream to drain,
        // short enough that a lost mark does not hold a wavefront for ever
        const uint64_t ms = env_u64("MEGRAY_VRANK_WAIT_LIMIT_MS", 10000);
        m_limit_ms.store(ms, std::memory_order_relaxed);
        m_limit_ticks = ms * uint64_t(khz);
        return true;
    }

    void prepare_edges() {
        std::call_once(m_edges_once, [&] {
            const char* choice = std::getenv("MEGRAY_VRANK_EDGES");
            if (choice && std::strcmp(choice, "events") == 0) return;
            EdgeWords* words = nullptr;
            uint64_t* status = nullptr;
            bool ok = wait_limit();
            ok = ok && hipMalloc(reinterpret_cast<void**>(&words), sizeof(EdgeWords)) == hipSuccess;
            ok = ok && clear_words(words, sizeof(EdgeWords)) == hipSuccess;
            ok = ok && hipHostMalloc(reinterpret_cast<void**>(&status), 2 * sizeof(uint64_t), hipHostMallocDefault) == hipSuccess;
            if (!ok) {
                (void)hipGetLastError();
                if (words) (void)hipFree(words);
                if (status) (void)hipHostFree(status);
                return;
            }
            status[0] = status[1] = 0;
            (void)hipGetDevice(&m_device);
            m_edges[0].status = status;
            m_edges[0].words = words;
        });
    }

    // The counters of the allocation-free entry point: a block of the library's static device array,
    // cleared once when the group takes it (a block keeps what its last user left).  Nothing is allocated.
    void prepare_fixed_edges() {
        std::call_once(m_fixed_once, [&] {
            if (!wait_limit()) {
                m_fixed_error = "the device's wall clock rate is unknown";
                return;
            }
            m_fixed_slot = take_static_slot();
            if (m_fixed_slot < 0) {
                m_fixed_error = "every counter block of the static array is in use (32 communicator groups at a time)";
                return;
            }
            EdgeWords* words = nullptr;
            if (edge_static_words(uint32_t(m_fixed_slot), &words) != hipSuccess ||
                clear_words(words, sizeof(EdgeWords)) != hipSuccess) {
                (void)hipGetLastError();
                m_fixed_error = "the static counter array could not be reached on this device";
                return;
            }
            (void)hipGetDevice(&m_device);
            m_fixed_checked = std::chrono::steady_clock::now();
            m_fixed_period = std::chrono::milliseconds(m_limit_ms.load(std::memory_order_relaxed) / 2);
            m_edges[1].words = words;
        });
    }

    Status mark(uint32_t rank, hipStream_t stream, bool fixed) {
        if (fixed) {
            prepare_fixed_edges();
            if (!m_edges[1].words) {
                MEGRAY_ERROR("allocation-free collective: %s", m_fixed_error);
                return MEGRAY_INVALID_USAGE;
            }
        } else {
            prepare_edges();
        }
        if (m_edges[fixed].words) {
            HIP_CHECK(edge_arrive(m_edges[fixed].words, stream));
            return MEGRAY_OK;
        }
        hipEvent_t& ev = m_arrive[rank];
        if (!ev) HIP_CHECK(hipEventCreateWithFlags(&ev, hipEventDisableTiming));
        HIP_CHECK(hipEventRecord(ev, stream));
        return MEGRAY_OK;
    }

    Status await_done(hipStream_t stream, uint64_t ticket, bool fixed) {
        const EdgeSet& set = m_edges[fixed];
        if (set.words) {
            HIP_CHECK(edge_wait_done(set.words, set.words, ticket, m_limit_ticks, set.status, stream));
            return MEGRAY_OK;
        }
        HIP_CHECK(hipStreamWaitEvent(stream, m_done, 0));
        return MEGRAY_OK;
    }

    CachedPlan* lookup(const Call& lead, const void* const* send, void* const* recv, uint64_t signature) {
        for (auto& cp : m_plans) {
            if (cp->signature == signature && same_collective(cp->key, lead) &&
                std::memcmp(cp->send, send, sizeof(cp->send)) == 0 && std::memcmp(cp->recv, recv, sizeof(cp->recv)) == 0)
                return cp.get();
        }
        return nullptr;
    }

    // Where a launch keeps its stream-ordering fields, if it is one that may carry them: one wavefront
    // per workgroup and fewer than kHookMaxTiles workgroups.
    struct HookFields {
        EdgeHooks* hooks;
        uint64_t* target;
        uint64_t* ticket;
    };
    static bool hook_fields(Step& step, HookFields& f) {
        // MEGRAY_VRANK_HOOK_MAX_TILES in the environment moves the border (0: no launch carries the ordering)
        static const uint64_t kHookMaxTiles = env_u64("MEGRAY_VRANK_HOOK_MAX_TILES", vrank::kHookMaxTiles);
        switch (step.kind) {
            case Step::kFlat:
                if (step.flat.waves != 1 || step.flat.total_tiles >= kHookMaxTiles) return false;
                f = {&step.flat.hooks, &step.flat.hook_target, &step.flat.hook_ticket};
                return true;
            case Step::kFold:
                if (step.fold.waves != 1 || step.fold.total_tiles >= kHookMaxTiles) return false;
                f = {&step.fold.hooks, &step.fold.hook_target, &step.fold.hook_ticket};
                return true;
            case Step::kTree:
                if (step.tree.total_tiles >= kHookMaxTiles) return false;
                f = {&step.tree.hooks, &step.tree.hook_target, &step.tree.hook_ticket};
                return true;
            case Step::kPack:
                if (step.pack.waves != 1 || uint64_t(step.pack.ncopies) * step.pack.tiles_per_copy >= kHookMaxTiles) return false;
                f = {&step.pack.hooks, &step.pack.hook_target, &step.pack.hook_ticket};
                return true;
        }
        return false;
    }

    // Tells a launch where the group's poison is (EdgeHooks::words; the wait / publish fields stay as they are).
    void guard(Step& step, const EdgeSet& set) {
        const EdgeHooks hooks{reinterpret_cast<uint64_t*>(set.words), set.status, m_limit_ticks};
        switch (step.kind) {
            case Step::kFlat:
                step.flat.hooks = hooks;
                step.flat.exchange = set.words ? step.flat.exchange | kFlatGuarded : step.flat.exchange & ~kFlatGuarded;
                break;
            case Step::kFold: step.fold.hooks = hooks; break;
            case Step::kTree: step.tree.hooks = hooks; break;
            case Step::kPack: step.pack.hooks = hooks; break;
        }
    }

    // A stream wait of the group that gave up poisons the group for good: the kernels behind it store nothing
    // (they test the poison in device memory), and from the moment the host knows, every call of the group -
    // collective or transfer, on every rank - fails with MEGRAY_UNEXPECTED_ERR.  The host knows through the two
    // words of pinned memory the waits report to; a group that only ever used the allocation-free entry point has
    // none, and reads the poison back from its counter block instead: a wait cannot give up sooner than the limit
    // after it was enqueued, so the block is read (a synchronous copy behind `stream`, not under stream capture)
    // when half the limit has passed since the last read, and when the group is torn down.
    Status check_alive(EdgeSet& set, hipStream_t stream) {
        if (!m_dead.load(std::memory_order_acquire)) {
            uint64_t gave_up = 0, at = 0;
            if (set.status) {
                gave_up = __atomic_load_n(&set.status[0], __ATOMIC_ACQUIRE);
                at = set.status[1];
            } else if (&set == &m_edges[1] && set.words && m_limit_ticks) {
                const auto now = std::chrono::steady_clock::now();
                if (now - m_fixed_checked >= m_fixed_period) {
                    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
                    if (hipStreamIsCapturing(stream, &capturing) != hipSuccess) (void)hipGetLastError();
                    if (capturing == hipStreamCaptureStatusNone) {
                        m_fixed_checked = now;
                        HIP_CHECK(edge_read_timeouts(set.words, stream, &gave_up, &at));
                    }
                }
            }
            if (!gave_up) return MEGRAY_OK;
            declare_dead(at);
        }
        set_plan_error(m_dead_text);
        return MEGRAY_UNEXPECTED_ERR;
    }

    void declare_dead(uint64_t at) {
        std::lock_guard<std::mutex> lock(m_poison_mutex);
        if (m_dead.load(std::memory_order_relaxed)) return;
        std::snprintf(m_dead_text, sizeof(m_dead_text),
                      "a stream wait of this group gave up after %llu ms (it was waiting for count / ticket %llu: a "
                      "rank's stream did not get there in time); what followed it was not written, and the group "
                      "takes no further calls",
                      static_cast<unsigned long long>(m_limit_ms.load(std::memory_order_relaxed)),
                      static_cast<unsigned long long>(at));
        m_dead.store(true, std::memory_order_release);
    }

    // Called by the last rank to arrive; every other rank is parked or has withdrawn.
    Status launch(uint32_t leader) {
        {
            std::lock_guard<std::mutex> lock(m_poison_mutex);
            if (m_poison_text[0]) {
                set_plan_error(m_poison_text);
                return MEGRAY_INVALID_USAGE;
            }
        }
        const Call& lead = m_slots[leader].call;
        for (uint32_t r = 0; r < m_nranks; ++r) {
            if (!same_collective(lead, m_slots[r].call)) {
                char text[160];
                std::snprintf(text, sizeof(text),
                              "rank %u and rank %u called different collectives (or with different arguments)", leader, r);
                set_plan_error(text);
                return MEGRAY_INVALID_USAGE;
            }
        }
        EdgeSet& set = m_edges[lead.fixed];
        MEGRAY_CHECK(check_alive(set, lead.stream));
        const void* send[kMaxRanks] = {};
        void* recv[kMaxRanks] = {};
        for (uint32_t r = 0; r < m_nranks; ++r) {
            send[r] = m_slots[r].call.send;
            recv[r] = m_slots[r].call.recv;
        }
        // plan first: a rejected call must not leave marks or waits behind
        const uint64_t signature = plan_signature(lead, send, recv);
        CachedPlan* cp = lookup(lead, send, recv, signature);
        m_stat_collectives.fetch_add(1, std::memory_order_relaxed);
        if (!cp) {
            m_stat_plans.fetch_add(1, std::memory_order_relaxed);
            auto fresh = std::make_unique<CachedPlan>();
            fresh->key = lead;
            fresh->signature = signature;
            std::memcpy(fresh->send, send, sizeof(send));
            std::memcpy(fresh->recv, recv, sizeof(recv));
            Status st = plan_collective(fresh->plan, lead.kind, send, recv, m_nranks, lead.len, lead.dtype, lead.order,
                                        lead.sched, lead.root);
            if (st == MEGRAY_OK) st = resolve(fresh->plan, lead.dtype, is_reduction(lead.kind) ? lead.op : MEGRAY_SUM, fresh->calls);
            if (st != MEGRAY_OK) return st;
            if (m_plans.size() < kPlanSlots) {
                m_plans.push_back(std::move(fresh));
                cp = m_plans.back().get();
            } else {
                // the plan that has gone unused for longest makes room
                size_t oldest = 0;
                for (size_t i = 1; i < m_plans.size(); ++i)
                    if (m_plans[i]->last_used < m_plans[oldest]->last_used) oldest = i;
                m_plans[oldest] = std::move(fresh);
                cp = m_plans[oldest].get();
            }
        }
        cp->last_used = ++m_plan_clock;
        // order the leader's stream behind everything already enqueued on the other ranks' streams
        hipStream_t stream = lead.stream;
        bool one_stream = true, wait_needed = false;
        for (uint32_t r = 0; r < m_nranks; ++r) {
            const Call& other = m_slots[r].call;
            if (other.stream == stream) continue;
            one_stream = false;
            // a rank that expected everyone on its stream did not mark it; it is parked in arrive(),
            // so its stream's tail is still the point it arrived at
            if (!other.marked) {
                MEGRAY_CHECK(mark(r, other.stream, lead.fixed));
                set.marks.fetch_add(1, std::memory_order_relaxed);
            }
            wait_needed = true;
            if (!set.words) HIP_CHECK(hipStreamWaitEvent(stream, m_arrive[r], 0));
        }
        m_shared_stream.store(static_cast<void*>(stream), std::memory_order_relaxed);
        m_shared_valid.store(one_stream, std::memory_order_release);
        const uint64_t ticket = m_generation.load(std::memory_order_relaxed) + 1;
        // every launch of the group knows where the group's poison is (null while the group has no counters:
        // without them nothing ever waits)
        for (Step& step : cp->plan.steps) guard(step, set);
        // A single short launch of one wavefront per workgroup waits for the marks and publishes its
        // completion itself: two launches less on this thread, on which every rank is waiting.
        // (Only short launches: one of many tiles must not wait inside the kernel - workgroups that hold a
        // whole CU's LDS would spin on streams that may need that CU - and announcing completion costs
        // an L2 write-back per workgroup.  Those get a wait kernel before and a notify kernel after.)
        HookFields hooked;
        const bool hook = set.words && !one_stream && cp->plan.steps.size() == 1 && hook_fields(cp->plan.steps[0], hooked);
        if (hook) {
            *hooked.target = wait_needed ? set.marks.load(std::memory_order_relaxed) : 0;
            *hooked.ticket = ticket;
        } else if (wait_needed && set.words) {
            HIP_CHECK(edge_wait_arrived(set.words, set.words, set.marks.load(std::memory_order_relaxed), m_limit_ticks, set.status, stream));
        }
        for (const KernelCall& call : cp->calls) HIP_CHECK(enqueue(call.kernel, call.grid, call.block, call.launch, stream, call.lds));
        // the other ranks order their streams behind this point themselves (none has to if all share the stream)
        if (hook) {
            *hooked.target = *hooked.ticket = 0;
        } else if (!one_stream) {
            if (set.words) {
                HIP_CHECK(edge_notify(set.words, set.words, ticket, stream));
            } else {
                if (!m_done) HIP_CHECK(hipEventCreateWithFlags(&m_done, hipEventDisableTiming));
                HIP_CHECK(hipEventRecord(m_done, stream));
            }
        }
        return MEGRAY_OK;
    }

    // Counters for point-to-point transfers between ranks on different streams: two blocks per (source,
    // destination) pair, "the sender's stream has reached the send" and "the copy is done", each holding
    // the number of the pair's last transfer that got there.  Allocated at the first such transfer.
    void prepare_p2p_edges() {
        std::call_once(m_p2p_once, [&] {
            prepare_edges();
            if (!m_edges[0].words) return;  // events are in use (by choice, or the counters could not be allocated)
            const size_t bytes = sizeof(EdgeWords) * 2 * m_mail.size();
            EdgeWords* words = nullptr;
            if (hipMalloc(reinterpret_cast<void**>(&words), bytes) != hipSuccess ||
                clear_words(words, bytes) != hipSuccess) {
                (void)hipGetLastError();
                if (words) (void)hipFree(words);
                return;
            }
            m_p2p_seq.assign(m_mail.size(), 0);
            m_p2p_words = words;
        });
    }

    // The copy itself: the library's own block copy (16 bytes per lane at any alignment), planned once per
    // (source, destination, size) and kept for the next transfer between the same buffers; buffers the
    // planner does not take (partly overlapping ones) go to the runtime's copy.  Called with m_mutex held.
    Status copy_bytes(void* dst, const void* src, size_t size, hipStream_t stream) {
        CachedCopy* cc = nullptr;
        for (auto& c : m_copies)
            if (c->src == src && c->dst == dst && c->size == size) cc = c.get();
        if (!cc) {
            auto fresh = std::make_unique<CachedCopy>();
            fresh->src = src;
            fresh->dst = dst;
            fresh->size = size;
            void* const recv[1] = {dst};
            Status st = plan_broadcast(fresh->plan, src, recv, 1, size, 1, 0);
            if (st == MEGRAY_OK) st = resolve(fresh->plan, MEGRAY_UINT8, MEGRAY_SUM, fresh->calls);
            if (st != MEGRAY_OK) {
                set_plan_error("");
                HIP_CHECK(hipMemcpyAsync(dst, src, size, hipMemcpyDeviceToDevice, stream));
                return MEGRAY_OK;
            }
            if (m_copies.size() < kCopySlots) {
                m_copies.push_back(std::move(fresh));
                cc = m_copies.back().get();
            } else {
                m_copies[m_copy_next] = std::move(fresh);
                cc = m_copies[m_copy_next].get();
                m_copy_next = (m_copy_next + 1) % kCopySlots;
            }
        }
        for (Step& step : cc->plan.steps) guard(step, m_edges[0]);
        for (const KernelCall& call : cc->calls) HIP_CHECK(enqueue(call.kernel, call.grid, call.block, call.launch, stream, call.lds));
        return MEGRAY_OK;
    }

    // Enqueue the copy of a matched send / receive pair: on the receiver's stream, after the
    // sender's stream has reached the send, and before the sender's stream goes on.  Between two
    // streams the order is kept by notify / wait kernels on the pair's counters (every wait is
    // enqueued after the kernel that satisfies it), or by events where the counters are not in use.
    // Called with m_mutex held, so a pair's transfers are numbered in the order they are enqueued.
    Status transfer(const PendingP2P& s, const PendingP2P& r, size_t pair) {
        if (s.size != r.size || s.device != r.device) {
            MEGRAY_ERROR("send of %zu bytes met a receive of %zu bytes", s.size, r.size);
            return MEGRAY_INVALID_USAGE;
        }
        if (!s.size) return MEGRAY_OK;
        if (s.stream == r.stream) return copy_bytes(r.dst, s.src, s.size, r.stream);
        prepare_p2p_edges();
        if (m_p2p_words) {
            EdgeWords* reached = m_p2p_words + 2 * pair;
            EdgeWords* copied = reached + 1;
            const uint64_t ticket = ++m_p2p_seq[pair];
            uint64_t* status = m_edges[0].status;
            EdgeWords* group = m_edges[0].words;
            HIP_CHECK(edge_notify(reached, group, ticket, s.stream));
            HIP_CHECK(edge_wait_done(reached, group, ticket, m_limit_ticks, status, r.stream));
            MEGRAY_CHECK(copy_bytes(r.dst, s.src, s.size, r.stream));
            HIP_CHECK(edge_notify(copied, group, ticket, r.stream));
            HIP_CHECK(edge_wait_done(copied, group, ticket, m_limit_ticks, status, s.stream));
            return MEGRAY_OK;
        }
        HIP_CHECK(hipEventRecord(event(0), s.stream));
        HIP_CHECK(hipStreamWaitEvent(r.stream, event(0), 0));
        MEGRAY_CHECK(copy_bytes(r.dst, s.src, s.size, r.stream));
        HIP_CHECK(hipEventRecord(event(1), r.stream));
        HIP_CHECK(hipStreamWaitEvent(s.stream, event(1), 0));
        return MEGRAY_OK;
    }

    struct alignas(64) Slot {  // one cache line (or more) per rank: ranks deposit at the same time
        Call call;
    };
    const uint32_t m_nranks;
    std::mutex m_mutex;  // point-to-point mailboxes; sleeping waiters
    std::condition_variable m_cv;
    std::mutex m_poison_mutex;
    std::vector<Slot> m_slots;
    std::vector<uint64_t> m_entered;  // per rank: the generation count that ends the collective it last entered
    static constexpr int kSpinPolls = 20000;
    // Plans kept per group: a training step repeats the same few dozen collectives (one per gradient bucket) in the
    // same order, which a cache smaller than that set would miss every time.
    static constexpr size_t kPlanSlots = 64;
    static constexpr size_t kCopySlots = 16;
    Status m_result[2] = {MEGRAY_OK, MEGRAY_OK};
    char m_error[2][256] = {"", ""};  // text that goes with m_result
    char m_poison_text[200] = "";
    hipStream_t m_lead_stream[2] = {nullptr, nullptr};
    std::atomic<void*> m_shared_stream{nullptr};  // the stream of the last collective, ...
    std::atomic<bool> m_shared_valid{false};      // ... if every rank passed that same one
    std::once_flag m_edges_once;
    EdgeSet m_edges[2];
    std::once_flag m_fixed_once;
    int m_fixed_slot = -1;
    const char* m_fixed_error = "";
    std::atomic<uint64_t> m_limit_ticks{0};
    std::atomic<uint64_t> m_limit_ms{0};
    int m_device = -1;                  // the device the counters live on
    std::atomic<bool> m_dead{false};    // a stream wait gave up: the group takes no further calls
    char m_dead_text[320] = "";
    std::chrono::steady_clock::time_point m_fixed_checked{};  // when the static counter block was last read back
    std::chrono::steady_clock::duration m_fixed_period{};
    std::atomic<uint32_t> m_sleepers{0};
    std::atomic<uint64_t> m_stat_collectives{0}, m_stat_plans{0}, m_stat_sleeps{0};
    alignas(64) std::atomic<uint32_t> m_arrived{0};     // ranks that have deposited their call
    alignas(64) std::atomic<uint64_t> m_generation{0};  // collectives released so far; parked ranks poll it
    [[maybe_unused]] alignas(64) char m_pad[64] = {};  // keeps what follows off the polled line
    std::vector<hipEvent_t> m_arrive;  // per rank: "my buffers are ready", recorded by the rank itself
    hipEvent_t m_done = nullptr;       // recorded by the leader behind the collective
    std::vector<hipEvent_t> m_events;  // point-to-point transfers, where the counters below are not in use
    std::once_flag m_p2p_once;
    EdgeWords* m_p2p_words = nullptr;  // point-to-point transfers: two counter blocks per (source, destination)
    std::vector<uint64_t> m_p2p_seq;   // per (source, destination): transfers enqueued between two streams so far
    std::vector<Mailbox> m_mail;
    std::vector<std::unique_ptr<CachedPlan>> m_plans;
    uint64_t m_plan_clock = 0;
    std::vector<std::unique_ptr<CachedCopy>> m_copies;  // point-to-point transfers
    size_t m_copy_next = 0;
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

// The device the calling thread works on; -1 without one (the group then fails at its first launch,
// on every rank alike, instead of on this rank alone).
int current_device() {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) {
        (void)hipGetLastError();
        return -1;
    }
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

// Argument checks run on the calling rank's own thread and throw there, like the reference's; the
// group is told, so that the other ranks' calls come back instead of waiting for this one.
#define VRANK_COLLECTIVE(KIND, LEN, DTYPE, OP, ROOT, CHECKS) VRANK_COLLECTIVE_ON(false, KIND, LEN, DTYPE, OP, ROOT, CHECKS)
#define VRANK_COLLECTIVE_ON(FIXED, KIND, LEN, DTYPE, OP, ROOT, CHECKS)                          \
    do {                                                                                        \
        MEGRAY_ASSERT(m_group != nullptr, "communicator used before init()");                   \
        hipStream_t stream = nullptr;                                                           \
        try {                                                                                   \
            CHECKS;                                                                             \
            stream = stream_of(ctx);                                                            \
        } catch (const MegRay::Exception& e) {                                                  \
            m_group->poison(m_rank, e.what());                                                  \
            throw;                                                                              \
        }                                                                                       \
        Call call{KIND, LEN, DTYPE, OP, ROOT, m_order, m_sched, sendbuff, recvbuff, stream,     \
                  current_device()};                                                            \
        call.fixed = FIXED;                                                                     \
        return m_group->collective(m_rank, call);                                               \
    } while (0)

#define VRANK_ROOT_IN_RANGE MEGRAY_ASSERT(root < m_nranks, "root %u out of range", root)

Status VRankCommunicator::scatter(const void* sendbuff, void* recvbuff, size_t recvlen, DType dtype, uint32_t root,
                                  std::shared_ptr<Context> ctx) {
    // get_dtype_size throws "unknown dtype" (src/core/common.cpp:35-36)
    VRANK_COLLECTIVE(kCollScatter, recvlen, dtype, MEGRAY_SUM, root, get_dtype_size(dtype); VRANK_ROOT_IN_RANGE);
}

Status VRankCommunicator::gather(const void* sendbuff, void* recvbuff, size_t sendlen, DType dtype, uint32_t root,
                                 std::shared_ptr<Context> ctx) {
    VRANK_COLLECTIVE(kCollGather, sendlen, dtype, MEGRAY_SUM, root, get_dtype_size(dtype); VRANK_ROOT_IN_RANGE);
}

Status VRankCommunicator::all_to_all(const void* sendbuff, void* recvbuff, size_t len, DType dtype,
                                     std::shared_ptr<Context> ctx) {
    VRANK_COLLECTIVE(kCollAllToAll, len, dtype, MEGRAY_SUM, 0, get_dtype_size(dtype));
}

Status VRankCommunicator::all_gather(const void* sendbuff, void* recvbuff, size_t sendlen, DType dtype,
                                     std::shared_ptr<Context> ctx) {
    VRANK_COLLECTIVE(kCollAllGather, sendlen, dtype, MEGRAY_SUM, 0, get_dtype_size(dtype));
}

Status VRankCommunicator::all_reduce(const void* sendbuff, void* recvbuff, size_t len, DType dtype, ReduceOp op,
                                     std::shared_ptr<Context> ctx) {
    // "unknown dtype" and "unknown reduce op", src/ucx/kernel.cu:95-96 and :55-56
    VRANK_COLLECTIVE(kCollAllReduce, len, dtype, op, 0, reduce_elem_size(dtype); check_reduce_op(op));
}

Status VRankCommunicator::all_reduce_no_alloc(const void* sendbuff, void* recvbuff, size_t len, DType dtype,
                                              ReduceOp op, std::shared_ptr<Context> ctx) {
    VRANK_COLLECTIVE_ON(true, kCollAllReduce, len, dtype, op, 0, reduce_elem_size(dtype); check_reduce_op(op));
}

VRankCommunicator::Stats VRankCommunicator::stats() const {
    uint64_t v[3] = {0, 0, 0};
    if (m_group) m_group->stats(v);
    return {v[0], v[1], v[2]};
}

Status VRankCommunicator::check(std::shared_ptr<Context> ctx) {
    MEGRAY_ASSERT(m_group != nullptr, "communicator used before init()");
    return m_group->check(stream_of(ctx));
}

Status VRankCommunicator::reduce_scatter(const void* sendbuff, void* recvbuff, size_t recvlen, DType dtype,
                                         ReduceOp op, std::shared_ptr<Context> ctx) {
    VRANK_COLLECTIVE(kCollReduceScatter, recvlen, dtype, op, 0, reduce_elem_size(dtype); check_reduce_op(op));
}

Status VRankCommunicator::broadcast(const void* sendbuff, void* recvbuff, size_t len, DType dtype, uint32_t root,
                                    std::shared_ptr<Context> ctx) {
    VRANK_COLLECTIVE(kCollBroadcast, len, dtype, MEGRAY_SUM, root, get_dtype_size(dtype); VRANK_ROOT_IN_RANGE);
}

Status VRankCommunicator::reduce(const void* sendbuff, void* recvbuff, size_t len, DType dtype, ReduceOp op,
                                 uint32_t root, std::shared_ptr<Context> ctx) {
    if (m_rank != root) recvbuff = nullptr;  // only the root's pointer means anything (test/test_opr.cpp:501-505)
    VRANK_COLLECTIVE(kCollReduce, len, dtype, op, root, reduce_elem_size(dtype); check_reduce_op(op); VRANK_ROOT_IN_RANGE);
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
