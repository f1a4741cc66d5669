// The thread-per-rank communicator on SIMULATED streams, built with the thread sanitizer: no GPU.
//
// The host side of the backend (rendezvous of the rank threads, plan cache, cross-stream ordering by
// arrive / wait / notify kernels or by events, point-to-point matching) is compiled as it is; this file
// supplies what it calls below that line - the HIP runtime entry points it uses, the edge kernels and the
// kernel launcher - on streams that are queues worked off by one executor thread in a random order, so
// that the interleavings a GPU rarely shows turn up within seconds:
//
//   a stream      a FIFO of operations; the executor runs the operation at a stream's head when it is ready
//   a wait        an operation that is not ready until its counter has reached its target
//   a kernel      an operation that checks the ordering the collective promises and leaves its mark:
//                 every rank's input must hold the version of the current round (its producer operation,
//                 enqueued on the rank's own stream before the call, has run; the next round's has not),
//                 and it stamps every output with that version
//   a consumer    enqueued on the rank's stream after the call: the rank's output must hold the round
//
// Rounds vary the rank count's streams (one each, all shared, mixed), the collective and its length (launches
// that carry the ordering themselves, launches between wait and notify kernels, group launches), the
// allocation-free entry point, the rooted collectives, rounds in which one rank's arguments are rejected, and rings of
// send / recv.
// Usage: stream_sim [rounds] [seed] [events | fixed]; prints "ok" or the first violation.
//   events: the ordering by event record / stream-wait-event instead of counters
//   fixed:  every round is the allocation-free all_reduce, and no round may allocate (hipMalloc, hipHostMalloc,
//           hipEventCreate are counted)
#include <sys/mman.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <random>
#include <thread>
#include <vector>

#include "megray.h"
#include "megray/hip_context.h"
#include "vrank_communicator.h"
#include "vrank_edges.h"
#include "vrank_kernels.h"

using namespace MegRay;
using namespace MegRay::vrank;

namespace {

[[noreturn]] void violation(const char* what) {
    std::printf("VIOLATION: %s\n", what);
    std::fflush(stdout);
    std::_Exit(1);
}

// ---------------------------------------------------------------------------------------------
// streams and their executor

struct SimStream {
    std::mutex mutex;
    std::deque<std::function<bool()>> ops;  // an operation returns false while it is not ready
};

std::mutex g_streams_mutex;
std::vector<SimStream*> g_streams;
SimStream g_null_stream;
std::atomic<bool> g_stop{false};
std::atomic<uint64_t> g_pending{0};

SimStream* sim(hipStream_t s) {
    return s ? reinterpret_cast<SimStream*>(s) : &g_null_stream;
}

void push(hipStream_t s, std::function<bool()> op) {
    SimStream* st = sim(s);
    g_pending.fetch_add(1);
    std::lock_guard<std::mutex> lock(st->mutex);
    st->ops.push_back(std::move(op));
}

void executor(uint64_t seed) {
    std::mt19937_64 rng(seed);
    while (!g_stop.load()) {
        std::vector<SimStream*> streams;
        {
            std::lock_guard<std::mutex> lock(g_streams_mutex);
            streams = g_streams;
        }
        streams.push_back(&g_null_stream);
        std::shuffle(streams.begin(), streams.end(), rng);
        bool progress = false;
        for (SimStream* st : streams) {
            if (rng() % 4 == 0) continue;  // a stream that simply is not served for a while
            std::function<bool()> op;
            {
                std::lock_guard<std::mutex> lock(st->mutex);
                if (st->ops.empty()) continue;
                op = st->ops.front();
            }
            if (!op()) continue;
            {
                std::lock_guard<std::mutex> lock(st->mutex);
                st->ops.pop_front();
            }
            g_pending.fetch_sub(1);
            progress = true;
        }
        if (!progress) std::this_thread::yield();
    }
}

void drain() {
    while (g_pending.load()) std::this_thread::yield();
}

// "device memory" counters are plain words the executor and nobody else touches after set-up
uint64_t load_word(const uint64_t* p) { return __atomic_load_n(p, __ATOMIC_ACQUIRE); }
void store_word(uint64_t* p, uint64_t v) { __atomic_store_n(p, v, __ATOMIC_RELEASE); }

// ---------------------------------------------------------------------------------------------
// rank buffers: address ranges large enough for the planner's overlap checks, of which only the first
// word is ever touched: the version the buffer holds

constexpr size_t kRegion = size_t(64) << 20;

uint64_t* region() {
    void* p = mmap(nullptr, kRegion, PROT_READ | PROT_WRITE, MAP_PRIVATE | MAP_ANONYMOUS | MAP_NORESERVE, -1, 0);
    if (p == MAP_FAILED) violation("mmap failed");
    return static_cast<uint64_t*>(p);
}

// what a kernel does: all inputs it reads hold one version, which it stamps on all outputs it writes
void run_kernel(const void* const* in, uint32_t nin, void* const* out, uint32_t nout) {
    uint64_t version = 0;
    bool first = true;
    for (uint32_t i = 0; i < nin; ++i) {
        if (!in[i]) continue;
        const uint64_t v = load_word(static_cast<const uint64_t*>(in[i]));
        if (!first && v != version) violation("a kernel ran while the ranks' inputs held different rounds");
        version = v;
        first = false;
    }
    for (uint32_t i = 0; i < nout; ++i)
        if (out[i]) store_word(static_cast<uint64_t*>(out[i]), version);
}

const int kTagFold = 1, kTagFlat = 2, kTagTree = 3, kTagPack = 4;
int g_tags[5] = {0, kTagFold, kTagFlat, kTagTree, kTagPack};

template <typename L>
std::function<bool()> kernel_op(const L& launch, std::function<void(const L&)> body) {
    return [launch, body]() {
        if (launch.hook_target && load_word(launch.hooks.words) < launch.hook_target) return false;
        body(launch);
        if (launch.hook_ticket) store_word(launch.hooks.words + 1, launch.hook_ticket);
        return true;
    };
}

}  // namespace

// ---------------------------------------------------------------------------------------------
// what the backend's host code calls

namespace MegRay {
namespace vrank {

const void* fold_kernel_for(const FoldLaunch&, DType, ReduceOp) { return &g_tags[kTagFold]; }
const void* flat_kernel_for(const FlatLaunch&, DType, ReduceOp) { return &g_tags[kTagFlat]; }
const void* tree_kernel_for(const TreeLaunch&, DType, ReduceOp) { return &g_tags[kTagTree]; }
const void* pack_kernel_for(const PackLaunch&) { return &g_tags[kTagPack]; }

hipError_t enqueue(const void* kernel, uint32_t grid, uint32_t, const void* launch, hipStream_t stream, uint32_t) {
    if (!kernel) return hipErrorInvalidValue;
    if (!grid) return hipSuccess;
    switch (*static_cast<const int*>(kernel)) {
        case kTagFlat:
            push(stream, kernel_op<FlatLaunch>(*static_cast<const FlatLaunch*>(launch), [](const FlatLaunch& L) {
                     run_kernel(L.in, L.nranks, L.out, L.nranks);
                 }));
            break;
        case kTagFold:
            push(stream, kernel_op<FoldLaunch>(*static_cast<const FoldLaunch*>(launch), [](const FoldLaunch& L) {
                     run_kernel(L.in, L.nranks, L.out, L.nranks);
                 }));
            break;
        case kTagTree:
            push(stream, kernel_op<TreeLaunch>(*static_cast<const TreeLaunch*>(launch), [](const TreeLaunch& L) {
                     void* out[1] = {L.out};
                     run_kernel(L.in, L.nranks, out, 1);
                 }));
            break;
        default:
            push(stream, kernel_op<PackLaunch>(*static_cast<const PackLaunch*>(launch), [](const PackLaunch& L) {
                     run_kernel(L.in, L.nranks, L.out, L.nranks);
                 }));
    }
    return hipSuccess;
}

uint32_t lds_for_waves_per_cu(const void*, uint32_t) { return 0; }

static uint64_t g_static_words[kStaticEdgeSlots * (sizeof(EdgeWords) / sizeof(uint64_t))];

hipError_t edge_static_words(uint32_t slot, EdgeWords** words) {
    if (!words || slot >= kStaticEdgeSlots) return hipErrorInvalidValue;
    *words = reinterpret_cast<EdgeWords*>(g_static_words) + slot;
    return hipSuccess;
}

hipError_t edge_arrive(EdgeWords* words, hipStream_t stream) {
    push(stream, [words]() {
        store_word(&words->arrived, load_word(&words->arrived) + 1);  // only the executor writes
        return true;
    });
    return hipSuccess;
}

hipError_t edge_notify(EdgeWords* words, EdgeWords*, uint64_t ticket, hipStream_t stream) {
    push(stream, [words, ticket]() {
        store_word(&words->done, ticket);
        return true;
    });
    return hipSuccess;
}

hipError_t edge_wait_arrived(EdgeWords* words, EdgeWords*, uint64_t target, uint64_t, uint64_t*, hipStream_t stream) {
    push(stream, [words, target]() { return load_word(&words->arrived) >= target; });
    return hipSuccess;
}

hipError_t edge_wait_done(EdgeWords* words, EdgeWords*, uint64_t ticket, uint64_t, uint64_t*, hipStream_t stream) {
    push(stream, [words, ticket]() { return load_word(&words->done) >= ticket; });
    return hipSuccess;
}

// simulated waits never give up
hipError_t edge_read_timeouts(const EdgeWords*, hipStream_t, uint64_t* timeouts, uint64_t* gave_up_at) {
    *timeouts = *gave_up_at = 0;
    return hipSuccess;
}

}  // namespace vrank
}  // namespace MegRay

// An event holds the marker of its latest record; a wait keeps the marker the event held when the wait was
// enqueued, so that a later record on the same event (from whatever stream) does not change what it waits for.
struct SimEvent {
    std::mutex mutex;
    std::shared_ptr<std::atomic<bool>> latest;
};

extern "C" {

hipError_t hipGetDevice(int* device) {
    *device = 0;
    return hipSuccess;
}
hipError_t hipDeviceGetAttribute(int* value, hipDeviceAttribute_t, int) {
    *value = 100000;
    return hipSuccess;
}
hipError_t hipSetDevice(int) { return hipSuccess; }
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* status) {
    *status = hipStreamCaptureStatusNone;
    return hipSuccess;
}
hipError_t hipGetLastError(void) { return hipSuccess; }
const char* hipGetErrorString(hipError_t) { return "simulated"; }
std::atomic<int> g_allocations{0};  // hipMalloc, hipHostMalloc, hipEventCreate*: what the allocation-free path must not call
hipError_t hipMalloc(void** p, size_t n) {
    g_allocations.fetch_add(1);
    *p = std::calloc(1, n);
    return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFree(void* p) {
    std::free(p);
    return hipSuccess;
}
hipError_t hipHostMalloc(void** p, size_t n, unsigned int) { return hipMalloc(p, n); }
hipError_t hipHostFree(void* p) { return hipFree(p); }
hipError_t hipMemset(void* p, int v, size_t n) {
    std::memset(p, v, n);
    return hipSuccess;
}
hipError_t hipMemsetAsync(void* p, int v, size_t n, hipStream_t) {
    std::memset(p, v, n);  // only ever used on counters nothing else touches yet
    return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipDeviceSynchronize(void) {
    drain();
    return hipSuccess;
}
hipError_t hipEventCreateWithFlags(hipEvent_t* ev, unsigned) {
    g_allocations.fetch_add(1);
    *ev = reinterpret_cast<hipEvent_t>(new SimEvent);
    return hipSuccess;
}
hipError_t hipEventDestroy(hipEvent_t ev) {
    delete reinterpret_cast<SimEvent*>(ev);
    return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t ev, hipStream_t stream) {
    SimEvent* e = reinterpret_cast<SimEvent*>(ev);
    auto marker = std::make_shared<std::atomic<bool>>(false);
    {
        std::lock_guard<std::mutex> lock(e->mutex);
        e->latest = marker;
    }
    push(stream, [marker]() {
        marker->store(true);
        return true;
    });
    return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t stream, hipEvent_t ev, unsigned int) {
    SimEvent* e = reinterpret_cast<SimEvent*>(ev);
    std::shared_ptr<std::atomic<bool>> marker;
    {
        std::lock_guard<std::mutex> lock(e->mutex);
        marker = e->latest;  // the record the event holds when the wait is enqueued
    }
    if (marker) push(stream, [marker]() { return marker->load(); });
    return hipSuccess;
}
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t, hipMemcpyKind, hipStream_t stream) {
    push(stream, [dst, src]() {
        store_word(static_cast<uint64_t*>(dst), load_word(static_cast<const uint64_t*>(src)));
        return true;
    });
    return hipSuccess;
}

}  // extern "C"

// ---------------------------------------------------------------------------------------------
// the driver: one thread per rank, as the reference's tests drive a communicator

namespace {

struct Round {
    int kind;                  // 0 all_reduce, 1 all_gather, 2 all_to_all, 3 reduce_scatter, 4 ring of send / recv,
                               // 5 broadcast, 6 reduce, 7 scatter, 8 gather
    uint32_t root;
    size_t len;
    bool fixed;                // the allocation-free all_reduce
    int poisoned;              // rank whose arguments are rejected, or -1
    std::vector<int> stream;   // per rank: index into the streams (ranks may share)
};

struct Barrier {
    std::mutex m;
    std::condition_variable cv;
    uint32_t n, count = 0, gen = 0;
    explicit Barrier(uint32_t ranks) : n(ranks) {}
    void wait() {
        std::unique_lock<std::mutex> lock(m);
        const uint32_t g = gen;
        if (++count == n) {
            count = 0;
            ++gen;
            cv.notify_all();
        } else {
            cv.wait(lock, [&] { return gen != g; });
        }
    }
};

}  // namespace

int main(int argc, char** argv) {
    const int rounds = argc > 1 ? std::atoi(argv[1]) : 2000;
    const uint64_t seed = argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 7;
    if (argc > 3 && std::strcmp(argv[3], "events") == 0) setenv("MEGRAY_VRANK_EDGES", "events", 1);
    const bool only_fixed = argc > 3 && std::strcmp(argv[3], "fixed") == 0;
    std::mt19937_64 rng(seed);
    const uint32_t nranks = 2 + uint32_t(rng() % 7);

    std::vector<std::unique_ptr<SimStream>> streams;
    for (uint32_t i = 0; i < nranks + 1; ++i) {
        streams.emplace_back(new SimStream);
        g_streams.push_back(streams.back().get());
    }
    std::thread exec(executor, seed ^ 0x5bd1e995);

    // lengths (int32 elements): launches that carry the stream ordering themselves (1 and 118 tiles), a short
    // launch between wait and notify kernels (391 tiles), the group form (2344 tiles), and off-grid lengths
    // that go through the general kernels
    const size_t lengths[] = {16, 30000, 100000, 600000, 3, 1001};
    std::vector<Round> plan(rounds);
    for (Round& r : plan) {
        r.kind = int(rng() % 9);
        r.root = uint32_t(rng() % nranks);
        r.len = lengths[rng() % 6];
        if (r.kind != 0) r.len = r.len / nranks + 1;
        if (only_fixed) {
            r.kind = 0;
            r.len = lengths[rng() % 6];
        }
        r.fixed = r.kind == 0 && (only_fixed || rng() % 5 == 0);
        r.poisoned = (r.kind == 0 && rng() % 10 == 0) ? int(rng() % nranks) : -1;
        r.stream.resize(nranks);
        const int mode = int(rng() % 3);
        for (uint32_t k = 0; k < nranks; ++k)
            r.stream[k] = mode == 0 ? int(k) : mode == 1 ? int(nranks) : (rng() % 2 ? int(k) : int(nranks));
    }

    std::vector<uint64_t*> in(nranks), out(nranks);
    for (uint32_t k = 0; k < nranks; ++k) {
        in[k] = region();
        out[k] = region();
    }

    // init through a caller-supplied broadcast: rank 0's id, handed over in memory
    std::mutex id_mutex;
    std::condition_variable id_cv;
    std::vector<char> id;
    std::vector<std::shared_ptr<Communicator>> comms(nranks);
    for (uint32_t k = 0; k < nranks; ++k) comms[k] = get_communicator(nranks, k, MEGRAY_VRANK);
    Barrier barrier(nranks);
    std::atomic<int> failures{0};

    auto rank_main = [&](uint32_t rank) {
        auto* comm = static_cast<VRankCommunicator*>(comms[rank].get());
        const Status st = comm->init([&](char* data, size_t len) {
            std::unique_lock<std::mutex> lock(id_mutex);
            if (rank == 0) {
                id.assign(data, data + len);
                id_cv.notify_all();
            } else {
                id_cv.wait(lock, [&] { return !id.empty(); });
                std::memcpy(data, id.data(), len);
            }
        });
        if (st != MEGRAY_OK) violation("init failed");
        std::mt19937_64 local(seed * 131 + rank);
        for (int r = 0; r < rounds; ++r) {
            const Round& round = plan[r];
            const uint64_t version = uint64_t(r) + 1;
            hipStream_t stream = reinterpret_cast<hipStream_t>(streams[round.stream[rank]].get());
            auto ctx = HipContext::make(stream);
            uint64_t* src = in[rank];
            uint64_t* dst = out[rank];
            if (local() % 3 == 0) std::this_thread::yield();
            // the producer: this rank's input takes the round's version, on this rank's stream
            push(stream, [src, version]() {
                store_word(src, version);
                return true;
            });
            Status got = MEGRAY_OK;
            bool threw = false;
            try {
                const DType dtype = round.poisoned == int(rank) ? MEGRAY_CHAR : MEGRAY_INT32;
                switch (round.kind) {
                    case 0:
                        got = round.fixed ? comm->all_reduce_no_alloc(src, dst, round.len, dtype, MEGRAY_SUM, ctx)
                                          : comm->all_reduce(src, dst, round.len, dtype, MEGRAY_SUM, ctx);
                        break;
                    case 1: got = comm->all_gather(src, dst, round.len, dtype, ctx); break;
                    case 2: got = comm->all_to_all(src, dst, round.len, dtype, ctx); break;
                    case 3: got = comm->reduce_scatter(src, dst, round.len, dtype, MEGRAY_SUM, ctx); break;
                    case 5: got = comm->broadcast(src, dst, round.len, dtype, round.root, ctx); break;
                    case 6: got = comm->reduce(src, dst, round.len, dtype, MEGRAY_MAX, round.root, ctx); break;
                    case 7: got = comm->scatter(src, dst, round.len, dtype, round.root, ctx); break;
                    case 8: got = comm->gather(src, dst, round.len, dtype, round.root, ctx); break;
                    default:
                        if (nranks < 2) break;
                        comm->group_start();
                        got = comm->send(src, round.len, dtype, (rank + 1) % nranks, ctx);
                        if (got == MEGRAY_OK) got = comm->recv(dst, round.len, dtype, (rank + nranks - 1) % nranks, ctx);
                        {
                            const Status end = comm->group_end();
                            if (got == MEGRAY_OK) got = end;
                        }
                }
            } catch (const MegRay::Exception&) {
                threw = true;
            }
            if (round.poisoned >= 0) {
                if (round.poisoned == int(rank) ? !threw : got != MEGRAY_INVALID_USAGE) violation("a rejected call was not reported");
            } else {
                if (threw || got != MEGRAY_OK) violation("a collective failed");
                // the consumer: this rank's output (if the collective gives it one) holds the round, on this rank's stream
                const bool has_output = (round.kind != 6 && round.kind != 8) || rank == round.root;
                if (has_output) push(stream, [dst, version]() {
                    if (load_word(dst) != version) violation("a rank's stream went on before the collective's result was there");
                    return true;
                });
            }
            // Rounds are kept apart on the host where a later round could overwrite an input the current round has
            // not read yet WITHOUT the library being able to know: a rejected round enqueues nothing, and on
            // shared streams the order of the ranks' own operations is theirs to keep.
            if (round.poisoned >= 0 || r + 1 == rounds || plan[r + 1].stream != round.stream) {
                barrier.wait();
                if (rank == 0) drain();
                barrier.wait();
            }
        }
    };
    std::vector<std::thread> threads;
    for (uint32_t k = 0; k < nranks; ++k) threads.emplace_back(rank_main, k);
    for (auto& t : threads) t.join();
    drain();
    comms.clear();
    g_stop.store(true);
    exec.join();
    if (failures.load()) return 1;
    if (only_fixed && g_allocations.load()) violation("the allocation-free entry point allocated (hipMalloc, hipHostMalloc or hipEventCreate)");
    std::printf("ok %d rounds, %u ranks\n", rounds, nranks);
    return 0;
}
