// extern "C" face of the library (include/megray_vrank.h).
#include "megray_vrank.h"

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <vector>

#include <hip/hip_runtime_api.h>

#include "megray.h"
#include "vrank_communicator.h"
#include "vrank_edges.h"
#include "megray/hip_context.h"
#include "vrank_engine.h"
#include "vrank_kernels.h"
#include "vrank_placement.h"
#include "vrank_plan.h"

struct mrv_comm {
    std::shared_ptr<MegRay::Communicator> comm;
};

struct mrv_client {
    std::unique_ptr<MegRay::Client> client;
};

using namespace MegRay;
using namespace MegRay::vrank;

namespace {

thread_local char g_last_error[256] = "";

void set_error(const char* text) {
    std::snprintf(g_last_error, sizeof(g_last_error), "%s", text);
}

// Runs `body` (which returns a Status), translating exceptions the way the header promises.
template <typename F>
int guarded(F&& body) {
    try {
        set_plan_error("");
        Status st = body();
        if (st == MEGRAY_OK) return int(st);
        // the planner and the rank rendezvous leave their reason in plan_error(), the same text on every rank
        if (plan_error()[0]) {
            set_error(plan_error());
        } else if (st == MEGRAY_HIP_ERR) {
            set_error("hip error (see the log line on stderr)");
        } else if (st == MEGRAY_INVALID_USAGE) {
            set_error("invalid usage (see the log line on stderr)");
        } else {
            set_error("error");
        }
        return int(st);
    } catch (const MegRay::Exception& e) {
        set_error(e.what());
        return int(MEGRAY_INVALID_ARGUMENT);
    } catch (const std::exception& e) {
        set_error(e.what());
        return int(MEGRAY_UNEXPECTED_ERR);
    } catch (...) {  // nothing may unwind through the C boundary
        set_error("unknown failure");
        return int(MEGRAY_UNEXPECTED_ERR);
    }
}

hipStream_t as_stream(void* stream) {
    return static_cast<hipStream_t>(stream);
}

FoldOrder as_order(int order) {
    if (order < 0 || order >= kOrderCount) MEGRAY_THROW("unknown fold order");
    return static_cast<FoldOrder>(order);
}

Schedule as_schedule(int schedule) {
    if (schedule < 0 || schedule >= kSchedCount) MEGRAY_THROW("unknown schedule");
    return static_cast<Schedule>(schedule);
}

void need(const void* p, const char* what) {
    if (!p) MEGRAY_THROW(what);
}

}  // namespace

extern "C" {

int mrv_abi_version(void) {
    return 1;
}

const char* mrv_last_error(void) {
    return g_last_error;
}

size_t mrv_dtype_size(int dtype) {
    try {
        return get_dtype_size(static_cast<DType>(dtype));
    } catch (const MegRay::Exception& e) {
        set_error(e.what());
        return 0;
    }
}

int mrv_reduce(const void* i0, const void* i1, void* o, size_t len, int dtype, int op, void* stream) {
    return guarded([&] {
        return reduce2(i0, i1, o, len, static_cast<DType>(dtype), static_cast<ReduceOp>(op), as_stream(stream));
    });
}

int mrv_all_reduce(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks, size_t len, int dtype,
                   int op, int order, int schedule, void* stream) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        need(recvbuffs, "recvbuffs is null");
        return all_reduce(sendbuffs, recvbuffs, nranks, len, static_cast<DType>(dtype), static_cast<ReduceOp>(op),
                          as_order(order), as_schedule(schedule), as_stream(stream));
    });
}

int mrv_reduce_scatter(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks, size_t recvlen,
                       int dtype, int op, int order, void* stream) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        need(recvbuffs, "recvbuffs is null");
        return reduce_scatter(sendbuffs, recvbuffs, nranks, recvlen, static_cast<DType>(dtype),
                              static_cast<ReduceOp>(op), as_order(order), as_stream(stream));
    });
}

int mrv_all_gather(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks, size_t sendlen,
                   int dtype, void* stream) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        need(recvbuffs, "recvbuffs is null");
        return all_gather(sendbuffs, recvbuffs, nranks, sendlen, static_cast<DType>(dtype), as_stream(stream));
    });
}

int mrv_all_to_all(const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks, size_t len, int dtype,
                   void* stream) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        need(recvbuffs, "recvbuffs is null");
        return all_to_all(sendbuffs, recvbuffs, nranks, len, static_cast<DType>(dtype), as_stream(stream));
    });
}

int mrv_scatter(const void* sendbuff_root, void* const* recvbuffs, uint32_t nranks, size_t recvlen, int dtype,
                uint32_t root, void* stream) {
    return guarded([&] {
        need(recvbuffs, "recvbuffs is null");
        return scatter(sendbuff_root, recvbuffs, nranks, recvlen, static_cast<DType>(dtype), root,
                       as_stream(stream));
    });
}

int mrv_gather(const void* const* sendbuffs, void* recvbuff_root, uint32_t nranks, size_t sendlen, int dtype,
               uint32_t root, void* stream) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        return gather(sendbuffs, recvbuff_root, nranks, sendlen, static_cast<DType>(dtype), root,
                      as_stream(stream));
    });
}

int mrv_broadcast(const void* sendbuff_root, void* const* recvbuffs, uint32_t nranks, size_t len, int dtype,
                  uint32_t root, void* stream) {
    return guarded([&] {
        need(recvbuffs, "recvbuffs is null");
        return broadcast(sendbuff_root, recvbuffs, nranks, len, static_cast<DType>(dtype), root,
                         as_stream(stream));
    });
}

int mrv_chunk_partition(size_t len, uint32_t nchunks, size_t* sizes, size_t* offsets) {
    return guarded([&] {
        if (!nchunks || !sizes || !offsets) MEGRAY_THROW("nchunks must be positive and the arrays non-null");
        uint64_t s[256], o[256];
        if (nchunks > 256) MEGRAY_THROW("at most 256 chunks");
        chunk_partition(len, nchunks, s, o);
        for (uint32_t i = 0; i < nchunks; ++i) {
            sizes[i] = size_t(s[i]);
            offsets[i] = size_t(o[i]);
        }
        return MEGRAY_OK;
    });
}

int mrv_fold_order(int collective, int order, uint32_t nranks, uint32_t chunk, uint32_t* ranks,
                   int* new_wins_ties, uint32_t* nchunks, uint32_t* owner) {
    return guarded([&] {
        if (collective != MRV_ALL_REDUCE && collective != MRV_REDUCE_SCATTER)
            MEGRAY_THROW("fold orders exist for all_reduce and reduce_scatter");
        if (nranks < 1 || nranks > kMaxRanks) MEGRAY_THROW("nranks must be in [1, 32]");
        const FoldOrder fo = as_order(order);
        const Collective coll = collective == MRV_ALL_REDUCE ? kAllReduce : kReduceScatter;
        const uint32_t chunks = order_chunks(fo, nranks);
        if (chunk >= chunks) MEGRAY_THROW("chunk out of range");
        uint8_t start, own;
        int8_t dir;
        chunk_fold_order(coll, fo, nranks, chunk, &start, &dir, &own);
        if (ranks)
            for (uint32_t j = 0; j < nranks; ++j)
                ranks[j] = dir > 0 ? ring_add(start, j, nranks) : ring_sub(start, j, nranks);
        if (new_wins_ties) *new_wins_ties = order_new_wins_ties(coll, fo) ? 1 : 0;
        if (nchunks) *nchunks = chunks;
        if (owner) *owner = own;
        return MEGRAY_OK;
    });
}

}  // extern "C"

namespace {

// Plans `collective` the way the device entry points do.  Throws for contract violations.
Status build_plan(Plan& plan, int collective, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                  size_t count, DType dt, int order, int schedule, uint32_t root) {
    return plan_collective(plan, collective, sendbuffs, recvbuffs, nranks, count, dt, order, schedule, root);
}

}  // namespace

struct mrv_plan {
    Plan plan;
    DType dtype;
    ReduceOp op;
    std::vector<KernelCall> calls;
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    mrv_plan() = default;
    mrv_plan(const mrv_plan&) = delete;
    mrv_plan& operator=(const mrv_plan&) = delete;
    ~mrv_plan() {
        if (exec) (void)hipGraphExecDestroy(exec);
        if (graph) (void)hipGraphDestroy(graph);
    }
};

extern "C" {

int mrv_plan_create(int collective, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                    size_t count, int dtype, int op, int order, int schedule, uint32_t root, uint32_t flags,
                    mrv_plan** out) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        need(recvbuffs, "recvbuffs is null");
        need(out, "plan is null");
        *out = nullptr;
        std::unique_ptr<mrv_plan> p(new mrv_plan);
        p->dtype = static_cast<DType>(dtype);
        p->op = is_reduction(collective) ? static_cast<ReduceOp>(op) : MEGRAY_SUM;
        if (is_reduction(collective)) check_reduce_op(p->op);
        Status st = build_plan(p->plan, collective, sendbuffs, recvbuffs, nranks, count, p->dtype, order, schedule, root);
        if (st != MEGRAY_OK) return st;
        st = resolve(p->plan, p->dtype, p->op, p->calls);
        if (st != MEGRAY_OK) return st;
        if ((flags & MRV_PLAN_GRAPH) && !p->calls.empty()) {
            // a chain of kernel nodes, each depending on the one before it
            HIP_CHECK(hipGraphCreate(&p->graph, 0));
            hipGraphNode_t prev = nullptr;
            for (const KernelCall& call : p->calls) {
                if (!call.grid) continue;
                void* args[] = {const_cast<void*>(call.launch)};
                hipKernelNodeParams params;
                std::memset(&params, 0, sizeof(params));
                params.func = const_cast<void*>(call.kernel);
                params.gridDim = dim3(call.grid);
                params.blockDim = dim3(call.block);
                params.sharedMemBytes = call.lds;
                params.kernelParams = args;
                hipGraphNode_t node = nullptr;
                HIP_CHECK(hipGraphAddKernelNode(&node, p->graph, prev ? &prev : nullptr, prev ? 1 : 0, &params));
                prev = node;
            }
            HIP_CHECK(hipGraphInstantiate(&p->exec, p->graph, nullptr, nullptr, 0));
        }
        *out = p.release();
        return MEGRAY_OK;
    });
}

int mrv_plan_launch(const mrv_plan* plan, void* stream) {
    return guarded([&] {
        need(plan, "plan is null");
        if (plan->exec) {
            HIP_CHECK(hipGraphLaunch(plan->exec, as_stream(stream)));
            return MEGRAY_OK;
        }
        for (const KernelCall& call : plan->calls)
            HIP_CHECK(enqueue(call.kernel, call.grid, call.block, call.launch, as_stream(stream), call.lds));
        return MEGRAY_OK;
    });
}

size_t mrv_plan_launch_count(const mrv_plan* plan) {
    return plan ? plan->calls.size() : 0;
}

void mrv_plan_destroy(mrv_plan* plan) {
    delete plan;  // destroys the graph, if any
}

int mrv_describe(int collective, const void* const* sendbuffs, void* const* recvbuffs, uint32_t nranks,
                 size_t count, int dtype, int order, int schedule, uint32_t root, mrv_plan_run* runs, size_t cap,
                 size_t* nruns, uint64_t* bytes_read, uint64_t* bytes_written) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        need(recvbuffs, "recvbuffs is null");
        Plan plan;
        Status st = build_plan(plan, collective, sendbuffs, recvbuffs, nranks, count, static_cast<DType>(dtype), order,
                               schedule, root);
        if (st != MEGRAY_OK) return st;
        size_t n = 0;
        auto emit = [&](const mrv_plan_run& run) {
            if (runs && n < cap) runs[n] = run;
            ++n;
        };
        for (size_t i = 0; i < plan.steps.size(); ++i) {
            const Step& step = plan.steps[i];
            if (step.kind == Step::kFold) {
                const FoldLaunch& L = step.fold;
                for (uint32_t s = 0; s < L.nseg; ++s) {
                    const FoldSegment& sg = L.seg[s];
                    mrv_plan_run run;
                    std::memset(&run, 0, sizeof(run));
                    run.step = uint32_t(i);
                    run.kind = 0;
                    run.nfold = L.nfold;
                    run.nout = L.nout;
                    run.new_wins_ties = L.new_wins_ties;
                    run.vector = (sg.flags & kSegVector) ? 1 : 0;
                    run.waves = L.waves;
                    run.deal = (L.waves == kGroupWaves && (sg.flags & kSegDeal)) ? 1 : 0;
                    run.paced = L.paced;
                    run.keep = L.keep;
                    run.start = sg.start;
                    run.dir = sg.dir;
                    run.out_first = sg.out_first;
                    const uint32_t next = s + 1 < L.nseg ? L.first_tile[s + 1] : L.total_tiles;
                    run.tiles = next - L.first_tile[s];
                    run.reads_recv = (collective == MRV_ALL_REDUCE && sg.start < nranks && L.in[sg.start] == recvbuffs[sg.start] &&
                                      L.in[sg.start] != sendbuffs[sg.start])
                                             ? 1
                                             : 0;
                    run.in_begin = sg.in_begin;
                    run.out_begin = sg.out_begin;
                    run.count = sg.count;
                    emit(run);
                }
            } else if (step.kind == Step::kFlat) {
                const FlatLaunch& L = step.flat;
                const uint64_t tile = uint64_t(kThreads) * (kVecBytes / L.elem_size);  // elements per tile
                for (uint32_t s = 0; s < L.nruns; ++s) {
                    const uint64_t begin = s ? L.end[s - 1] : 0, end = L.end[s];
                    const uint32_t start = L.meta[s] & 0xffu, out_first = (L.meta[s] >> 16) & 0xffu;
                    mrv_plan_run run;
                    std::memset(&run, 0, sizeof(run));
                    run.step = uint32_t(i);
                    run.kind = 0;
                    run.nfold = L.nranks;
                    run.nout = L.nout;
                    run.new_wins_ties = L.new_wins_ties;
                    run.vector = 2;
                    run.waves = L.waves;
                    run.deal = (L.exchange & 2u) ? 1 : 0;
                    run.paced = (L.exchange & kFlatPaced) ? 1 : 0;
                    run.keep = (L.exchange & kFlatKeep) ? 1 : 0;
                    run.start = start;
                    run.dir = L.tree ? 0 : int(int8_t((L.meta[s] >> 8) & 0xffu));
                    run.out_first = out_first;
                    const uint64_t lo = (begin + tile - 1) / tile, hi = end / tile;  // tiles wholly inside the run
                    run.tiles = uint32_t(hi > lo ? hi - lo : 0);
                    run.reads_recv = (collective == MRV_ALL_REDUCE && start < nranks && L.in[start] == recvbuffs[start] &&
                                      L.in[start] != sendbuffs[start])
                                             ? 1
                                             : 0;
                    run.in_begin = begin;
                    run.out_begin = begin - L.shift[s];
                    run.count = end - begin;
                    emit(run);
                }
            } else if (step.kind == Step::kTree) {
                const TreeLaunch& L = step.tree;
                mrv_plan_run run;
                std::memset(&run, 0, sizeof(run));
                run.step = uint32_t(i);
                run.nfold = L.nranks;
                run.nout = 1;
                run.waves = 1;
                run.keep = L.keep;
                run.start = L.root;
                run.dir = 0;
                run.out_first = L.root;
                run.tiles = L.total_tiles;
                run.count = L.count;
                emit(run);
            } else {
                const PackLaunch& L = step.pack;
                // the slice of every block this launch copies
                // (tiles count whole 16-byte vectors, which start at the destination's first 16-byte boundary, so
                // this is the slice up to a tile's worth of bytes; a launch that reaches the last tile takes the
                // block's end with it)
                const uint64_t per_tile = uint64_t(kThreads) * kVecBytes;
                const uint64_t slice_begin = std::min(L.first_tile * per_tile, L.block_bytes);
                const bool last = L.first_tile + L.tiles_per_copy >= pack_tiles(L.block_bytes);
                const uint64_t slice_bytes = last ? L.block_bytes - slice_begin
                                                  : uint64_t(L.tiles_per_copy) * per_tile;
                for (uint32_t c = 0; c < L.ncopies; ++c) {
                    mrv_plan_run run;
                    std::memset(&run, 0, sizeof(run));
                    run.step = uint32_t(i);
                    run.kind = 1;
                    run.nfold = 1;
                    run.nout = 1;
                    run.vector = L.width;
                    run.waves = L.waves;
                    run.paced = L.paced;
                    run.keep = L.keep;
                    run.dir = 1;
                    run.tiles = L.tiles_per_copy;
                    run.count = slice_bytes;
                    if (L.mode == kPackAllToAll) {
                        run.start = c / L.nranks;
                        run.in_begin = uint64_t(c % L.nranks) * L.block_bytes;
                        run.out_first = c % L.nranks;
                        run.out_begin = uint64_t(c / L.nranks) * L.block_bytes;
                    } else if (L.mode == kPackScatter) {
                        run.start = L.root;
                        run.in_begin = uint64_t(c) * L.block_bytes;
                        run.out_first = c;
                        run.out_begin = 0;
                    } else if (L.mode == kPackBroadcast) {
                        run.start = L.root;
                        run.in_begin = 0;
                        run.out_first = 0;
                        run.nout = L.nranks;
                        run.out_begin = 0;
                    } else if (L.mode == kPackAllGather) {
                        run.start = c;
                        run.in_begin = 0;
                        run.out_first = 0;
                        run.nout = L.nranks;
                        run.out_begin = uint64_t(c) * L.block_bytes;
                    } else {
                        run.start = c;
                        run.in_begin = 0;
                        run.out_first = L.root;
                        run.out_begin = uint64_t(c) * L.block_bytes;
                    }
                    run.in_begin += slice_begin;
                    run.out_begin += slice_begin;
                    emit(run);
                }
            }
        }
        if (nruns) *nruns = n;
        if (bytes_read) *bytes_read = plan.bytes_read;
        if (bytes_written) *bytes_written = plan.bytes_written;
        return MEGRAY_OK;
    });
}

int mrv_reduce_to_root(const void* const* sendbuffs, void* recvbuff_root, uint32_t nranks, size_t len, int dtype,
                       int op, int order, uint32_t root, void* stream) {
    return guarded([&] {
        need(sendbuffs, "sendbuffs is null");
        return reduce_to_root(sendbuffs, recvbuff_root, nranks, len, static_cast<DType>(dtype),
                              static_cast<ReduceOp>(op), as_order(order), root, as_stream(stream));
    });
}

int mrv_probe_bounded_wait(uint64_t limit_us, void* stream, uint64_t* gave_up) {
    return guarded([&] {
        need(gave_up, "gave_up is null");
        *gave_up = 0;
        int device = 0, khz = 0;
        HIP_CHECK(hipGetDevice(&device));
        HIP_CHECK(hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, device));
        EdgeWords* words = nullptr;
        HIP_CHECK(hipMalloc(reinterpret_cast<void**>(&words), sizeof(EdgeWords)));
        Status st = MEGRAY_OK;
        EdgeWords host{};
        // nothing ever counts itself in: the wait can only end by giving up
        if (hipMemsetAsync(words, 0, sizeof(EdgeWords), as_stream(stream)) != hipSuccess ||
            edge_wait_arrived(words, words, 1, limit_us * uint64_t(khz) / 1000, nullptr, as_stream(stream)) != hipSuccess ||
            hipStreamSynchronize(as_stream(stream)) != hipSuccess ||
            hipMemcpy(&host, words, sizeof(host), hipMemcpyDeviceToHost) != hipSuccess) {
            (void)hipGetLastError();
            st = MEGRAY_HIP_ERR;
        }
        (void)hipFree(words);
        *gave_up = host.timeouts;
        return st;
    });
}

namespace {

PlacementUse placement_use(int collective) {
    if (collective < 0) return kPlaceAny;
    if (collective > MRV_REDUCE) MEGRAY_THROW("unknown collective");
    return collective == MRV_ALL_GATHER ? kPlaceOneToAll : kPlaceAny;
}

Status layout_buffers(int collective, int count, const size_t* bytes, const unsigned char* written, size_t* offsets,
                      size_t* total) {
    if (count < 0) MEGRAY_THROW("negative buffer count");
    need(total, "total is null");
    if (count > 0) {
        need(bytes, "bytes is null");
        need(offsets, "offsets is null");
    }
    if (!placement_layout(count, bytes, offsets, total, placement_use(collective), written))
        MEGRAY_THROW("the buffers do not fit the address space");
    return MEGRAY_OK;
}

Status alloc_buffers(int collective, int count, const size_t* bytes, const unsigned char* written, void** ptrs,
                     void** base) {
    if (count <= 0) MEGRAY_THROW("no buffers asked for");
    need(bytes, "bytes is null");
    need(ptrs, "ptrs is null");
    need(base, "base is null");
    *base = nullptr;
    std::vector<size_t> offsets(static_cast<size_t>(count));
    size_t total = 0;
    if (!placement_layout(count, bytes, offsets.data(), &total, placement_use(collective), written))
        MEGRAY_THROW("the buffers do not fit the address space");
    void* p = nullptr;
    HIP_CHECK(hipMalloc(&p, total ? total : 1));
    *base = p;
    for (int i = 0; i < count; ++i) ptrs[i] = static_cast<char*>(p) + offsets[size_t(i)];
    return MEGRAY_OK;
}

}  // namespace

int mrv_rank_buffers_layout(int count, const size_t* bytes, size_t* offsets, size_t* total) {
    return guarded([&] { return layout_buffers(-1, count, bytes, nullptr, offsets, total); });
}

int mrv_rank_buffers_layout_for(int collective, int count, const size_t* bytes, const unsigned char* written,
                                size_t* offsets, size_t* total) {
    return guarded([&] { return layout_buffers(collective, count, bytes, written, offsets, total); });
}

int mrv_rank_buffers_alloc(int count, const size_t* bytes, void** ptrs, void** base) {
    return guarded([&] { return alloc_buffers(-1, count, bytes, nullptr, ptrs, base); });
}

int mrv_rank_buffers_alloc_for(int collective, int count, const size_t* bytes, const unsigned char* written,
                               void** ptrs, void** base) {
    return guarded([&] { return alloc_buffers(collective, count, bytes, written, ptrs, base); });
}

int mrv_rank_buffers_free(void* base) {
    return guarded([&] {
        if (base) HIP_CHECK(hipFree(base));
        return MEGRAY_OK;
    });
}

int mrv_get_free_port(void) {
    try {
        return get_free_port();
    } catch (const std::exception& e) {
        set_error(e.what());
        return -1;
    }
}

int mrv_create_server(uint32_t nranks, int port) {
    return guarded([&] { return create_server(nranks, port); });
}

int mrv_comm_create(uint32_t nranks, uint32_t rank, int backend, mrv_comm** comm) {
    return guarded([&] {
        need(comm, "comm is null");
        *comm = nullptr;
        auto ptr = get_communicator(nranks, rank, static_cast<Backend>(backend));
        *comm = new mrv_comm{ptr};
        return MEGRAY_OK;
    });
}

void mrv_comm_destroy(mrv_comm* comm) {
    delete comm;
}

int mrv_comm_init(mrv_comm* comm, const char* master_ip, int port) {
    return guarded([&] {
        need(comm, "comm is null");
        need(master_ip, "master_ip is null");
        return comm->comm->init(master_ip, port);
    });
}

int mrv_comm_init_callback(mrv_comm* comm, mrv_bcast_fn broadcast, void* user) {
    return guarded([&] {
        need(comm, "comm is null");
        need(reinterpret_cast<const void*>(broadcast), "broadcast is null");
        return comm->comm->init([broadcast, user](char* data, size_t len) { broadcast(data, len, user); });
    });
}

int mrv_comm_check(mrv_comm* comm, void* stream) {
    return guarded([&] {
        need(comm, "comm is null");
        auto* vr = dynamic_cast<VRankCommunicator*>(comm->comm.get());
        if (!vr) MEGRAY_THROW("not a vrank communicator");
        return vr->check(HipContext::make(as_stream(stream)));
    });
}

int mrv_comm_stats(mrv_comm* comm, uint64_t* collectives, uint64_t* plans_built, uint64_t* sleeps) {
    return guarded([&] {
        need(comm, "comm is null");
        auto* vr = dynamic_cast<VRankCommunicator*>(comm->comm.get());
        if (!vr) MEGRAY_THROW("not a vrank communicator");
        const VRankCommunicator::Stats st = vr->stats();
        if (collectives) *collectives = st.collectives;
        if (plans_built) *plans_built = st.plans_built;
        if (sleeps) *sleeps = st.sleeps;
        return MEGRAY_OK;
    });
}

int mrv_comm_configure(mrv_comm* comm, int order, int schedule) {
    return guarded([&] {
        need(comm, "comm is null");
        auto* vr = dynamic_cast<VRankCommunicator*>(comm->comm.get());
        if (!vr) MEGRAY_THROW("not a vrank communicator");
        vr->set_fold_order(as_order(order));
        vr->set_schedule(as_schedule(schedule));
        return MEGRAY_OK;
    });
}

#define COMM_CALL(expr)                                               \
    return guarded([&] {                                              \
        need(comm, "comm is null");                                   \
        auto ctx = HipContext::make(as_stream(stream));               \
        return comm->comm->expr;                                      \
    })

int mrv_comm_send(mrv_comm* comm, const void* sendbuff, size_t len, int dtype, uint32_t rank, void* stream) {
    COMM_CALL(send(sendbuff, len, static_cast<DType>(dtype), rank, ctx));
}

int mrv_comm_recv(mrv_comm* comm, void* recvbuff, size_t len, int dtype, uint32_t rank, void* stream) {
    COMM_CALL(recv(recvbuff, len, static_cast<DType>(dtype), rank, ctx));
}

int mrv_comm_scatter(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t recvlen, int dtype, uint32_t root,
                     void* stream) {
    COMM_CALL(scatter(sendbuff, recvbuff, recvlen, static_cast<DType>(dtype), root, ctx));
}

int mrv_comm_gather(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t sendlen, int dtype, uint32_t root,
                    void* stream) {
    COMM_CALL(gather(sendbuff, recvbuff, sendlen, static_cast<DType>(dtype), root, ctx));
}

int mrv_comm_all_to_all(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype, void* stream) {
    COMM_CALL(all_to_all(sendbuff, recvbuff, len, static_cast<DType>(dtype), ctx));
}

int mrv_comm_all_gather(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t sendlen, int dtype,
                        void* stream) {
    COMM_CALL(all_gather(sendbuff, recvbuff, sendlen, static_cast<DType>(dtype), ctx));
}

int mrv_comm_all_reduce(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype, int op,
                        void* stream) {
    COMM_CALL(all_reduce(sendbuff, recvbuff, len, static_cast<DType>(dtype), static_cast<ReduceOp>(op), ctx));
}

int mrv_comm_all_reduce_no_alloc(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype, int op,
                                 void* stream) {
    return guarded([&] {
        need(comm, "comm is null");
        auto* vr = dynamic_cast<VRankCommunicator*>(comm->comm.get());
        if (!vr) MEGRAY_THROW("not a vrank communicator");
        auto ctx = HipContext::make(as_stream(stream));
        return vr->all_reduce_no_alloc(sendbuff, recvbuff, len, static_cast<DType>(dtype), static_cast<ReduceOp>(op),
                                       ctx);
    });
}

int mrv_comm_reduce_scatter(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t recvlen, int dtype, int op,
                            void* stream) {
    COMM_CALL(reduce_scatter(sendbuff, recvbuff, recvlen, static_cast<DType>(dtype), static_cast<ReduceOp>(op), ctx));
}

int mrv_comm_broadcast(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype, uint32_t root,
                       void* stream) {
    COMM_CALL(broadcast(sendbuff, recvbuff, len, static_cast<DType>(dtype), root, ctx));
}

int mrv_comm_reduce(mrv_comm* comm, const void* sendbuff, void* recvbuff, size_t len, int dtype, int op,
                    uint32_t root, void* stream) {
    COMM_CALL(reduce(sendbuff, recvbuff, len, static_cast<DType>(dtype), static_cast<ReduceOp>(op), root, ctx));
}

int mrv_comm_group_start(mrv_comm* comm) {
    return guarded([&] {
        need(comm, "comm is null");
        return comm->comm->group_start();
    });
}

int mrv_comm_group_end(mrv_comm* comm) {
    return guarded([&] {
        need(comm, "comm is null");
        return comm->comm->group_end();
    });
}

int mrv_client_create(uint32_t nranks, uint32_t rank, mrv_client** client) {
    return guarded([&] {
        need(client, "client is null");
        *client = new mrv_client{std::make_unique<Client>(nranks, rank)};
        return MEGRAY_OK;
    });
}

void mrv_client_destroy(mrv_client* client) {
    delete client;
}

int mrv_client_connect(mrv_client* client, const char* master_ip, int port) {
    return guarded([&] {
        need(client, "client is null");
        return client->client->connect(master_ip, port);
    });
}

int mrv_client_barrier(mrv_client* client) {
    return guarded([&] {
        need(client, "client is null");
        return client->client->barrier();
    });
}

int mrv_client_broadcast(mrv_client* client, const void* sendbuff, void* recvbuff, size_t len, uint32_t root) {
    return guarded([&] {
        need(client, "client is null");
        return client->client->broadcast(sendbuff, recvbuff, len, root);
    });
}

int mrv_client_allgather(mrv_client* client, const void* sendbuff, void* recvbuff, size_t sendlen) {
    return guarded([&] {
        need(client, "client is null");
        return client->client->allgather(sendbuff, recvbuff, sendlen);
    });
}

}  // extern "C"
