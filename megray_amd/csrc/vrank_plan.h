// Host planner of the virtual-rank backend: turns one collective call into a short list of kernel
// launches.  Pure host code (no HIP calls), so it can be exercised without a GPU.
//
// The reference runs a ring: N-1 steps, each a 2-input reduce on one chunk per rank, separated by
// sends, receives and host synchronisation (src/ucx/all_reduce.cpp:61-101,
// src/ucx/reduce_scatter.cpp:44-53, src/shm/all_reduce.cpp:88-124).  With all N rank buffers in one
// GPU's memory a "send" is a pointer, and the only thing the ring leaves behind is the ORDER in
// which a chunk's N contributions are combined.  The planner keeps that order per chunk and lets one
// kernel pass do the whole fold.
#pragma once

#include <cstdint>
#include <vector>

#include "megray/common.h"
#include "vrank_types.h"

namespace MegRay {
namespace vrank {

// Which reference loop the per-chunk fold order is taken from.
enum FoldOrder : int {
    kOrderUcx = 0,    // src/ucx/all_reduce.cpp:61-82 resp. src/ucx/reduce_scatter.cpp:44-53
    kOrderShm = 1,    // src/shm/all_reduce.cpp:38-127 + src/shm/communicator.cpp:24-75 (2N chunks)
    kOrderRank0 = 2,  // ranks 0..N-1 for every element (the tests' expectation, test/test_opr.cpp:321-330)
    kOrderCount = 3,
};

// How the fold is laid out in launches.
enum Schedule : int {
    kSchedFused = 0,     // one launch: read N inputs, write every destination
    kSchedTwoPhase = 1,  // reduce-scatter launch (1 destination per chunk) + broadcast-copy launch
    kSchedRing = 2,      // the reference's 2(N-1) ring steps, one launch per step (kOrderUcx only)
    kSchedCount = 3,
};

enum Collective : int { kAllReduce = 0, kReduceScatter = 1 };

struct Step {
    enum Kind : int { kFold = 0, kPack = 1, kFlat = 2, kTree = 3 } kind;
    FoldLaunch fold;
    PackLaunch pack;
    FlatLaunch flat;
    TreeLaunch tree;
};

struct Plan {
    std::vector<Step> steps;
    uint64_t bytes_read = 0;     // algorithmic bytes over all steps
    uint64_t bytes_written = 0;
};

// q = len / C, r = len % C, chunk i has q + (i < r) elements (src/ucx/all_reduce.cpp:33-38,48-51).
void chunk_partition(uint64_t len, uint32_t nchunks, uint64_t* sizes, uint64_t* offsets);

// (n + d) % m and (n + m - d % m) % m (src/ucx/utils.h:24-30)
inline uint32_t ring_add(uint32_t n, uint32_t delta, uint32_t m) { return (n + delta) % m; }
inline uint32_t ring_sub(uint32_t n, uint32_t delta, uint32_t m) { return (n + m - delta % m) % m; }

// Number of chunks `order` splits a buffer into, and whether MAX/MIN ties keep the newcomer.
uint32_t order_chunks(FoldOrder order, uint32_t nranks);
bool order_new_wins_ties(Collective coll, FoldOrder order);
// Seed rank and direction of chunk `chunk`, and the rank on which the ring leaves the finished chunk.
void chunk_fold_order(Collective coll, FoldOrder order, uint32_t nranks, uint32_t chunk, uint8_t* start,
                      int8_t* dir, uint8_t* owner);

// Planners.  Pointers are only inspected (alignment, aliasing), never dereferenced.
// They return MEGRAY_INVALID_ARGUMENT for a rank count outside [1, kMaxRanks], an order / schedule
// combination that does not exist, or buffers that overlap in a way a single pass cannot honour.
Status plan_all_reduce(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                       uint64_t len, uint32_t elem_size, FoldOrder order, Schedule sched);
Status plan_reduce_scatter(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                           uint64_t recvlen, uint32_t elem_size, FoldOrder order, Schedule sched);
Status plan_all_gather(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                       uint64_t sendlen, uint32_t elem_size);
Status plan_all_to_all(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                       uint64_t len, uint32_t elem_size);
Status plan_scatter(Plan& plan, const void* send_root, void* const* recv, uint32_t nranks, uint64_t recvlen,
                    uint32_t elem_size, uint32_t root);
Status plan_gather(Plan& plan, const void* const* send, void* recv_root, uint32_t nranks, uint64_t sendlen,
                   uint32_t elem_size, uint32_t root);
Status plan_broadcast(Plan& plan, const void* send_root, void* const* recv, uint32_t nranks, uint64_t len,
                      uint32_t elem_size, uint32_t root);
// recv_root = combination of send[*] on rank `root`.  kOrderUcx: the binomial tree of
// src/ucx/reduce.cpp:56-80; kOrderShm: the 2N-chunk fold of src/shm/reduce.cpp:21-100; kOrderRank0.
Status plan_reduce(Plan& plan, const void* const* send, void* recv_root, uint32_t nranks, uint64_t len,
                   uint32_t elem_size, FoldOrder order, uint32_t root);
// o = reduce(i0, i1) with the tie convention of src/ucx/kernel.cu:24-38 (equal / unordered -> i1)
Status plan_reduce2(Plan& plan, const void* i0, const void* i1, void* o, uint64_t len, uint32_t elem_size);

// Chooses the store policy of a finished plan (kKeepMaxBytes in vrank_types.h): a collective that writes little leaves
// its results in the last-level cache.  MEGRAY_VRANK_KEEP=always|never in the environment overrides the choice.
void set_store_policy(Plan& plan);
// What the environment says about the planner's choices (pacing, store policy), as one number: part of what a cached
// plan depends on.
int plan_overrides();

const char* plan_error();  // text for the last MEGRAY_INVALID_ARGUMENT of this thread
void set_plan_error(const char* text);  // lets a thread pass the text on to the threads it planned for

}  // namespace vrank
}  // namespace MegRay
