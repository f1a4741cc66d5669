// Cross-stream ordering for the thread-per-rank API: small kernels that let the stream a collective
// runs on wait for the other ranks' streams, and those wait for the collective.
//
// The reference orders its ranks with host-side synchronisation (cudaStreamSynchronize per ring
// step, src/ucx/all_reduce.cpp:30,77) and with flags in shared memory that stream callbacks set and
// a thread polls (src/shm/utils.cpp:71-95).  Here the flags live in device memory and the polling
// is done by a one-wavefront kernel on the waiting stream, so the host never blocks:
//
//   arrive   (a rank's stream)     arrived += 1 once everything enqueued before it has finished
//   wait     (the launch stream)   returns when arrived >= target: the inputs are ready
//   notify   (the launch stream)   done = ticket, after the collective's launches
//   wait     (a rank's stream)     returns when done >= ticket: the outputs are ready
//
// Every wait is enqueued after the kernel that satisfies it, so streams that share a hardware queue
// cannot block each other; and every wait gives up after a time limit, so no wavefront spins for ever.
//
// A wait that gives up POISONS the group: it raises the group's `timeouts` word, and from then on every
// wait of the group returns at once, no notify publishes anything, and every kernel the communicator
// launches for the group returns before its first store (EdgeHooks).  The data a collective would have
// combined too early is never written; the host learns of it through `status` (or, where no host-visible
// word exists, by reading `timeouts` back) and fails every later call of the group.
#pragma once

#include <hip/hip_runtime_api.h>

#include <cstdint>

namespace MegRay {
namespace vrank {

// Device-side words of one communicator group.
struct EdgeWords {
    uint64_t arrived;   // arrive kernels that have run since the group was formed
    uint64_t done;      // ticket of the last collective whose launches have finished
    uint64_t timeouts;  // waits that gave up; not 0 = the group is poisoned
    uint64_t finished;  // workgroups of a launch that publishes `done` itself (EdgeHooks) that have stored
    uint64_t gave_up_at;  // the count or ticket the first wait that gave up was waiting for
    uint64_t reserved[3];
};

// Counters for callers that may not allocate: the library keeps a small array in device memory
// (a file-scope variable of the code object, so every GPU the library runs on holds its own copy
// until the process ends), cut into kStaticEdgeSlots counter blocks.  `edge_static_words` returns
// block `slot` of the current device's copy; the address is looked up once per device and no memory
// is allocated.  A block keeps what its last user left in it: whoever takes a slot clears it.
constexpr uint32_t kStaticEdgeSlots = 32;
hipError_t edge_static_words(uint32_t slot, EdgeWords** words);

// `group` is the block whose `timeouts` word the kernels test and raise (the block of the group the counters
// belong to; `words` itself for the collectives, the group's block for the per-pair blocks of send / recv).
// `status` is host-visible memory of two words: a wait that gives up adds 1 to status[0] and leaves what it
// was waiting for in status[1] (null: neither).
hipError_t edge_arrive(EdgeWords* words, hipStream_t stream);
hipError_t edge_notify(EdgeWords* words, EdgeWords* group, uint64_t ticket, hipStream_t stream);
hipError_t edge_wait_arrived(EdgeWords* words, EdgeWords* group, uint64_t target, uint64_t limit_ticks,
                             uint64_t* status, hipStream_t stream);
hipError_t edge_wait_done(EdgeWords* words, EdgeWords* group, uint64_t ticket, uint64_t limit_ticks,
                          uint64_t* status, hipStream_t stream);
// Reads a block's `timeouts` and `gave_up_at` back: a synchronous copy that waits for `stream` first.
hipError_t edge_read_timeouts(const EdgeWords* words, hipStream_t stream, uint64_t* timeouts, uint64_t* gave_up_at);

}  // namespace vrank
}  // namespace MegRay
