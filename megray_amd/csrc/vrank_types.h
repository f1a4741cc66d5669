// Shared between the host planner and the gfx950 kernels: launch descriptors for the
// virtual-rank collectives.  Everything here is plain data that travels as a kernel argument.
#pragma once

#include <cstddef>
#include <cstdint>

namespace MegRay {
namespace vrank {

constexpr uint32_t kMaxRanks = 32;            // virtual ranks per group (the pointer tables of a launch descriptor)
constexpr uint32_t kFlatMaxRanks = 8;         // ... of a flat launch, whose kernels exist for 2, 3, 4 and 8 ranks
constexpr uint32_t kMaxChunks = 2 * kMaxRanks;  // the shm order splits a buffer into 2N chunks
// Segments one general launch descriptor holds (a chunk gives a head, an aligned body and a tail); a collective with
// more of them is cut into several launches.  With the pointer tables the descriptor stays below 4 KiB.
constexpr uint32_t kMaxSegments = 96;
constexpr uint32_t kThreads = 64;             // one 64-wide wavefront per tile (measured best: 1 KiB per buffer per tile)
constexpr uint32_t kVecBytes = 16;            // one 128-bit global load / store per lane

enum SegmentFlags : uint8_t {
    kSegVector = 1,  // tile is walked in 16-byte vectors; begin offsets are vector aligned
    kSegDeal = 2,    // group form: the tiles do not sit on the cache lines of every buffer, so neighbouring tiles
                     // share lines; whole runs of kGroupStride workgroups are dealt to one XCD (one L2) each
};

// A run of elements that all share one fold order and one set of destinations.
struct FoldSegment {
    uint64_t in_begin;    // first element, same index in every input buffer
    uint64_t out_begin;   // first element in every output buffer
    uint64_t count;       // elements
    uint32_t reserved;
    uint8_t start;        // rank whose buffer seeds the accumulator
    int8_t dir;           // +1: start, start+1, ...   -1: start, start-1, ...   (mod nranks)
    uint8_t out_first;    // destinations are ranks out_first .. out_first+nout-1 (mod nranks)
    uint8_t flags;
};

// Cross-stream ordering carried by a launch itself (thread-per-rank API, short launches of one wavefront
// per workgroup): before it reads, every workgroup waits until `arrived` has reached the launch's
// hook_target (the other ranks' streams have got to the collective); after its stores, the last workgroup
// to finish publishes the launch's hook_ticket in `done`.  The words are the group's counters in
// device memory.  Every launch descriptor carries the three fields; 0 in hook_target / hook_ticket
// (what the planner leaves there) means "do not wait" / "do not publish".
//
// `words`, where the communicator sets it (every launch it makes for a group, hooked or not), also tells the
// kernel where the group's poison is: a stream wait of the group that gave up has raised words[2], and a
// kernel that finds it raised returns before its first store - what it would combine was not ready.
// Launches that do not come from a communicator group (the flat entry points) leave `words` null.
struct EdgeHooks {
    uint64_t* words;       // [0] arrived  [1] done  [2] timeouts (not 0: poisoned)  [3] workgroups finished
                           // [4] what the first wait that gave up was waiting for
    uint64_t* status;      // host-visible: [0] waits that gave up, [1] what the last of them was waiting for
    uint64_t limit_ticks;  // a wait gives up after this many wall-clock ticks
};

// One launch of the fold kernel: every output element is a left fold, in a fixed order, over the
// same element of `nfold` input buffers, written to `nout` output buffers.
struct FoldLaunch {
    const void* in[kMaxRanks];
    void* out[kMaxRanks];
    FoldSegment seg[kMaxSegments];
    uint32_t first_tile[kMaxSegments];  // tiles of all earlier segments; unused entries 0xffffffff
    uint32_t nranks;         // modulus of the rank rotation
    uint32_t nfold;          // inputs folded per element (1 = plain copy)
    uint32_t nout;           // destinations per element
    uint32_t nseg;
    uint32_t total_tiles;
    uint32_t new_wins_ties;  // float MAX/MIN: an equal / unordered compare keeps the newcomer
    uint32_t elem_size;
    uint32_t waves;          // wavefronts per workgroup: 1, or 4 for the group form (long vector bodies)
    uint32_t paced;          // group form: a wavefront keeps two loads and two stores in flight (as kFlatPaced)
    uint32_t keep;           // 1: the stores leave their data in the last-level cache (as kFlatKeep)
    uint32_t short_tiles;    // one wavefront per workgroup: 1 = a tile is one group of vectors / kShortElemsPerLane elements
                             // per lane instead of kVecIters groups / kElemsPerLane (short launches: their time is latency)
    uint32_t reserved;
    EdgeHooks hooks;         // one wavefront per workgroup only
    uint64_t hook_target;
    uint64_t hook_ticket;
};

constexpr uint32_t kFlatGuarded = 4;  // FlatLaunch::exchange
constexpr uint32_t kFlatPaced = 8;    // FlatLaunch::exchange, group form: a wavefront keeps two loads and two stores in flight
constexpr uint32_t kFlatKeep = 16;    // FlatLaunch::exchange: the stores leave their data in the last-level cache

// Store policy.  Results normally stream past the caches ("sc1 nt" stores: written through, not kept), which sustains the
// most HBM bandwidth on long launches.  A collective that writes no more than kKeepMaxBytes in all leaves its results in
// the last-level cache instead ("sc1" stores: written through, kept; 256 MiB on MI355X, shared with what the launch reads): whoever
// reads them next finds them there.  Measured on MI355X, all_reduce fp32 over 8 ranks inside a chain "elementwise kernel
// over every rank's result -> all_reduce", time per link, streamed -> kept, per-rank buffers of 4 / 8 / 16 / 32 / 64 / 128 MiB:
// 40.0 -> 38.4 / 55.2 -> 53.4 / 91.8 -> 80.7 / 178 -> 184 / 343 -> 351 / 664 -> 681 us (the all_reduce alone, back to back, % of
// the HBM peak: 96 -> 101 / 80 -> 83 / 77 -> 83 / 81 -> 87 / 83 -> 82.5 / 84.5 -> 83.8).  So: up to 128 MiB written.
// (Loads stay "nt": keeping what a collective reads once gains the chain 4 % up to 8 MiB and costs it 5 % from 32 MiB.)
constexpr uint64_t kKeepMaxBytes = uint64_t(128) << 20;

constexpr uint32_t kMaxFlatRuns = 48;  // 2N chunks cut again at N-1 rank borders

// A flat run's fold order and destinations in one word: start | (dir & 0xff) << 8 | out_first << 16
// (start: the rank whose buffer seeds the accumulator; dir +1 / -1; destinations are ranks
// out_first .. out_first + nout - 1 mod nranks).
constexpr uint32_t flat_meta(uint32_t start, int dir, uint32_t out_first) {
    return (start & 0xffu) | ((uint32_t(dir) & 0xffu) << 8) | ((out_first & 0xffu) << 16);
}

// One launch of the flat fold kernel.  Tile t always covers bytes [1024 t, 1024 t + 1024) of every
// input buffer, so a wavefront can issue its loads before it knows which run it is in; the run (and
// with it the fold order) is looked up while the loads are in flight.  Needs nfold == nranks, all
// buffers 16-byte aligned, runs that tile [0, count) in order, and every shift a multiple of a vector.
//
// The layout serves the short launches, whose time is the latency of a few reads of this very
// structure: a kernel-argument cache line that a wavefront touches for the first time costs about
// 0.2 us on MI355X, so what every wavefront needs sits in as few 64-byte lines as possible (eight
// input pointers, eight output pointers, the scalars, eight run ends, eight run words: five lines for
// an all_reduce of eight ranks) and tables a launch does not need (shifts) are never read.
struct FlatLaunch {
    const void* in[kFlatMaxRanks];
    void* out[kFlatMaxRanks];
    // one line of scalars
    uint64_t count;          // elements per input buffer
    uint64_t hook_target;    // 0: do not wait (see EdgeHooks)
    uint64_t hook_ticket;    // 0: do not publish
    uint32_t nranks;         // == fold width
    uint32_t nout;
    uint32_t nruns;
    uint32_t total_tiles;    // ceil(count * elem_size / 1024)
    uint32_t new_wins_ties;
    uint32_t elem_size;
    uint32_t tree;  // 1: combine in binomial-tree order towards rank `start` instead of a left fold
    uint32_t waves;     // wavefronts per workgroup: 1, or kGroupWaves for the group form (launches of many tiles)
    uint32_t exchange;  // group form: bit 0 = every rank is an output at the inputs' offsets, results are exchanged too;
                        // bit 1 = tiles share cache lines with their neighbours, deal runs of workgroups to XCDs;
                        // bit 3 (kFlatPaced) = a wavefront keeps kGroupLoadsInFlight loads / stores in flight instead of all;
                        // either form: bit 4 (kFlatKeep) = the stores leave their data in the last-level cache;
                        // either form: bit 2 (kFlatGuarded) = the launch belongs to a communicator group, hooks.words
                        // is set and the group's poison is tested before anything is stored (the flag sits here, in
                        // the line of scalars every wavefront reads anyway; `hooks` lies several cache lines further)
    uint32_t unshifted; // 1 = every run's outputs sit at the inputs' offsets (shift == 0 throughout)
    // run i covers elements [end[i - 1], end[i]) (from 0 for the first); unused entries are 0
    uint64_t end[kMaxFlatRuns];
    uint32_t meta[kMaxFlatRuns];   // flat_meta() of the run
    uint64_t shift[kMaxFlatRuns];  // output index = element index - shift
    EdgeHooks hooks;               // one wavefront per tile only
};

// Group form: a workgroup of kGroupWaves wavefronts owns kGroupWaves tiles that lie kGroupStride tiles
// apart.  Short launches keep one wavefront per tile: as long as (nearly) every wavefront of the launch finds room on
// the device at once, one tile per wavefront is the shorter way, and a fold of fewer inputs takes fewer registers and
// less LDS, so more of its wavefronts fit.  Measured crossovers on MI355X, all_reduce, microseconds per launch, group
// form / one wavefront per tile, by tiles per buffer (fp32; fp16 and int64 cross at the same points; reduce_scatter and
// reduce cross at these points or later):
//   8 ranks   2048 5.64 / 4.87   2560 6.62 / 6.86   3072 6.91 / 7.81   4096 8.33 / 11.71
//   4 ranks   4096 5.14 / 4.68   6144 6.55 / 6.18   7168 8.44 / 9.79   8192 9.86 / 10.84
//   3 ranks   8192 6.70 / 5.99   9216 7.47 / 6.87   10240 8.26 / 8.01   12288 10.73 / 12.35
//   2 ranks   12288 6.75 / 6.26   14336 7.64 / 6.97   16384 9.70 / 10.54
// The segment and pack kernels take the group form from 512 tiles on.
constexpr uint32_t kGroupWaves = 4;
constexpr uint32_t kGroupStride = 32;
// A wavefront of the flat group kernel has this many loads in flight, and (where every rank is an output) this many
// stores: two each.  With all eight at once a workgroup puts 32 loads, then 32 stores, on the memory system within a
// few hundred cycles, to the same offsets of buffers whose addresses may differ in a few high bits only; spaced out,
// the same accesses are served faster, and the worse the buffers lie the more it gains.  Measured on MI355X, bare
// kernel of the same shape, 8 x 1 GiB fp32 in, 8 x 1 GiB out, % of the HBM peak, all at once -> two in flight:
// sixteen buffers of one allocation 1 GiB apart 76.3 -> 80.1, 1 GiB + 128 MiB apart 82.1 -> 84.0, sixteen separate
// allocations (inputs first) 76.3 -> 79.1, (each rank's input next to its output) 81.7 -> 82.9.  One in flight loses
// 6 points, three or four gain half as much; two stores with four or eight loads gain 1; fewer workgroups per CU on
// top of it lose.  Short launches, whose time is latency, keep everything in flight at once: the planner sets
// kFlatPaced per launch (paced_launch in vrank_plan.cpp).
constexpr uint32_t kGroupLoadsInFlight = 2;
constexpr uint32_t kGroupStoresInFlight = 2;
constexpr uint32_t kGroupMinTiles = 512;
constexpr uint32_t flat_group_min_tiles(uint32_t nranks) {  // the flat fold's group form starts here
    return nranks >= 8 ? 2560u : nranks == 4 ? 6400u : nranks == 3 ? 10752u : 15360u;
}
// Large flat folds with ONE output (reduce_scatter, reduce, the first launch of the two-phase all_reduce), three
// or more inputs and input tiles on cache-line boundaries stay at one wavefront per tile and run at an occupancy of
// their own: a wavefront has its K loads of 1 KiB in flight at once, and what HBM needs to stay busy (bandwidth x
// latency, 32 - 64 KiB per CU) is in flight with far fewer wavefronts than a CU can hold - the rest only queue up
// in the memory system and get in each other's way.  The occupancy is set by LDS reserved per workgroup at launch,
// on top of what the kernel declares, which nothing ever touches (lds_for_waves_per_cu; LDS is handed out in 128
// units per CU, so only occupancies of 128 / n are to be had).  How many wavefronts serve best depends on the size
// of the buffers, with a step between 128 and 256 MiB per buffer whatever the number of buffers (see below).  Measured on MI355X,
// % of the HBM peak, fp32, buffers placed, reduce_scatter (reduce), by MiB per buffer; "group" is the group form,
// the numbers name wavefronts per CU, "all" no reservation (18 / 25 / 28 per CU for 8 / 4 / 3 ranks):
//   8 ranks    group        7            8            9            10           12           14           all
//      8     82.9 (85.7)  79.1 (80.3)  83.7 (83.2)  83.6 (84.0)  84.7 (87.5)  89.5 (93.4)  90.5 (92.8)  89.5 (90.9)
//     16     85.3 (85.9)  82.1 (79.1)  84.9 (82.2)  85.8 (84.5)  86.9 (87.2)  88.0 (88.6)  88.1 (88.9)  86.7 (87.3)
//     32     80.2 (80.8)  81.7 (79.0)  84.5 (81.2)  84.7 (84.1)  84.9 (85.0)  84.5 (84.9)  84.4 (84.7)  82.3 (82.8)
//     64     82.5 (83.1)  85.0 (83.2)  87.5 (85.1)  88.5 (87.7)  87.7 (87.9)  87.3 (87.8)  87.1 (87.3)  84.8 (85.1)
//    128     83.3 (83.4)  85.5 (84.7)  89.0 (86.8)  89.9 (89.3)  89.1 (89.3)  88.4 (88.9)  88.1 (87.9)  85.8 (85.7)
//    256     81.1 (81.3)  85.4 (83.5)  87.0 (85.0)  85.1 (84.1)  83.4 (83.4)  82.7 (82.5)  81.6 (81.8)  79.5 (79.3)
//   1024     82.3 (82.0)  85.9 (84.4)  85.4 (84.7)  84.3 (83.6)  83.1 (82.7)  82.0 (81.7)  80.2 (80.2)  77.7 (77.4)
//   4 ranks    group        11           12           14           16           18           21           all
//      8     84.5 (86.1)  74.6 (77.1)  76.2 (79.2)  78.4 (78.3)  80.2 (81.5)  81.1 (81.4)  80.6 (82.2)  81.2 (83.8)
//     16     89.4 (89.6)  81.4 (83.4)  83.1 (84.0)  85.3 (86.2)  87.2 (89.0)  88.6 (91.0)  91.0 (93.0)  91.5 (91.9)
//     32     88.7 (88.8)  79.3 (78.5)  81.1 (80.9)  83.0 (82.9)  84.5 (85.2)  85.7 (85.0)  84.3 (82.7)  84.9 (83.3)
//     64     84.9 (85.0)  86.2 (81.8)  87.4 (82.7)  86.3 (85.1)  86.1 (86.7)  86.2 (86.4)  86.1 (85.2)  85.5 (85.6)
//    128     86.7 (87.0)  90.3 (85.2)  91.6 (86.3)  90.6 (89.4)  87.6 (88.4)  87.6 (87.6)  88.5 (87.6)  88.4 (87.9)
//    256     80.2 (80.9)  86.9 (83.8)  87.0 (84.8)  82.6 (82.9)  81.4 (80.5)  81.0 (80.5)  80.7 (80.6)  80.4 (80.2)
//   1024     81.2 (81.4)  87.9 (85.4)  87.4 (85.9)  83.4 (83.0)  81.8 (82.1)  81.7 (81.7)  81.6 (81.9)  81.4 (81.6)
//   3 ranks    group        12           14           16           18           21           25           all
//      8     72.0 (74.5)  70.2 (72.4)  73.0 (74.4)  77.0 (78.4)  77.6 (81.1)  80.9 (83.7)  84.2 (83.2)  83.6 (86.1)
//     16     87.0 (89.3)  77.6 (79.8)  82.1 (83.6)  84.2 (85.9)  85.6 (87.2)  87.2 (88.2)  87.7 (88.4)  87.9 (88.1)
//     32     89.1 (90.4)  78.8 (80.1)  81.1 (82.5)  84.1 (84.7)  87.3 (87.5)  90.0 (90.8)  90.5 (90.2)  90.2 (90.4)
//     64     85.7 (84.8)  77.3 (77.0)  80.0 (80.2)  81.7 (82.1)  84.5 (85.8)  87.5 (88.2)  88.2 (88.6)  88.2 (88.5)
//    128     88.7 (88.1)  82.2 (81.7)  84.1 (83.5)  86.7 (87.0)  90.0 (90.0)  91.1 (92.1)  91.6 (91.7)  91.1 (92.3)
//    256     81.2 (81.2)  84.2 (82.2)  86.2 (83.8)  83.9 (83.3)  82.3 (82.3)  81.4 (81.6)  81.1 (81.8)  80.6 (81.7)
//   1024     82.0 (82.8)  86.3 (83.7)  87.6 (85.2)  84.5 (84.6)  83.5 (83.7)  82.8 (82.5)  82.5 (82.4)  82.7 (82.7)
//   2 ranks  84 in the group form against 84 / 76 / 69 at 16 / 12 / 11: two loads per wavefront need every wavefront there
//            is; left in the group form
// The step between 128 and 256 MiB per buffer is the store policy (kKeepMaxBytes: up to 128 MiB written the stores
// leave their data in the last-level cache, beyond that they stream past it), not the size: with the policy forced,
// 8 / 9 / 12 per CU for eight ranks, 12 / 14 / 18 for four, 14 / 18 / all for three, reduce_scatter (reduce):
//   kept      64 MiB  87.3 / 88.4 / 87.7 (85.5 / 87.9 / 87.1)   87.2 / 86.5 / 84.9 (82.2 / 85.2 / 85.7)   79.4 / 84.5 / 87.5 (80.8 / 85.8 / 88.6)
//            256 MiB  88.3 / 89.7 / 88.0 (86.8 / 89.4 / 88.2)   93.5 / 92.4 / 88.8 (88.4 / 91.3 / 89.0)   87.4 / 91.9 / 92.0 (85.2 / 91.9 / 92.7)
//   streamed  64 MiB  85.4 / 84.2 / 82.1 (83.3 / 83.4 / 81.9)   82.3 / 79.5 / 79.3 (79.6 / 79.7 / 78.6)   78.4 / 79.9 / 79.4 (77.8 / 79.6 / 79.4)
//            256 MiB  87.5 / 85.2 / 82.8 (85.1 / 84.7 / 82.5)   86.8 / 82.5 / 81.0 (84.7 / 82.3 / 79.9)   86.1 / 82.4 / 81.5 (82.9 / 81.9 / 81.1)
// (buffers of 132 MiB already behave like those of 256: 87.1 / 84.6 at 8 / 9 for eight ranks, 83.8 / 81.3 at 14 / all
// for three).  Hence, for launches whose stores are kept: eight ranks 14 per CU below 32 MiB per buffer and 9 from there
// on; four ranks stay in the group form below 64 MiB per buffer, then 14 (elements of 4 and 8 bytes) or 12 (of 1 and
// 2 bytes: at 64 / 128 MiB fp16 reduce 86.9 / 90.0 at 14 against 87.8 / 91.9 at 12, int8 86.8 / 89.7 against 88.0 /
// 91.8; fp32 85.3 / 89.3 against 82.1 / 86.3, int64 84.9 / 88.8 against 82.4 / 86.4); three ranks all that fit.  For
// launches whose stores stream: 8 / 12 / 14 for eight / four / three ranks.  Below 8 MiB per buffer (4 MiB: group
// 85 - 91 against 80 at best for eight ranks) the group form is level or ahead for every rank count.
constexpr uint32_t kFlatOneOutMinTiles = 8192;                  // 8 MiB per buffer
constexpr uint32_t kFlatOneOutMinTilesFourRanks = 65536;        // 64 MiB per buffer
constexpr uint32_t kFlatOneOutSmallTiles = 32768;               // 32 MiB per buffer
// wavefronts per CU of such a launch; 0 = all that fit
constexpr uint32_t flat_one_out_waves_per_cu(uint32_t nranks, uint64_t tiles_per_buffer, bool keep, uint32_t elem_size) {
    if (!keep) return nranks >= 8 ? 8u : nranks == 4 ? 12u : 14u;
    return nranks >= 8   ? (tiles_per_buffer < kFlatOneOutSmallTiles ? 14u : 9u)
           : nranks == 4 ? (elem_size >= 4 ? 14u : 12u)
                         : 0u;
}
// The tree kernel (reduce towards a root for rank counts the flat kernels do not have) has eight loads of 1 KiB in
// flight per wavefront, and like the one-output flat folds it wants fewer wavefronts per CU than fit once its launches
// are long, fewer still where its stores stream past the cache (from 128 MiB written on, kKeepMaxBytes) and the more
// ranks it folds.  Measured on MI355X, % of the HBM peak, fp32, all that fit / 9 / 10 / 12 / 14 / 16 / 20 wavefronts per CU, by
// MiB per buffer:
//    5 ranks   16 MiB 86.2 / 72.5 / 76.0 / 79.8 / 82.6 / 83.5 / 87.1   64 MiB 83.8 / 77.3 / 81.0 / 85.6 / 87.3 / 87.4 / 86.1
//             128 MiB 86.2 / 79.2 / 82.9 / 87.6 / 89.6 / 90.6 / 88.3   256 MiB 79.0 / 76.3 / 80.2 / 84.8 / 85.5 / 83.4 / 80.6
//    7 ranks   16 MiB 85.2 / 79.8 / 81.2 / 82.9 / 83.8 / 86.2 / 87.5   64 MiB 82.5 / 83.4 / 85.1 / 87.0 / 87.0 / 87.3 / 86.0
//             128 MiB 83.1 / 83.8 / 85.5 / 88.2 / 88.6 / 88.2 / 87.2   256 MiB 77.1 / 82.7 / 83.9 / 83.9 / 81.0 / 81.6 / 79.5
//   12 ranks   16 MiB 84.7 / 78.1 / 80.5 / 82.6 / 83.5 / 86.2 / 85.0   64 MiB 82.0 / 82.2 / 84.1 / 86.1 / 86.1 / 86.4 / 84.9
//             128 MiB 81.8 / 82.5 / 84.9 / 87.4 / 87.2 / 86.7 / 85.2   256 MiB 76.9 / 80.3 / 82.6 / 84.5 / 82.1 / 81.6 / 80.1
//   16 ranks   16 MiB 83.9 / 82.1 / 83.6 / 85.4 / 85.6 / 86.6 / 84.6   64 MiB 80.9 / 84.3 / 85.8 / 86.4 / 85.8 / 85.4 / 83.3
//             128 MiB 78.9 / 83.2 / 85.0 / 85.6 / 84.8 / 83.6 / 80.9   256 MiB 76.0 / 83.5 / 84.7 / 82.0 / 80.9 / 80.1 / 78.1
//   32 ranks   16 MiB 81.9 / 84.5 / 86.1 / 86.3 / 86.1 / 87.6 / 82.7   64 MiB 80.3 / 85.1 / 86.1 / 85.4 / 84.5 / 84.5 / 81.8
//             128 MiB 80.2 / 84.4 / 85.6 / 85.1 / 84.1 / 83.7 / 81.8   256 MiB 75.7 / 81.8 / 81.9 / 80.8 / 80.1 / 79.8 / 77.6
// (1 GiB reads like 256 MiB, 8 MiB is best left alone; fp16: 7 ranks x 64 / 256 MiB 82.8 / 77.9 with all that fit, 87.2 at 16 and
// 84.8 at 12; 16 ranks 80.5 / 76.3, 84.8 and 82.2 at 12 and 10.)
// Where the stores stream (256 MiB and 1 GiB per buffer) the plain recursive walk at 16 wavefronts per CU (two or three
// loads per wavefront in flight) is level with the batches at their best occupancy or 1 - 4 points ahead for up to nine
// ranks of 4- and 8-byte elements (same session: 5 ranks fp32 85.9 / 87.5 against 85.5 / 85.5 at 14 / 12, 7 ranks 85.7 / 85.7
// against 83.9 / 81.3 at 12 / 10, 9 ranks 84.7 / 84.2 against 83.6 / 81.2), behind from twelve ranks on (82.6 / 81.8 against
// 84.2 / 81.3 at 12 / 10, 16 ranks 82.3 / 81.1 against 83.6 / 82.3 at 10) and for fp16 and uint8, which it serves at full
// occupancy only (5 ranks 81.0 / 81.2 against 84.9 / 85.6 at 14, 7 ranks 79.9 / 79.4 against 84.8 / 81.8 at 12, 16 ranks
// 78.4 / 77.9 against 82.6 / 80.8 at 10).
// It is also ahead between 2 and 8 MiB per buffer from twelve ranks on, whatever the element type (same-process A/B, fp32,
// microseconds, walk / batches: 12 ranks x 2 MiB 4.10 / 4.15, 4 MiB 8.38 / 9.09, 6 MiB 12.3 / 13.4, 7 MiB 16.5 / 15.7, 8 MiB 17.0 / 16.0; 32 ranks x
// 1.5 MiB 13.0 / 8.4, 2 MiB 14.1 / 11.3, 4 MiB 20.9 / 24.1, 6 MiB 30.5 / 33.7, 7 MiB 37.6 / 41.0, 8 MiB 41.5 / 42.2).
constexpr uint32_t tree_batch(uint32_t nranks, uint32_t elem_size, bool keep, uint64_t tiles_per_buffer) {  // TreeLaunch::batch
    if (!keep) return elem_size >= 4 && nranks <= 9 ? 1u : 8u;
    return nranks >= 12 && tiles_per_buffer > 2048 && tiles_per_buffer < 8192 ? 1u : 8u;
}
constexpr uint32_t tree_waves_per_cu(uint32_t nranks, uint64_t tiles_per_buffer, bool keep, uint32_t elem_size) {  // 0: all that fit
    if (!keep) return tree_batch(nranks, elem_size, keep, tiles_per_buffer) == 1 ? 16u : nranks <= 6 ? 14u : nranks <= 12 ? 12u : 10u;
    if (tiles_per_buffer >= 32768) return nranks <= 8 ? 16u : nranks <= 12 ? 14u : nranks <= 24 ? 12u : 10u;
    return tiles_per_buffer >= 16384 && nranks >= 12 ? 16u : 0u;
}
// The group form of the flat fold behaves the same way once its launches are long: with all of a wavefront's accesses
// issued at once (launches that do not pace them, kFlatPaced) fewer workgroups per CU than its LDS allows serve the
// all_reduce shapes better.  Measured on MI355X, fp32 all_reduce, % of the HBM peak, interleaved in one process, as
// the LDS allows (4 workgroups per CU at 8 ranks, 7 - 8 at 2 - 4) -> capped:
//   8 ranks -> 3 per CU   placed, per-rank buffers of 128 / 256 / 512 MiB / 1 GiB: 84.8 -> 84.8 / 84.3 -> 84.7 / 84.2 -> 84.4 / 83.9 -> 84.4
//                         (int64, 1 GiB: 82.7 -> 83.3); 2 per CU loses 2 points; at 4 / 16 MiB the cap costs 16 points / 1 point
//   4 ranks -> 4 per CU   placed 128 / 256 / 512 MiB: 83.0 -> 84.3 / 83.6 -> 84.5 / 84.4 -> 84.9 (6 per CU 84.5, 3 per CU 85.0);
//                         separate allocations, 256 MiB: 83.6 -> 84.9
//   3 ranks -> 4 per CU   placed 83.1 -> 84.4 / 84.7 -> 85.6 / 83.6 -> 85.1 (6 per CU 83.6, 3 per CU 83.9); separate, 256 MiB: 84.6 -> 85.2
//   2 ranks -> 5 per CU   placed 82.6 -> 83.0 / 84.7 -> 85.2 / 85.3 -> 86.1 (4 per CU 85.4, 3 per CU 76.7); separate, 256 / 512 MiB: 85.1 -> 85.6 / 84.4 -> 85.5
// Launches that pace their accesses need every wavefront they can get (8 ranks: 83 at 4 per CU, 77 at 3, 62 at 2) and are left alone.
constexpr uint64_t kGroupCapMinBytes8 = uint64_t(256) << 20;  // per-rank buffer from which eight-rank launches are capped
constexpr uint64_t kGroupCapMinBytes = uint64_t(128) << 20;   // ... and launches of two to four ranks
constexpr uint32_t group_cap_per_cu(uint32_t nranks) { return nranks >= 8 ? 3u : nranks == 2 ? 5u : 4u; }  // workgroups per CU
constexpr bool flat_one_out(uint32_t nranks, uint32_t nout, uint64_t total_tiles) {
    return nout == 1 && nranks >= 3 && total_tiles >= (nranks == 4 ? kFlatOneOutMinTilesFourRanks : kFlatOneOutMinTiles);
}
// One-wavefront launches below this many workgroups carry the thread-per-rank API's stream ordering
// themselves (EdgeHooks).  Beyond it the release fence every workgroup then executes (it writes the L2 back)
// costs the DEVICE more than the two launches it saves the host: the calls still return quickly, but the
// device falls behind them.  Measured, 8 ranks, a stream per rank, 2000 all_reduces back to back, microseconds
// per all_reduce INCLUDING the final stream synchronisation (and what the calls alone cost the host), with /
// without: 4 tiles 16 (16) / 21, 64 tiles 16 (15) / 21, 128 tiles 19 (16) / 19.5, 192 tiles 20 - 23 (16) / 21,
// 256 tiles 27 - 29 (15) / 19 - 21, 384 tiles 27 - 45 (15) / 21, 512 tiles 36 - 41 (16) / 20.5.
constexpr uint32_t kHookMaxTiles = 136;
constexpr uint32_t group_grid(uint32_t total_tiles) {
    return (total_tiles + kGroupWaves * kGroupStride - 1) / (kGroupWaves * kGroupStride) * kGroupStride;
}

// One launch of the element-wise tree kernel: out[e] = binomial-tree combination of in[*][e]
// towards `root`, any rank count, any alignment.
struct TreeLaunch {
    const void* in[kMaxRanks];
    void* out;
    uint64_t count;
    uint32_t nranks;
    uint32_t root;
    uint32_t elem_size;
    uint32_t total_tiles;  // kThreads lanes per tile
    uint32_t vector;       // 1: a lane takes a 16-byte vector (the last workgroup also the odd elements at the end);
                           // 0: a lane takes one element
    uint32_t keep;         // 1: the stores leave their data in the last-level cache
    uint32_t batch;        // leaves per batch of the tree walk: 8, or 1 (tree_batch)
    EdgeHooks hooks;
    uint64_t hook_target;
    uint64_t hook_ticket;
};

enum PackMode : uint32_t {
    kPackAllToAll = 0,  // copy b = i*N + j : in[i] block j  -> out[j] block i
    kPackScatter = 1,   // copy b = i       : in[root] block i -> out[i] block 0
    kPackGather = 2,    // copy b = i       : in[i] block 0    -> out[root] block i
    kPackAllGather = 3, // copy b = i       : in[i] block 0    -> block i of EVERY out
    kPackBroadcast = 4, // one copy         : in[root] block 0 -> block 0 of EVERY out
};

// One launch of the pack kernel: `ncopies` equally sized block copies whose endpoints follow
// arithmetically from the copy index.
struct PackLaunch {
    const void* in[kMaxRanks];
    void* out[kMaxRanks];
    uint64_t block_bytes;
    uint32_t nranks;
    uint32_t mode;
    uint32_t root;
    uint32_t ncopies;
    uint32_t tiles_per_copy;
    uint32_t width;   // what every block address and the block size are a multiple of: 16, 8, 4, 2 or 1
    uint32_t waves;   // wavefronts per workgroup: 1, or kGroupWaves (long blocks)
    uint32_t groups_per_copy;  // group form: workgroups per block copy
    uint32_t paced;   // group form, all_gather and broadcast: a wavefront issues its N stores one at a time (paced_gather, paced_broadcast in vrank_plan.cpp)
    uint32_t keep;    // 1: the stores leave their data in the last-level cache
    uint64_t first_tile;  // the launch covers tiles [first_tile, first_tile + tiles_per_copy) of every copy (blocks
                          // too long for one grid are cut into several launches; a multiple of the group span)
    EdgeHooks hooks;      // one wavefront per workgroup only
    uint64_t hook_target;
    uint64_t hook_ticket;
};

// The pack kernels move 16 bytes per lane whatever the blocks' alignment.  Each copy lays its tiles out from the
// destination's side: vectors start at the destination's first 16-byte boundary and tile 1 starts at its first 1 KiB
// boundary (tile 0 holds the up to 63 vectors in front of it), so that every whole tile's stores cover whole cache
// lines wherever the block lies; only the loads take the source as it lies (gfx950 serves 128-bit loads at any
// byte address).  The up to 15 bytes in front of the first and behind the last vector are copied one by one, in
// units of the blocks' common alignment (4 bytes at most).
//
// Tiles (kThreads vectors each) of one block copy: at most block_bytes / 16 whole vectors wherever they start, in
// whole tiles plus one partial tile at each end; there is always a tile 0, which also takes the bytes around the
// vectors.
inline uint64_t pack_tiles(uint64_t block_bytes) {
    return (block_bytes / 16 + kThreads - 1) / kThreads + 1;
}
// Tile sizes of the one-wavefront-per-tile kernels.  Measured on MI355X: one 16-byte vector per lane and
// access beats every deeper unroll, for every fold width; a vector tile is kVecIters such groups
// taken one after the other, an element tile kElemsPerLane elements per lane.
constexpr uint32_t kElemsPerLane = 16;
constexpr uint32_t kVecIters = 4;
// Short launches of the general kernel (FoldLaunch::short_tiles: up to kShortTilesMaxBytes per buffer) take a quarter
// of that per workgroup: a wavefront goes through its groups one after the other, one memory round trip each, and
// when every wavefront of the launch fits the device at once anyway, four times the wavefronts finish in a quarter of
// the time (5 ranks x 256 KiB fp32 all_reduce: 10.9 -> 5 us).
// Folds whose buffers are all vectors keep that form well beyond the point where the device is full, because the
// group form (which begins where it ends) only pays on long launches.  Measured on MI355X, microseconds per launch,
// group form / one wavefront per group of vectors, fp32, by KiB per buffer:
//   all_reduce      5 ranks  2048 6.00 / 5.39   4096 8.74 / 7.63   8192 15.5 / 15.4   12288 21.6 / 21.0   16384 27.6 / 28.0   32768 61.3 / 66.4
//                   7 ranks  2048 7.72 / 5.76   4096 11.0 / 9.61   8192 22.7 / 20.3   12288 29.2 / 29.5   16384 37.6 / 38.1   32768 77.6 / 81.2
//                  12 ranks  2048 13.2 / 8.85   4096 18.9 / 16.1   8192 34.0 / 31.8   12288 53.5 / 54.8   16384 71.0 / 74.7   32768 135 / 145
//                  16 ranks  2048 12.0 / 10.2   4096 22.0 / 20.1   8192 43.3 / 44.1   12288 69.7 / 71.8   16384 100 / 104     32768 174 / 192
//     8 ranks, 4 bytes off   2048 8.95 / 6.54   4096 14.1 / 11.4   8192 23.0 / 20.5   12288 31.7 / 31.8   16384 43.5 / 41.4   32768 95.7 / 92.9
//   reduce_scatter  5 ranks  2048 5.43 / 4.60   4096 6.56 / 5.53   8192 9.77 / 8.59   12288 13.2 / 13.2   16384 16.9 / 17.5   32768 31.4 / 34.0
//                   7 ranks  2048 5.99 / 4.69   4096 6.65 / 5.98   8192 12.3 / 11.6   12288 16.7 / 16.9   16384 21.0 / 22.3   32768 42.4 / 41.8
//                  16 ranks  2048 8.56 / 7.33   4096 12.0 / 10.9   8192 23.2 / 22.0   12288 33.6 / 33.7   16384 45.4 / 46.0   32768 89.0 / 91.8
// (with the usual four groups per wavefront the one-wavefront form takes 9 - 25 us at 2048 KiB; from 16 MiB to 256 MiB
// the group form is 2 - 20 % ahead).  fp16 and int64 cross at the same sizes.  One-byte elements, whose arithmetic
// takes longer, cross earlier: int8 all_reduce of 5 / 7 / 16 ranks x 2 MiB 5.97 / 5.65, 11.4 / 7.69, 12.3 / 16.9, x 4 MiB
// 9.44 / 9.89, 11.7 / 12.7, 22.5 / 22.5.  On placed buffers the all_reduce of 12 and 16 ranks x 4 MiB reads 19.1 / 21.0 and
// 22.9 / 25.3 (its stores are kept in the cache at that size), x 8 MiB 35.4 / 32.2 and 43.5 / 43.2.  Hence: up to 8 MiB per
// buffer (3 MiB for folds of twelve and more ranks with several destinations), for one-byte elements up to 2 MiB (1 MiB
// from twelve ranks on).  Launches with element tiles (buffers at differing offsets from a 4-byte boundary) and copies
// keep the 1 MiB limit and take the group form for their vector bodies from kGroupMinTiles on.
constexpr uint32_t kShortElemsPerLane = 4;
constexpr uint64_t kShortTilesMaxBytes = uint64_t(1) << 20;
constexpr uint64_t short_vector_max_bytes(uint32_t elem_size, uint32_t nranks, uint32_t nout) {
    if (elem_size == 1) return nranks >= 12 ? uint64_t(1) << 20 : uint64_t(2) << 20;
    return nranks >= 12 && nout > 1 ? uint64_t(3) << 20 : uint64_t(8) << 20;
}
constexpr uint32_t vec_iters(const FoldLaunch& L) { return L.short_tiles ? 1u : kVecIters; }
constexpr uint32_t elems_per_lane(const FoldLaunch& L) { return L.short_tiles ? kShortElemsPerLane : kElemsPerLane; }

// Elements a workgroup takes of a vector or an element segment (group form: on average).
inline uint64_t tile_elems(const FoldLaunch& L, bool vector) {
    if (vector && L.waves == kGroupWaves) return uint64_t(kThreads) * kGroupWaves * (kVecBytes / L.elem_size);
    uint64_t per_lane = vector ? uint64_t(vec_iters(L)) * (kVecBytes / L.elem_size) : elems_per_lane(L);
    return uint64_t(kThreads) * per_lane;
}

// Workgroups a segment of `count` elements takes.  Group form: the vector body is cut into groups of
// kThreads vectors, and workgroups come in blocks of kGroupStride that cover kGroupWaves * kGroupStride groups.
inline uint64_t segment_tiles(const FoldLaunch& L, bool vector, uint64_t count) {
    if (vector && L.waves == kGroupWaves) {
        const uint64_t per_group = uint64_t(kThreads) * (kVecBytes / L.elem_size);
        const uint64_t groups = (count + per_group - 1) / per_group;
        const uint64_t span = uint64_t(kGroupWaves) * kGroupStride;
        return (groups + span - 1) / span * kGroupStride;
    }
    const uint64_t per_tile = tile_elems(L, vector);
    return (count + per_tile - 1) / per_tile;
}

}  // namespace vrank
}  // namespace MegRay
