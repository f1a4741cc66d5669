// Where the ranks' buffers lie in HBM relative to each other.
//
// A collective over N virtual ranks reads and writes up to 2N buffers in step: a workgroup touches
// the same offset in all of them at the same time.  The memory system picks channel and bank from
// address bits, so buffers whose start addresses differ by a multiple of a large power of two put
// all these streams on the same banks, row after row, and the rate drops: the 8-rank fp32
// all_reduce of 1 GiB buffers runs at 75 - 78 % of the HBM peak when the buffers are 1 GiB (or
// 1 GiB + 4 MiB, + 8 MiB, + 256 MiB) apart and at 84 % when they are an odd multiple of 128 MiB
// apart; buffers of 16 MiB lying back to back reach 66 %, 128 MiB apart 78 %.  An odd multiple of
// 128 MiB was the best or within half a point of the best distance at every size from 6 MiB to
// 1 GiB per rank (measured with distances of 2, 32, 64 and 128 MiB times an odd number).
//
// The reference has nothing like this: its ranks are devices, and each allocates its own buffers
// (test/performance.cpp:108-110, test/test_base.h:57-66).
#pragma once

#include <cstddef>

namespace MegRay {
namespace vrank {

constexpr size_t kSpreadUnit = size_t(128) << 20;  // distances between spread buffers are odd multiples of this
constexpr size_t kSpreadFrom = size_t(8) << 20;    // smaller buffers stay close together (they live in the caches)
// The buffers an all_gather WRITES (every rank's block is read once and stored into every rank's buffer: eight
// write streams to one read stream, each walking through eight blocks) are served best a multiple of 128 MiB PLUS
// 32 MiB apart:
// all_gather of 8 x 16 MiB fp16 into 128 MiB buffers 79.4 % of the HBM peak with the outputs 128 MiB apart, 82.9 /
// 84.2 / 84.0 / 83.9 / 82.7 / 83.2 / 80.4 / 84.3 at 128 MiB + 8 / 16 / 32 / 48 / 64 / 96 / 128 / 160 MiB; into 512 MiB
// buffers 82.1 % at 512 MiB and 84.9 - 85.4 at + 16 ... + 96 MiB, 82.5 at + 128.  The all_reduce family loses one to two
// points at such distances (8 x 1 GiB 84.0 -> 83.5, 8 x 128 MiB 84.8 -> 82.6, whether all buffers or only the outputs
// move), and a broadcast (one block into every buffer) reads 84 - 85 % either way, so the distance depends on what the
// buffers are for.
constexpr size_t kWrittenShift = size_t(32) << 20;

// What the buffers handed to placement_layout are for.
enum PlacementUse : int {
    kPlaceAny = 0,        // folds and pairwise copies: everything an odd multiple of 128 MiB apart
    kPlaceOneToAll = 1,   // all_gather: the buffers marked as written lie 128 MiB * k + 32 MiB apart
};

// Distance from the start of a buffer of `bytes` bytes to the start of the next one (`written_one_to_all`: the
// buffer is one of those an all_gather stores every rank's block into).
size_t placement_pitch(size_t bytes, bool written_one_to_all = false);

// offsets[i] of buffer i (bytes[i] long) from a common base, *total = bytes to allocate.  `written` (may be null:
// nothing is) marks the buffers the collective writes; it matters for kPlaceOneToAll only.
// false if the sum does not fit a size_t.
bool placement_layout(int count, const size_t* bytes, size_t* offsets, size_t* total, PlacementUse use = kPlaceAny,
                      const unsigned char* written = nullptr);

}  // namespace vrank
}  // namespace MegRay
