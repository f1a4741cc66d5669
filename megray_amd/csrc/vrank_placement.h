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

// Distance from the start of a buffer of `bytes` bytes to the start of the next one.
size_t placement_pitch(size_t bytes);

// offsets[i] of buffer i (bytes[i] long) from a common base, *total = bytes to allocate.
// false if the sum does not fit a size_t.
bool placement_layout(int count, const size_t* bytes, size_t* offsets, size_t* total);

}  // namespace vrank
}  // namespace MegRay
