#include "vrank_placement.h"

#include <cstdint>

namespace MegRay {
namespace vrank {

namespace {

constexpr size_t kPage = 4096, kLargePage = size_t(2) << 20;

bool round_up(size_t value, size_t unit, size_t* out) {
    const size_t units = value / unit + (value % unit != 0);
    if (units > SIZE_MAX / unit) return false;
    *out = units * unit;
    return true;
}

}  // namespace

size_t placement_pitch(size_t bytes, bool written_one_to_all) {
    size_t pitch = 0;
    if (bytes >= kSpreadFrom && written_one_to_all) {
        const size_t units = bytes / kSpreadUnit + (bytes % kSpreadUnit != 0);
        if (units > (SIZE_MAX - kWrittenShift) / kSpreadUnit) return 0;
        return units * kSpreadUnit + kWrittenShift;
    }
    if (bytes >= kSpreadFrom) {
        size_t units = bytes / kSpreadUnit + (bytes % kSpreadUnit != 0);
        units |= 1;  // odd: buffer i starts at i * units * 128 MiB, which differs in bits 27 and up for every i < 32
        if (units > SIZE_MAX / kSpreadUnit) return 0;
        return units * kSpreadUnit;
    }
    const size_t unit = bytes >= kLargePage ? kLargePage : kPage;
    if (!round_up(bytes ? bytes : 1, unit, &pitch)) return 0;
    return pitch;
}

bool placement_layout(int count, const size_t* bytes, size_t* offsets, size_t* total, PlacementUse use,
                      const unsigned char* written) {
    size_t at = 0, end = 0;
    for (int i = 0; i < count; ++i) {
        const size_t pitch = placement_pitch(bytes[i], use == kPlaceOneToAll && written && written[i]);
        size_t own = 0;  // the last buffer needs its own pages only, not the distance to a next one
        if (bytes[i] >= kLargePage && !round_up(at, kLargePage, &at)) return false;  // after smaller buffers
        if (pitch == 0 || pitch > SIZE_MAX - at || !round_up(bytes[i] ? bytes[i] : 1, kPage, &own)) return false;
        offsets[i] = at;
        end = at + own;
        at += pitch;
    }
    *total = end;
    return true;
}

}  // namespace vrank
}  // namespace MegRay
