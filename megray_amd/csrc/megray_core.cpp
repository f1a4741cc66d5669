// Core helpers of the MegRay API: dtype sizes and the logger.
#include <cstdarg>
#include <cstdio>

#include "megray/common.h"

namespace MegRay {

// Bytes per element, indexed by DType (src/core/common.cpp:19-38): int8, uint8, int32, uint32, int64,
// uint64, float16, float32, float64, char.
size_t get_dtype_size(DType dtype) {
    static const unsigned char kBytes[MEGRAY_DTYPE_COUNT] = {1, 1, 4, 4, 8, 8, 2, 4, 8, 1};
    const int index = static_cast<int>(dtype);
    if (index < 0 || index >= static_cast<int>(MEGRAY_DTYPE_COUNT)) MEGRAY_THROW("unknown dtype");
    return kBytes[index];
}

// One line per message on stderr: level, place, text (src/core/debug.cpp:19-27).
void MEGRAY_LOG(const char* level, const char* file, int line, const char* fmt, ...) {
    char text[1024];
    va_list args;
    va_start(args, fmt);
    std::vsnprintf(text, sizeof(text), fmt, args);
    va_end(args);
    std::fprintf(stderr, "[%s]\t%s:%d, %s\n", level, file, line, text);
}

}  // namespace MegRay
