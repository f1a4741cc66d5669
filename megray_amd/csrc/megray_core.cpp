// Core helpers of the MegRay API: dtype sizes and the logger.
#include <cstdarg>
#include <cstdio>

#include "megray/common.h"

namespace MegRay {

// src/core/common.cpp:19-38
size_t get_dtype_size(DType dtype) {
    switch (dtype) {
        case MEGRAY_INT8:
        case MEGRAY_UINT8:
        case MEGRAY_CHAR:
            return 1;
        case MEGRAY_FLOAT16:
            return 2;
        case MEGRAY_INT32:
        case MEGRAY_UINT32:
        case MEGRAY_FLOAT32:
            return 4;
        case MEGRAY_INT64:
        case MEGRAY_UINT64:
        case MEGRAY_FLOAT64:
            return 8;
        default:
            MEGRAY_THROW("unknown dtype");
    }
}

// src/core/debug.cpp:19-27
void MEGRAY_LOG(const char* level, const char* file, int line, const char* fmt, ...) {
    std::fprintf(stderr, "[%s]\t%s:%d, ", level, file, line);
    va_list args;
    va_start(args, fmt);
    std::vfprintf(stderr, fmt, args);
    va_end(args);
    std::fputc('\n', stderr);
}

}  // namespace MegRay
