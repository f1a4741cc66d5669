// Logging and the exception type of the MegRay API.
// Mirrors include/megray/debug.h:19-72 of the reference: same macro names, same log-level
// numbering, MegRay::Exception derived from std::runtime_error, MEGRAY_ASSERT logs twice and
// throws "assertion failed".
#pragma once

#include <cstdio>
#include <stdexcept>
#include <string>

#include "megray/config.h"

namespace MegRay {

enum LogLevel { DEBUG = 0, INFO = 1, WARN = 2, ERROR = 3 };

// printf-style line on stderr: "[LEVEL]\tfile:line, message" (src/core/debug.cpp:19-27)
void MEGRAY_LOG(const char* level, const char* file, int line, const char* fmt, ...)
        __attribute__((format(printf, 4, 5)));

#define MEGRAY_LOG_AT(LEVEL, NAME, ...)                                    \
    do {                                                                   \
        if (static_cast<int>(MegRay::LEVEL) >= MEGRAY_LOG_LEVEL)           \
            MegRay::MEGRAY_LOG(NAME, __FILE__, __LINE__, __VA_ARGS__);     \
    } while (0)

#define MEGRAY_DEBUG(...) MEGRAY_LOG_AT(DEBUG, "DEBUG", __VA_ARGS__)
#define MEGRAY_INFO(...) MEGRAY_LOG_AT(INFO, "INFO", __VA_ARGS__)
#define MEGRAY_WARN(...) MEGRAY_LOG_AT(WARN, "WARN", __VA_ARGS__)
#define MEGRAY_ERROR(...) MEGRAY_LOG_AT(ERROR, "ERROR", __VA_ARGS__)

class Exception : public std::runtime_error {
public:
    explicit Exception(const std::string& what_arg) : std::runtime_error(what_arg) {}
};

#define MEGRAY_THROW(message) throw MegRay::Exception(message)

#define MEGRAY_ASSERT(expr, ...)                             \
    do {                                                     \
        if (!(expr)) {                                       \
            MEGRAY_ERROR("assertion failed: %s", #expr);     \
            MEGRAY_ERROR(__VA_ARGS__);                       \
            MEGRAY_THROW("assertion failed");                \
        }                                                    \
    } while (0)

}  // namespace MegRay
