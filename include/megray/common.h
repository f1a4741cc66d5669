// Enumerations and status macros of the MegRay API.
// Numeric values follow include/megray/common.h of the reference (Status :23-37, Backend :98-104,
// DType :106-118, ReduceOp :122-127) so that callers compiled against either agree; the one
// addition is the MEGRAY_VRANK backend, appended where MEGRAY_BACKEND_COUNT used to be.
#pragma once

#include <cerrno>
#include <cstddef>
#include <cstring>

#include "megray/config.h"
#include "megray/debug.h"

namespace MegRay {

typedef enum {
    MEGRAY_OK = 0,
    MEGRAY_SYS_ERROR = 1,
    MEGRAY_CUDA_ERR = 2,
    MEGRAY_NCCL_ERR = 3,
    MEGRAY_UCX_ERR = 4,
    MEGRAY_ENV_ERROR = 5,
    MEGRAY_INVALID_ARGUMENT = 6,
    MEGRAY_INVALID_USAGE = 7,
    MEGRAY_UNEXPECTED_ERR = 8,
    MEGRAY_NOT_IMPLEMENTED = 9,
    MEGRAY_HIP_ERR = 10,
    MEGRAY_RCCL_ERR = 11,
    MEGRAY_STATUS_COUNT = 12,
} Status;

typedef enum {
    MEGRAY_NCCL = 0,   // not built here
    MEGRAY_UCX = 1,    // not built here
    MEGRAY_RCCL = 2,   // not built here
    MEGRAY_SHM = 3,    // not built here
    MEGRAY_VRANK = 4,  // N virtual ranks resident in one GPU's HBM
    MEGRAY_BACKEND_COUNT = 5,
} Backend;

typedef enum {
    MEGRAY_INT8 = 0,
    MEGRAY_UINT8 = 1,
    MEGRAY_INT32 = 2,
    MEGRAY_UINT32 = 3,
    MEGRAY_INT64 = 4,
    MEGRAY_UINT64 = 5,
    MEGRAY_FLOAT16 = 6,
    MEGRAY_FLOAT32 = 7,
    MEGRAY_FLOAT64 = 8,
    MEGRAY_CHAR = 9,
    MEGRAY_DTYPE_COUNT = 10,
} DType;

typedef enum {
    MEGRAY_SUM = 0,
    MEGRAY_MAX = 1,
    MEGRAY_MIN = 2,
    MEGRAY_REDUCEOP_COUNT = 3,
} ReduceOp;

// Bytes per element; throws MegRay::Exception("unknown dtype") for anything outside DType
// (src/core/common.cpp:19-38).
size_t get_dtype_size(DType dtype);

// Propagate a non-OK Status to the caller (include/megray/common.h:39-46).
#define MEGRAY_CHECK(expr)                            \
    do {                                              \
        MegRay::Status megray_status_ = (expr);       \
        if (megray_status_ != MegRay::MEGRAY_OK) {    \
            MEGRAY_ERROR("error [%d]", megray_status_); \
            return megray_status_;                    \
        }                                             \
    } while (0)

// System-call helpers (include/megray/common.h:48-80): *_CHECK returns MEGRAY_SYS_ERROR,
// *_ASSERT throws.
#define SYS_CHECK_RET(expr, errval, retval)                                    \
    do {                                                                       \
        retval = (expr);                                                       \
        if (retval == errval) {                                                \
            MEGRAY_ERROR("system error [%d]: %s", errno, std::strerror(errno)); \
            return MegRay::MEGRAY_SYS_ERROR;                                   \
        }                                                                      \
    } while (0)

#define SYS_CHECK(expr, errval)                          \
    do {                                                 \
        int megray_ret_;                                 \
        SYS_CHECK_RET(expr, errval, megray_ret_);        \
    } while (0)

#define SYS_ASSERT_RET(expr, errval, retval)                                   \
    do {                                                                       \
        retval = (expr);                                                       \
        if (retval == errval) {                                                \
            MEGRAY_ERROR("system error [%d]: %s", errno, std::strerror(errno)); \
            MEGRAY_THROW("system error");                                      \
        }                                                                      \
    } while (0)

#define SYS_ASSERT(expr, errval)                         \
    do {                                                 \
        int megray_ret_;                                 \
        SYS_ASSERT_RET(expr, errval, megray_ret_);       \
    } while (0)

}  // namespace MegRay
