// HIP stream context and HIP error macros, include/megray/hip_context.h:21-54 of the reference.
#pragma once

#include <memory>

#include "megray/context.h"

#ifdef MEGRAY_WITH_HIP

#include <hip/hip_runtime_api.h>

// returns MEGRAY_HIP_ERR from the enclosing function
#define HIP_CHECK(expr)                                                                     \
    do {                                                                                    \
        hipError_t megray_hip_ = (expr);                                                    \
        if (megray_hip_ != hipSuccess) {                                                    \
            MEGRAY_ERROR("hip error [%d]: %s", megray_hip_, hipGetErrorString(megray_hip_)); \
            return MegRay::MEGRAY_HIP_ERR;                                                  \
        }                                                                                   \
    } while (0)

// throws MegRay::Exception("hip error")
#define HIP_ASSERT(expr)                                                                    \
    do {                                                                                    \
        hipError_t megray_hip_ = (expr);                                                    \
        if (megray_hip_ != hipSuccess) {                                                    \
            MEGRAY_ERROR("hip error [%d]: %s", megray_hip_, hipGetErrorString(megray_hip_)); \
            MEGRAY_THROW("hip error");                                                      \
        }                                                                                   \
    } while (0)

namespace MegRay {

class HipContext : public Context {
public:
    HipContext(hipStream_t stream) : m_stream{stream} {}
    static std::shared_ptr<HipContext> make(hipStream_t stream) {
        return std::make_shared<HipContext>(stream);
    }
    ContextType type() const override { return MEGRAY_CTX_HIP; }
    hipStream_t get_stream() { return m_stream; }

private:
    hipStream_t m_stream;
};

}  // namespace MegRay

#endif  // MEGRAY_WITH_HIP
