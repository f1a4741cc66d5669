// HIP stream context and HIP error macros, include/megray/hip_context.h:21-54 of the reference.
#pragma once

#include <memory>

#include "megray/context.h"

#ifdef MEGRAY_WITH_HIP

#include <hip/hip_runtime_api.h>

namespace MegRay {

// Logs a failed HIP call; true if `err` is a failure.
inline bool hip_failed(hipError_t err, const char* file, int line) {
    if (err == hipSuccess) return false;
    MEGRAY_LOG("ERROR", file, line, "hip error [%d]: %s", int(err), hipGetErrorString(err));
    return true;
}

}  // namespace MegRay

// returns MEGRAY_HIP_ERR from the enclosing function
#define HIP_CHECK(expr) \
    do { if (MegRay::hip_failed((expr), __FILE__, __LINE__)) return MegRay::MEGRAY_HIP_ERR; } while (0)

// throws MegRay::Exception("hip error")
#define HIP_ASSERT(expr) \
    do { if (MegRay::hip_failed((expr), __FILE__, __LINE__)) MEGRAY_THROW("hip error"); } while (0)

namespace MegRay {

// A HIP stream as the per-call context of a collective.
class HipContext : public Context {
public:
    HipContext(hipStream_t s) : m_stream(s) {}
    ContextType type() const override { return MEGRAY_CTX_HIP; }
    hipStream_t get_stream() { return m_stream; }
    static std::shared_ptr<HipContext> make(hipStream_t s) { return std::make_shared<HipContext>(s); }

private:
    hipStream_t m_stream;
};

}  // namespace MegRay

#endif  // MEGRAY_WITH_HIP
