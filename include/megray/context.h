// The per-call communication context (a stream on some platform), include/megray/context.h:19-35.
#pragma once

#include "megray/common.h"

namespace MegRay {

// numeric values as in the reference
enum ContextType {
    MEGRAY_CTX_DEFAULT = 0,
    MEGRAY_CTX_CUDA = 1,  // not built here
    MEGRAY_CTX_HIP = 2,
    MEGRAY_CTX_COUNT = 3,
};

class Context {
public:
    virtual ContextType type() const = 0;  // first in the vtable, as in the reference
    virtual ~Context() = default;
};

}  // namespace MegRay
