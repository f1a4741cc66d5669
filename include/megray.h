// Umbrella header of the MegRay API (include/megray.h:13-36 of the reference).
#pragma once

#include "megray/communicator.h"
#include "megray/config.h"
#include "megray/server.h"

#ifdef MEGRAY_WITH_HIP
#include "megray/hip_context.h"
#endif

namespace MegRay {

// Factory (src/megray.cpp:32-60).  This build knows one backend, MEGRAY_VRANK; any other value
// throws MegRay::Exception("unknown backend") exactly as a reference build without that backend.
std::shared_ptr<Communicator> get_communicator(uint32_t nranks, uint32_t rank, Backend backend);

}  // namespace MegRay
