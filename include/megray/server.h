// Bootstrap service of the MegRay API (include/megray/server.h:19-24).
#pragma once

#include <cstdint>

#include "megray/common.h"

namespace MegRay {

// dotted-quad address of the first non-loopback interface (or of $MEGRAY_NET_DEVICE)
char* get_host_ip();

// a TCP port that was free when asked
int get_free_port();

// start the detached rendezvous thread for a group of `nranks` ranks
Status create_server(uint32_t nranks, int port);

}  // namespace MegRay
