// Rendezvous client of the MegRay bootstrap service (include/megray/client.h:24-49).
#pragma once

#include <cstdint>
#include <mutex>

#include "megray/common.h"

namespace MegRay {

// One per rank.  Talks to the server started by create_server(): barrier, broadcast and
// allgather of small host-side metadata.  All sizes are bytes.
class Client {
public:
    Client(uint32_t group_size, uint32_t own_rank);
    ~Client();

    Status connect(const char* master_ip, int port);

    // Returns when every rank has arrived.
    Status barrier();
    // `bytes` from `src` on `root` into `dst` on every rank.
    Status broadcast(const void* src, void* dst, size_t bytes, uint32_t root);
    // `bytes` from every rank's `src`, concatenated by rank into `dst` (bytes * nranks) on every rank.
    Status allgather(const void* src, void* dst, size_t bytes);

private:
    uint32_t m_nranks;
    uint32_t m_rank;
    bool m_connected = false;
    int m_conn;
    std::mutex m_mutex;
};

}  // namespace MegRay
