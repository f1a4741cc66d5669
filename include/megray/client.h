// Rendezvous client of the MegRay bootstrap service (include/megray/client.h:24-49).
#pragma once

#include <cstdint>
#include <mutex>

#include "megray/common.h"

namespace MegRay {

// One per rank.  Talks to the server started by create_server(): barrier, broadcast and
// allgather of small host-side metadata.
class Client {
public:
    Client(uint32_t nranks, uint32_t rank);
    ~Client();

    Status connect(const char* master_ip, int port);

    // returns when every rank has arrived
    Status barrier();

    // sendbuff (on root) and recvbuff both hold sendlen bytes
    Status broadcast(const void* sendbuff, void* recvbuff, size_t sendlen, uint32_t root);

    // sendbuff holds sendlen bytes, recvbuff holds sendlen * nranks bytes
    Status allgather(const void* sendbuff, void* recvbuff, size_t sendlen);

private:
    uint32_t m_nranks;
    uint32_t m_rank;
    bool m_connected = false;
    int m_conn;
    std::mutex m_mutex;
};

}  // namespace MegRay
