// Rendezvous client of the MegRay bootstrap service (include/megray/client.h; behaviour of
// src/core/client.cpp:22-139 of the reference: retry connecting every 100 ms, one request at a
// time under a mutex, MEGRAY_INVALID_USAGE on double connect or use before connect).
#include <cstring>
#include <mutex>

#include <arpa/inet.h>
#include <netdb.h>
#include <netinet/in.h>
#include <netinet/tcp.h>
#include <unistd.h>

#include "bootstrap_wire.h"
#include "megray/client.h"

namespace MegRay {

namespace {

bool resolve(const char* host, int port, struct sockaddr_in* out) {
    std::memset(out, 0, sizeof(*out));
    out->sin_family = AF_INET;
    out->sin_port = htons(uint16_t(port));
    if (inet_pton(AF_INET, host, &out->sin_addr) == 1) return true;
    struct addrinfo hints;
    std::memset(&hints, 0, sizeof(hints));
    hints.ai_family = AF_INET;
    hints.ai_socktype = SOCK_STREAM;
    struct addrinfo* res = nullptr;
    if (getaddrinfo(host, nullptr, &hints, &res) != 0 || !res) return false;
    out->sin_addr = reinterpret_cast<struct sockaddr_in*>(res->ai_addr)->sin_addr;
    freeaddrinfo(res);
    return true;
}

}  // namespace

Client::Client(uint32_t nranks, uint32_t rank) : m_nranks(nranks), m_rank(rank), m_connected(false), m_conn(-1) {}

Client::~Client() {
    if (m_conn >= 0) close(m_conn);
}

Status Client::connect(const char* master_ip, int port) {
    std::lock_guard<std::mutex> lock(m_mutex);
    if (m_connected) {
        MEGRAY_ERROR("Client already connected");
        return MEGRAY_INVALID_USAGE;
    }
    struct sockaddr_in addr;
    if (!resolve(master_ip, port, &addr)) {
        MEGRAY_ERROR("cannot resolve %s", master_ip);
        return MEGRAY_SYS_ERROR;
    }
    for (;;) {
        SYS_CHECK_RET(socket(AF_INET, SOCK_STREAM, 0), -1, m_conn);
        if (::connect(m_conn, reinterpret_cast<struct sockaddr*>(&addr), sizeof(addr)) == 0) break;
        close(m_conn);  // the server may not be listening yet: try again in 100 ms
        m_conn = -1;
        usleep(100000);
    }
    int one = 1;
    setsockopt(m_conn, IPPROTO_TCP, TCP_NODELAY, &one, sizeof(one));
    uint32_t ack = 0;
    if (!wire::send_all(m_conn, &m_rank, sizeof(m_rank)) || !wire::recv_all(m_conn, &ack, sizeof(ack))) {
        MEGRAY_ERROR("system error [%d]: %s", errno, std::strerror(errno));
        return MEGRAY_SYS_ERROR;
    }
    m_connected = true;
    return MEGRAY_OK;
}

#define CLIENT_IO(expr)                                                          \
    do {                                                                         \
        if (!(expr)) {                                                           \
            MEGRAY_ERROR("system error [%d]: %s", errno, std::strerror(errno));   \
            return MEGRAY_SYS_ERROR;                                             \
        }                                                                        \
    } while (0)

Status Client::barrier() {
    std::lock_guard<std::mutex> lock(m_mutex);
    if (!m_connected) {
        MEGRAY_ERROR("Client not connected");
        return MEGRAY_INVALID_USAGE;
    }
    const uint32_t request = wire::kBarrier;
    uint32_t ack = 0;
    CLIENT_IO(wire::send_all(m_conn, &request, sizeof(request)));
    CLIENT_IO(wire::recv_all(m_conn, &ack, sizeof(ack)));
    return MEGRAY_OK;
}

Status Client::broadcast(const void* sendbuff, void* recvbuff, size_t sendlen, uint32_t root) {
    std::lock_guard<std::mutex> lock(m_mutex);
    if (!m_connected) {
        MEGRAY_ERROR("Client not connected");
        return MEGRAY_INVALID_USAGE;
    }
    const uint32_t request = wire::kBroadcast;
    const uint64_t len = sendlen;
    CLIENT_IO(wire::send_all(m_conn, &request, sizeof(request)));
    CLIENT_IO(wire::send_all(m_conn, &root, sizeof(root)));
    CLIENT_IO(wire::send_all(m_conn, &len, sizeof(len)));
    if (m_rank == root) CLIENT_IO(wire::send_all(m_conn, sendbuff, sendlen));
    CLIENT_IO(wire::recv_all(m_conn, recvbuff, sendlen));
    return MEGRAY_OK;
}

Status Client::allgather(const void* sendbuff, void* recvbuff, size_t sendlen) {
    std::lock_guard<std::mutex> lock(m_mutex);
    if (!m_connected) {
        MEGRAY_ERROR("Client not connected");
        return MEGRAY_INVALID_USAGE;
    }
    const uint32_t request = wire::kAllGather;
    const uint64_t len = sendlen;
    CLIENT_IO(wire::send_all(m_conn, &request, sizeof(request)));
    CLIENT_IO(wire::send_all(m_conn, &len, sizeof(len)));
    CLIENT_IO(wire::send_all(m_conn, sendbuff, sendlen));
    CLIENT_IO(wire::recv_all(m_conn, recvbuff, sendlen * m_nranks));
    return MEGRAY_OK;
}

}  // namespace MegRay
