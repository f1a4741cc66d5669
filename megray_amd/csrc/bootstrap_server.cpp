// Rendezvous server of the MegRay bootstrap service: get_host_ip, get_free_port, create_server
// (include/megray/server.h; behaviour of src/core/server.cpp:26-265 of the reference).
//
// One detached thread per group.  It accepts `nranks` connections, learns each peer's rank,
// acknowledges all of them, then serves requests in the order rank 0 issues them: every request is
// collective, so after reading rank 0's request id the thread expects the same id from every other
// rank.  It ends when rank 0 closes its socket.
#include <cstdlib>
#include <cstring>
#include <memory>
#include <thread>
#include <vector>

#include <arpa/inet.h>
#include <ifaddrs.h>
#include <netinet/in.h>
#include <unistd.h>

#include "bootstrap_wire.h"
#include "megray/server.h"

namespace MegRay {

char* get_host_ip() {
    const char* wanted = std::getenv("MEGRAY_NET_DEVICE");
    if (wanted && std::strcmp(wanted, "lo") == 0) {
        MEGRAY_ERROR("illegal net device: lo");
        MEGRAY_THROW("invalid argument");  // src/core/server.cpp:29-33
    }
    struct ifaddrs* list = nullptr;
    SYS_ASSERT(getifaddrs(&list), -1);
    char* result = nullptr;
    for (struct ifaddrs* it = list; it && !result; it = it->ifa_next) {
        if (!it->ifa_addr || it->ifa_addr->sa_family != AF_INET || !it->ifa_name) continue;
        if (std::strcmp(it->ifa_name, "lo") == 0) continue;
        if (wanted && std::strcmp(it->ifa_name, wanted) != 0) continue;
        char text[INET_ADDRSTRLEN];
        const auto* sin = reinterpret_cast<const struct sockaddr_in*>(it->ifa_addr);
        if (!inet_ntop(AF_INET, &sin->sin_addr, text, sizeof(text))) continue;
        MEGRAY_INFO("using net device %s (%s)", it->ifa_name, text);
        result = new char[std::strlen(text) + 1];
        std::strcpy(result, text);
    }
    freeifaddrs(list);
    if (!result) {
        MEGRAY_ERROR("failed to get host ip%s%s", wanted ? " for device " : "", wanted ? wanted : "");
        MEGRAY_THROW("system error");
    }
    return result;
}

int get_free_port() {
    int fd;
    SYS_ASSERT_RET(socket(AF_INET, SOCK_STREAM, 0), -1, fd);
    struct sockaddr_in addr;
    std::memset(&addr, 0, sizeof(addr));
    addr.sin_family = AF_INET;
    addr.sin_addr.s_addr = htonl(INADDR_ANY);
    addr.sin_port = 0;  // the kernel picks
    SYS_ASSERT(bind(fd, reinterpret_cast<struct sockaddr*>(&addr), sizeof(addr)), -1);
    socklen_t len = sizeof(addr);
    SYS_ASSERT(getsockname(fd, reinterpret_cast<struct sockaddr*>(&addr), &len), -1);
    SYS_ASSERT(close(fd), -1);
    return ntohs(addr.sin_port);
}

namespace {

class Session {
public:
    Session(int listen_fd, uint32_t nranks) : m_listen(listen_fd), m_conn(nranks, -1) {}
    ~Session() {
        for (int fd : m_conn)
            if (fd >= 0) close(fd);
        close(m_listen);
    }

    void run() {
        if (!accept_all()) return;
        for (;;) {
            uint32_t request = 0;
            bool closed = false;
            if (!wire::recv_all(m_conn[0], &request, sizeof(request), &closed)) {
                if (!closed) MEGRAY_ERROR("bootstrap server: recv from rank 0 failed");
                return;  // rank 0 went away: the group is done
            }
            bool ok = false;
            switch (request) {
                case wire::kBarrier: ok = barrier(); break;
                case wire::kBroadcast: ok = broadcast(); break;
                case wire::kAllGather: ok = allgather(); break;
                default: MEGRAY_ERROR("bootstrap server: unexpected request id %u", request); break;
            }
            if (!ok) return;
        }
    }

private:
    uint32_t nranks() const { return uint32_t(m_conn.size()); }

    bool accept_all() {
        for (uint32_t i = 0; i < nranks(); ++i) {
            int fd = accept(m_listen, nullptr, nullptr);
            if (fd < 0) {
                MEGRAY_ERROR("bootstrap server: accept failed: %s", std::strerror(errno));
                return false;
            }
            uint32_t rank = 0;
            if (!wire::recv_all(fd, &rank, sizeof(rank)) || rank >= nranks() || m_conn[rank] >= 0) {
                MEGRAY_ERROR("bootstrap server: bad rank announcement");
                close(fd);
                return false;
            }
            m_conn[rank] = fd;
        }
        return ack_all();
    }

    bool ack_all() {
        const uint32_t ack = 0;
        for (int fd : m_conn)
            if (!wire::send_all(fd, &ack, sizeof(ack))) return false;
        return true;
    }

    // every rank but 0 must announce the same request rank 0 did
    bool expect_request(uint32_t rank, uint32_t request) {
        uint32_t got = 0;
        if (!wire::recv_all(m_conn[rank], &got, sizeof(got))) return false;
        if (got != request) {
            MEGRAY_ERROR("bootstrap server: inconsistent request_id from rank %u", rank);
            return false;
        }
        return true;
    }

    bool barrier() {
        for (uint32_t r = 1; r < nranks(); ++r)
            if (!expect_request(r, wire::kBarrier)) return false;
        return ack_all();
    }

    bool broadcast() {
        uint32_t root0 = 0;
        uint64_t len0 = 0;
        if (!wire::recv_all(m_conn[0], &root0, sizeof(root0)) || !wire::recv_all(m_conn[0], &len0, sizeof(len0)))
            return false;
        for (uint32_t r = 1; r < nranks(); ++r) {
            uint32_t root = 0;
            uint64_t len = 0;
            if (!expect_request(r, wire::kBroadcast) || !wire::recv_all(m_conn[r], &root, sizeof(root)) ||
                !wire::recv_all(m_conn[r], &len, sizeof(len)))
                return false;
            if (root != root0 || len != len0) {
                MEGRAY_ERROR("bootstrap server: inconsistent broadcast root / len from rank %u", r);
                return false;
            }
        }
        if (root0 >= nranks()) {
            MEGRAY_ERROR("bootstrap server: broadcast root %u out of range", root0);
            return false;
        }
        std::vector<char> data(len0);
        if (!wire::recv_all(m_conn[root0], data.data(), data.size())) return false;
        for (int fd : m_conn)
            if (!wire::send_all(fd, data.data(), data.size())) return false;
        return true;
    }

    bool allgather() {
        uint64_t len0 = 0;
        if (!wire::recv_all(m_conn[0], &len0, sizeof(len0))) return false;
        for (uint32_t r = 1; r < nranks(); ++r) {
            uint64_t len = 0;
            if (!expect_request(r, wire::kAllGather) || !wire::recv_all(m_conn[r], &len, sizeof(len))) return false;
            if (len != len0) {
                MEGRAY_ERROR("bootstrap server: inconsistent allgather len from rank %u", r);
                return false;
            }
        }
        std::vector<char> data(len0 * nranks());
        for (uint32_t r = 0; r < nranks(); ++r)
            if (!wire::recv_all(m_conn[r], data.data() + r * len0, len0)) return false;
        for (int fd : m_conn)
            if (!wire::send_all(fd, data.data(), data.size())) return false;
        return true;
    }

    int m_listen;
    std::vector<int> m_conn;
};

}  // namespace

Status create_server(uint32_t nranks, int port) {
    if (nranks == 0) {
        MEGRAY_ERROR("create_server: nranks must be positive");
        return MEGRAY_INVALID_ARGUMENT;
    }
    int fd;
    SYS_CHECK_RET(socket(AF_INET, SOCK_STREAM, 0), -1, fd);
    struct sockaddr_in addr;
    std::memset(&addr, 0, sizeof(addr));
    addr.sin_family = AF_INET;
    addr.sin_addr.s_addr = htonl(INADDR_ANY);
    addr.sin_port = htons(uint16_t(port));
    int one = 1;
    if (setsockopt(fd, SOL_SOCKET, SO_REUSEADDR, &one, sizeof(one)) == -1 ||
        bind(fd, reinterpret_cast<struct sockaddr*>(&addr), sizeof(addr)) == -1 ||
        listen(fd, int(nranks)) == -1) {
        MEGRAY_ERROR("system error [%d]: %s", errno, std::strerror(errno));
        close(fd);
        return MEGRAY_SYS_ERROR;
    }
    auto session = std::make_shared<Session>(fd, nranks);
    std::thread([session] { session->run(); }).detach();
    return MEGRAY_OK;
}

}  // namespace MegRay
