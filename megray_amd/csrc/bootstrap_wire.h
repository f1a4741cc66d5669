// Socket helpers shared by the rendezvous server and client.
//
// Wire format of the bootstrap service (little-endian host integers, as the reference sends them:
// src/core/client.cpp:56-60,75-80,95-111,125-136):
//   connect    client -> u32 rank                         server -> u32 ack (once all ranks are in)
//   barrier    client -> u32 1                            server -> u32 ack
//   broadcast  client -> u32 2, u32 root, u64 len [, len bytes from root]   server -> len bytes
//   allgather  client -> u32 3, u64 len, len bytes        server -> len * nranks bytes
#pragma once

#include <cerrno>
#include <cstddef>
#include <cstdint>

#include <sys/socket.h>
#include <sys/types.h>

namespace MegRay {
namespace wire {

enum Request : uint32_t { kBarrier = 1, kBroadcast = 2, kAllGather = 3 };

// Both return false on error or when the peer closed the connection (*closed says which).
inline bool send_all(int fd, const void* data, size_t len) {
    const char* p = static_cast<const char*>(data);
    while (len) {
        ssize_t n = ::send(fd, p, len, MSG_NOSIGNAL);
        if (n < 0) {
            if (errno == EINTR) continue;
            return false;
        }
        p += n;
        len -= size_t(n);
    }
    return true;
}

inline bool recv_all(int fd, void* data, size_t len, bool* closed = nullptr) {
    char* p = static_cast<char*>(data);
    if (closed) *closed = false;
    while (len) {
        ssize_t n = ::recv(fd, p, len, 0);
        if (n < 0) {
            if (errno == EINTR) continue;
            return false;
        }
        if (n == 0) {
            if (closed) *closed = true;
            return false;
        }
        p += n;
        len -= size_t(n);
    }
    return true;
}

}  // namespace wire
}  // namespace MegRay
