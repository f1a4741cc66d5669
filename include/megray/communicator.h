// The abstract MegRay communicator (include/megray/communicator.h:32-123 of the reference).
//
// One object per rank.  All lengths are element counts.  The order of the virtual functions and of
// the data members is the reference's, so the object layout is the same.
#pragma once

#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>

#include "megray/client.h"
#include "megray/common.h"
#include "megray/context.h"

namespace MegRay {

using BcastCallback = std::function<void(char*, size_t len)>;

class Communicator {
public:
    Communicator(uint32_t nranks, uint32_t rank) : m_nranks(nranks), m_rank(rank) {}

    uint32_t nranks() { return m_nranks; }
    uint32_t rank() { return m_rank; }

    // join the group: either through the rendezvous server at master_ip:port, or with a
    // caller-supplied broadcast
    Status init(const char* master_ip, int port);
    Status init(BcastCallback cb);

    // point to point, `len` elements of `dtype` (forwarded to _send / _recv in bytes)
    Status send(const void* sendbuff, size_t len, DType dtype, uint32_t rank,
                std::shared_ptr<Context> ctx);
    Status recv(void* recvbuf, size_t len, DType dtype, uint32_t rank, std::shared_ptr<Context> ctx);

    virtual Status do_init() = 0;
    virtual Status do_init(BcastCallback cb) = 0;

    // sendbuff (root only): recvlen * nranks elements; recvbuff: recvlen elements
    virtual Status scatter(const void* sendbuff, void* recvbuff, size_t recvlen, DType dtype,
                           uint32_t root, std::shared_ptr<Context> ctx) = 0;

    // sendbuff: sendlen elements; recvbuff (root only): sendlen * nranks elements
    virtual Status gather(const void* sendbuff, void* recvbuff, size_t sendlen, DType dtype,
                          uint32_t root, std::shared_ptr<Context> ctx) = 0;

    // both buffers: len * nranks elements
    virtual Status all_to_all(const void* sendbuff, void* recvbuff, size_t len, DType dtype,
                              std::shared_ptr<Context> ctx) = 0;

    // sendbuff: sendlen elements; recvbuff: sendlen * nranks elements
    virtual Status all_gather(const void* sendbuff, void* recvbuff, size_t sendlen, DType dtype,
                              std::shared_ptr<Context> ctx) = 0;

    // both buffers: len elements
    virtual Status all_reduce(const void* sendbuff, void* recvbuff, size_t len, DType dtype,
                              ReduceOp op, std::shared_ptr<Context> ctx) = 0;

    // sendbuff: recvlen * nranks elements; recvbuff: recvlen elements
    virtual Status reduce_scatter(const void* sendbuff, void* recvbuff, size_t recvlen, DType dtype,
                                  ReduceOp op, std::shared_ptr<Context> ctx) = 0;

    // both buffers: len elements
    virtual Status broadcast(const void* sendbuff, void* recvbuff, size_t len, DType dtype,
                             uint32_t root, std::shared_ptr<Context> ctx) = 0;

    // both buffers: len elements; recvbuff is read on root only
    virtual Status reduce(const void* sendbuff, void* recvbuff, size_t len, DType dtype, ReduceOp op,
                          uint32_t root, std::shared_ptr<Context> ctx) = 0;

    // bracket a series of send / recv calls
    virtual Status group_start() = 0;
    virtual Status group_end() = 0;

protected:
    uint32_t m_nranks;
    uint32_t m_rank;
    std::shared_ptr<Client> m_client;

    // sizes in bytes
    virtual Status _send(const void* sendbuff, size_t size, uint32_t rank,
                         std::shared_ptr<Context> ctx) = 0;
    virtual Status _recv(void* recvbuf, size_t size, uint32_t rank, std::shared_ptr<Context> ctx) = 0;
};

}  // namespace MegRay
