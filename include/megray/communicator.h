// The abstract MegRay communicator (include/megray/communicator.h:32-123 of the reference).
//
// One object per rank.  All lengths are element counts.  The order of the virtual functions and of
// the data members is the reference's, so the object layout and the vtable are the same; parameter
// types are the reference's too (ContextPtr is std::shared_ptr<Context> spelled once).
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
using ContextPtr = std::shared_ptr<Context>;

class Communicator {
public:
    Communicator(uint32_t group_size, uint32_t own_rank) : m_nranks(group_size), m_rank(own_rank) {}

    uint32_t nranks() { return m_nranks; }
    uint32_t rank() { return m_rank; }

    // Joins the group: through the rendezvous server at master_ip:port, or with a broadcast the
    // caller supplies.  Both end in do_init of the backend.
    Status init(const char* master_ip, int port);
    Status init(BcastCallback broadcast_fn);

    // Point to point: `count` elements of `dtype` to / from `peer` (forwarded to _send / _recv in bytes).
    Status send(const void* src, size_t count, DType dtype, uint32_t peer, ContextPtr ctx);
    Status recv(void* dst, size_t count, DType dtype, uint32_t peer, ContextPtr ctx);

    virtual Status do_init() = 0;
    virtual Status do_init(BcastCallback broadcast_fn) = 0;

    // src (root only): per_rank * nranks elements; dst: per_rank elements
    virtual Status scatter(const void* src, void* dst, size_t per_rank, DType dtype, uint32_t root, ContextPtr ctx) = 0;
    // src: per_rank elements; dst (root only): per_rank * nranks elements
    virtual Status gather(const void* src, void* dst, size_t per_rank, DType dtype, uint32_t root, ContextPtr ctx) = 0;
    // src, dst: per_pair * nranks elements
    virtual Status all_to_all(const void* src, void* dst, size_t per_pair, DType dtype, ContextPtr ctx) = 0;
    // src: per_rank elements; dst: per_rank * nranks elements
    virtual Status all_gather(const void* src, void* dst, size_t per_rank, DType dtype, ContextPtr ctx) = 0;
    // src, dst: count elements
    virtual Status all_reduce(const void* src, void* dst, size_t count, DType dtype, ReduceOp op, ContextPtr ctx) = 0;
    // src: per_rank * nranks elements; dst: per_rank elements
    virtual Status reduce_scatter(const void* src, void* dst, size_t per_rank, DType dtype, ReduceOp op,
                                  ContextPtr ctx) = 0;
    // src, dst: count elements
    virtual Status broadcast(const void* src, void* dst, size_t count, DType dtype, uint32_t root, ContextPtr ctx) = 0;
    // src, dst: count elements; dst is touched on the root only
    virtual Status reduce(const void* src, void* dst, size_t count, DType dtype, ReduceOp op, uint32_t root,
                          ContextPtr ctx) = 0;

    // Bracket a series of send / recv calls.
    virtual Status group_start() = 0;
    virtual Status group_end() = 0;

protected:
    uint32_t m_nranks;
    uint32_t m_rank;
    std::shared_ptr<Client> m_client;

    // byte counts
    virtual Status _send(const void* src, size_t bytes, uint32_t peer, ContextPtr ctx) = 0;
    virtual Status _recv(void* dst, size_t bytes, uint32_t peer, ContextPtr ctx) = 0;
};

}  // namespace MegRay
