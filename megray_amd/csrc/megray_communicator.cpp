// The non-virtual part of MegRay::Communicator and the backend factory
// (src/core/communicator.cpp:17-37 and src/megray.cpp:32-60 of the reference).
#include "megray.h"
#include "vrank_communicator.h"

namespace MegRay {

Status Communicator::init(const char* master_ip, int port) {
    m_client = std::make_shared<Client>(m_nranks, m_rank);
    MEGRAY_CHECK(m_client->connect(master_ip, port));
    return do_init();
}

Status Communicator::init(BcastCallback broadcast_fn) {
    return do_init(broadcast_fn);
}

// element counts become byte counts here; the backends' _send / _recv know nothing of types
Status Communicator::send(const void* src, size_t count, DType dtype, uint32_t peer, ContextPtr ctx) {
    const size_t bytes = count * get_dtype_size(dtype);
    return _send(src, bytes, peer, ctx);
}

Status Communicator::recv(void* dst, size_t count, DType dtype, uint32_t peer, ContextPtr ctx) {
    const size_t bytes = count * get_dtype_size(dtype);
    return _recv(dst, bytes, peer, ctx);
}

std::shared_ptr<Communicator> get_communicator(uint32_t nranks, uint32_t rank, Backend backend) {
    switch (backend) {
        case MEGRAY_VRANK:
            return std::make_shared<VRankCommunicator>(nranks, rank);
        default:
            // the NCCL / UCX / RCCL / SHM backends are not part of this build, exactly like a
            // reference build configured without them
            MEGRAY_THROW("unknown backend");
    }
}

}  // namespace MegRay
