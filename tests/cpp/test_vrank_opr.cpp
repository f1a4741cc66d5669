// Thread-per-rank test of the MegRay C++ API on the MEGRAY_VRANK backend.
//
// Same shape as the reference's driver (test/test_base.h:26-62): create_server on a free port, N
// communicators in one process, one std::thread per rank doing init -> alloc -> H2D -> collective ->
// sync -> D2H, join, compare.  Inputs and expectations are the closed forms of test/test_opr.cpp
// (cited per case).  No gtest: prints one line per case, exits non-zero on the first failure.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <condition_variable>
#include <limits>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "megray.h"

#define REQUIRE(cond)                                                                   \
    do {                                                                                \
        if (!(cond)) {                                                                  \
            std::fprintf(stderr, "FAILED %s:%d: %s\n", __FILE__, __LINE__, #cond);      \
            std::exit(1);                                                               \
        }                                                                               \
    } while (0)

namespace {

using MegRay::Communicator;
using MegRay::Context;

void* dev_alloc(size_t bytes) {
    void* p = nullptr;
    REQUIRE(hipMalloc(&p, bytes ? bytes : 1) == hipSuccess);
    return p;
}

template <typename T>
using RankMain = std::function<void(std::shared_ptr<Communicator>, int port, int rank, std::vector<T>& input,
                                    std::vector<T>& output)>;

// run_test<T> of test/test_base.h:26-62
template <typename T>
void run_test(const char* name, int nranks, std::vector<std::vector<T>>& inputs,
              std::vector<std::vector<T>>& expected, RankMain<T> main_func) {
    std::vector<std::shared_ptr<Communicator>> comms(nranks);
    std::vector<std::vector<T>> outputs(nranks);
    int port = MegRay::get_free_port();
    REQUIRE(MegRay::create_server(nranks, port) == MegRay::MEGRAY_OK);
    for (int i = 0; i < nranks; i++) {
        comms[i] = MegRay::get_communicator(nranks, i, MegRay::MEGRAY_VRANK);
        outputs[i].resize(expected[i].size());
    }
    std::vector<std::thread> threads;
    for (int i = 0; i < nranks; i++)
        threads.emplace_back(main_func, comms[i], port, i, std::ref(inputs[i]), std::ref(outputs[i]));
    for (auto& t : threads) t.join();
    for (int i = 0; i < nranks; i++) {
        for (size_t j = 0; j < expected[i].size(); j++) {
            if (std::memcmp(&expected[i][j], &outputs[i][j], sizeof(T)) != 0) {
                std::fprintf(stderr, "FAILED %s: rank %d element %zu: got %g, want %g\n", name, i, j,
                             double(outputs[i][j]), double(expected[i][j]));
                std::exit(1);
            }
        }
    }
    std::printf("ok   %s\n", name);
}

std::shared_ptr<Context> make_context(hipStream_t* stream) {
    REQUIRE(hipStreamCreate(stream) == hipSuccess);
    return MegRay::HipContext::make(*stream);
}

void enter_rank(std::shared_ptr<Communicator>& comm, int port) {
    REQUIRE(hipSetDevice(0) == hipSuccess);  // every virtual rank lives on the one GPU
    REQUIRE(comm->init("localhost", port) == MegRay::MEGRAY_OK);
}

template <typename T>
void* upload(const std::vector<T>& host) {
    void* p = dev_alloc(host.size() * sizeof(T));
    REQUIRE(hipMemcpy(p, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice) == hipSuccess);
    return p;
}

template <typename T>
void download(std::vector<T>& host, const void* dev, hipStream_t stream) {
    REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
    REQUIRE(hipMemcpy(host.data(), dev, host.size() * sizeof(T), hipMemcpyDeviceToHost) == hipSuccess);
}

void test_init() {  // TEST_COMMUNICATOR_INIT, test/test_opr.cpp:26-45
    const int nranks = 3;
    int port = MegRay::get_free_port();
    REQUIRE(MegRay::create_server(nranks, port) == MegRay::MEGRAY_OK);
    std::vector<std::thread> threads;
    for (int i = 0; i < nranks; i++)
        threads.emplace_back([=] {
            REQUIRE(hipSetDevice(0) == hipSuccess);
            auto comm = MegRay::get_communicator(nranks, i, MegRay::MEGRAY_VRANK);
            REQUIRE(comm->init("localhost", port) == MegRay::MEGRAY_OK);
        });
    for (auto& t : threads) t.join();
    std::printf("ok   Init\n");
}

void test_send_recv() {  // test/test_opr.cpp:63-99
    std::string msg("test_message");
    const size_t len = msg.size();
    std::vector<std::vector<char>> inputs(2), expected(2);
    inputs[0].assign(msg.begin(), msg.end());
    expected[1].assign(msg.begin(), msg.end());
    run_test<char>("SendRecv", 2, inputs, expected,
                   [len](std::shared_ptr<Communicator> comm, int port, int rank, std::vector<char>& in,
                         std::vector<char>& out) {
                       enter_rank(comm, port);
                       hipStream_t stream;
                       auto ctx = make_context(&stream);
                       void* ptr = dev_alloc(len);
                       if (rank == 0) {
                           REQUIRE(hipMemcpy(ptr, in.data(), len, hipMemcpyHostToDevice) == hipSuccess);
                           REQUIRE(comm->send(ptr, len, MegRay::MEGRAY_CHAR, 1, ctx) == MegRay::MEGRAY_OK);
                           REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
                       } else {
                           REQUIRE(comm->recv(ptr, len, MegRay::MEGRAY_CHAR, 0, ctx) == MegRay::MEGRAY_OK);
                           download(out, ptr, stream);
                       }
                   });
}

void test_scatter_gather() {  // test/test_opr.cpp:101-196
    const int nranks = 3, root = 1;
    const size_t len = 10;
    std::vector<std::vector<float>> root_in(nranks), parts(nranks);
    for (int i = 0; i < nranks; i++)
        for (size_t j = 0; j < len; j++) {
            float val = 1.0f * (i + 1) * (j + 2);
            root_in[root].push_back(val);
            parts[i].push_back(val);
        }
    run_test<float>("Scatter", nranks, root_in, parts,
                    [=](std::shared_ptr<Communicator> comm, int port, int rank, std::vector<float>& in,
                        std::vector<float>& out) {
                        enter_rank(comm, port);
                        hipStream_t stream;
                        auto ctx = make_context(&stream);
                        void* out_ptr = dev_alloc(len * sizeof(float));
                        void* in_ptr = rank == root ? upload(in) : nullptr;  // :133-135
                        REQUIRE(comm->scatter(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, root, ctx) == 0);
                        download(out, out_ptr, stream);
                    });
    std::vector<std::vector<float>> gathered(nranks);
    gathered[root] = root_in[root];
    run_test<float>("Gather", nranks, parts, gathered,
                    [=](std::shared_ptr<Communicator> comm, int port, int rank, std::vector<float>& in,
                        std::vector<float>& out) {
                        enter_rank(comm, port);
                        hipStream_t stream;
                        auto ctx = make_context(&stream);
                        void* in_ptr = upload(in);
                        void* out_ptr = rank == root ? dev_alloc(nranks * len * sizeof(float)) : nullptr;
                        REQUIRE(comm->gather(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, root, ctx) == 0);
                        REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
                        if (rank == root) download(out, out_ptr, stream);
                    });
}

void test_all_to_all() {  // test/test_opr.cpp:198-241
    const int nranks = 3;
    const size_t len = 6;
    std::vector<std::vector<float>> in(nranks, std::vector<float>(nranks * len)), out(in);
    for (int i = 0; i < nranks; i++)
        for (int j = 0; j < nranks; j++)
            for (size_t k = 0; k < len; k++) {
                float val = 1.0f * (i + 1) * (j + 2) * (k + 3);
                in[i][j * len + k] = val;
                out[j][i * len + k] = val;
            }
    run_test<float>("AllToAll", nranks, in, out,
                    [=](std::shared_ptr<Communicator> comm, int port, int, std::vector<float>& input,
                        std::vector<float>& output) {
                        enter_rank(comm, port);
                        hipStream_t stream;
                        auto ctx = make_context(&stream);
                        void* in_ptr = upload(input);
                        void* out_ptr = dev_alloc(nranks * len * sizeof(float));
                        REQUIRE(comm->all_to_all(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, ctx) == 0);
                        download(output, out_ptr, stream);
                    });
}

void test_all_gather() {  // test/test_opr.cpp:243-284
    const int nranks = 3;
    const size_t sendlen = 10;
    std::vector<std::vector<float>> in(nranks, std::vector<float>(sendlen));
    std::vector<std::vector<float>> out(nranks, std::vector<float>(nranks * sendlen));
    for (size_t j = 0; j < sendlen; j++)
        for (int i = 0; i < nranks; i++) {
            in[i][j] = 1.0f * (i + 1) * (j + 1);
            for (int k = 0; k < nranks; k++) out[k][i * sendlen + j] = in[i][j];
        }
    run_test<float>("AllGather", nranks, in, out,
                    [=](std::shared_ptr<Communicator> comm, int port, int, std::vector<float>& input,
                        std::vector<float>& output) {
                        enter_rank(comm, port);
                        hipStream_t stream;
                        auto ctx = make_context(&stream);
                        void* in_ptr = upload(input);
                        void* out_ptr = dev_alloc(nranks * sendlen * sizeof(float));
                        REQUIRE(comm->all_gather(in_ptr, out_ptr, sendlen, MegRay::MEGRAY_FLOAT32, ctx) == 0);
                        download(output, out_ptr, stream);
                    });
}

float fold(MegRay::ReduceOp op, const std::vector<std::vector<float>>& in, int nranks, size_t j) {
    // the reference's expectations: sum from 0, max from numeric_limits::min(), min from max()
    // (test/test_opr.cpp:321-358)
    if (op == MegRay::MEGRAY_SUM) {
        float sum = 0;
        for (int i = 0; i < nranks; i++) sum += in[i][j];
        return sum;
    }
    if (op == MegRay::MEGRAY_MAX) {
        float v = std::numeric_limits<float>::min();
        for (int i = 0; i < nranks; i++) v = std::max(v, in[i][j]);
        return v;
    }
    float v = std::numeric_limits<float>::max();
    for (int i = 0; i < nranks; i++) v = std::min(v, in[i][j]);
    return v;
}

void test_all_reduce() {  // test/test_opr.cpp:286-359
    const int nranks = 3;
    const size_t len = 10;
    for (auto op : {MegRay::MEGRAY_SUM, MegRay::MEGRAY_MAX, MegRay::MEGRAY_MIN}) {
        std::vector<std::vector<float>> in(nranks, std::vector<float>(len)), out(in);
        for (size_t j = 0; j < len; j++) {
            for (int i = 0; i < nranks; i++) in[i][j] = 1.0f * (i + 1) * (j + 1);
            for (int i = 0; i < nranks; i++) out[i][j] = fold(op, in, nranks, j);
        }
        std::string name = "AllReduce op=" + std::to_string(int(op));
        run_test<float>(name.c_str(), nranks, in, out,
                        [=](std::shared_ptr<Communicator> comm, int port, int, std::vector<float>& input,
                            std::vector<float>& output) {
                            enter_rank(comm, port);
                            hipStream_t stream;
                            auto ctx = make_context(&stream);
                            void* in_ptr = upload(input);
                            void* out_ptr = dev_alloc(len * sizeof(float));
                            REQUIRE(comm->all_reduce(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, op, ctx) == 0);
                            download(output, out_ptr, stream);
                        });
    }
}

// Communicator::init(BcastCallback) (include/megray/communicator.h:49, src/core/communicator.cpp:23-25): the group is
// formed through the caller's own broadcast - here a buffer in host memory that rank 0 fills and the others copy, the
// way the reference's NCCL backend hands its unique id to the callback (src/nccl/communicator.cpp:54-64) - with no
// bootstrap server anywhere; then an AllReduce as in test/test_opr.cpp:286-330.
void test_init_with_callback() {
    const int nranks = 4;
    const size_t len = 1000;
    std::vector<std::vector<float>> in(nranks, std::vector<float>(len)), out(nranks, std::vector<float>(len));
    for (size_t j = 0; j < len; j++) {
        float sum = 0;
        for (int i = 0; i < nranks; i++) in[i][j] = 0.25f * float((i + 1) * (j % 97 + 1));
        for (int i = 0; i < nranks; i++) sum += in[i][j];  // ranks 0..N-1; these values add exactly in any order
        for (int i = 0; i < nranks; i++) out[i][j] = sum;
    }
    std::mutex m;
    std::condition_variable cv;
    std::vector<char> id;
    std::vector<std::shared_ptr<Communicator>> comms(nranks);
    std::vector<std::vector<float>> got(nranks, std::vector<float>(len));
    for (int i = 0; i < nranks; i++) comms[i] = MegRay::get_communicator(nranks, i, MegRay::MEGRAY_VRANK);
    std::vector<std::thread> threads;
    for (int i = 0; i < nranks; i++)
        threads.emplace_back([&, i] {
            REQUIRE(hipSetDevice(0) == hipSuccess);
            const MegRay::Status st = comms[i]->init([&, i](char* data, size_t bytes) {
                std::unique_lock<std::mutex> lock(m);
                if (i == 0) {
                    id.assign(data, data + bytes);
                    cv.notify_all();
                } else {
                    cv.wait(lock, [&] { return !id.empty(); });
                    REQUIRE(id.size() == bytes);
                    std::memcpy(data, id.data(), bytes);
                }
            });
            REQUIRE(st == MegRay::MEGRAY_OK);
            hipStream_t stream;
            auto ctx = make_context(&stream);
            void* in_ptr = upload(in[i]);
            void* out_ptr = dev_alloc(len * sizeof(float));
            REQUIRE(comms[i]->all_reduce(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, MegRay::MEGRAY_SUM, ctx) == 0);
            download(got[i], out_ptr, stream);
        });
    for (auto& t : threads) t.join();
    for (int i = 0; i < nranks; i++) REQUIRE(std::memcmp(got[i].data(), out[i].data(), len * sizeof(float)) == 0);
    std::printf("ok   InitCallback\n");
}

void test_reduce_scatter() {  // test/test_opr.cpp:361-438
    const int nranks = 3;
    const size_t recvlen = 10;
    for (auto op : {MegRay::MEGRAY_SUM, MegRay::MEGRAY_MAX, MegRay::MEGRAY_MIN}) {
        std::vector<std::vector<float>> in(nranks, std::vector<float>(nranks * recvlen));
        std::vector<std::vector<float>> out(nranks, std::vector<float>(recvlen));
        for (int k = 0; k < nranks; k++)
            for (size_t j = 0; j < recvlen; j++) {
                size_t m = k * recvlen + j;
                for (int i = 0; i < nranks; i++) in[i][m] = 1.0f * (i + 1) * (m + 1);
                out[k][j] = fold(op, in, nranks, m);
            }
        std::string name = "ReduceScatter op=" + std::to_string(int(op));
        run_test<float>(name.c_str(), nranks, in, out,
                        [=](std::shared_ptr<Communicator> comm, int port, int, std::vector<float>& input,
                            std::vector<float>& output) {
                            enter_rank(comm, port);
                            hipStream_t stream;
                            auto ctx = make_context(&stream);
                            void* in_ptr = upload(input);
                            void* out_ptr = dev_alloc(recvlen * sizeof(float));
                            REQUIRE(comm->reduce_scatter(in_ptr, out_ptr, recvlen, MegRay::MEGRAY_FLOAT32, op, ctx) == 0);
                            download(output, out_ptr, stream);
                        });
    }
}

void test_broadcast_and_reduce() {  // test/test_opr.cpp:440-551
    const int nranks = 3, root = 1;
    const size_t len = 10;
    std::vector<std::vector<float>> in(nranks, std::vector<float>(len)), out(in);
    for (size_t j = 0; j < len; j++)
        for (int i = 0; i < nranks; i++) in[i][j] = 1.0f * (i + 1) * (j + 1);
    for (int i = 0; i < nranks; i++) out[i] = in[root];
    run_test<float>("Broadcast", nranks, in, out,
                    [=](std::shared_ptr<Communicator> comm, int port, int, std::vector<float>& input,
                        std::vector<float>& output) {
                        enter_rank(comm, port);
                        hipStream_t stream;
                        auto ctx = make_context(&stream);
                        void* in_ptr = upload(input);
                        void* out_ptr = dev_alloc(len * sizeof(float));
                        REQUIRE(comm->broadcast(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, root, ctx) == 0);
                        download(output, out_ptr, stream);
                    });
    for (auto op : {MegRay::MEGRAY_SUM, MegRay::MEGRAY_MAX, MegRay::MEGRAY_MIN}) {
        std::vector<std::vector<float>> want(nranks);
        want[root].resize(len);
        for (size_t j = 0; j < len; j++) want[root][j] = fold(op, in, nranks, j);
        std::string name = "Reduce op=" + std::to_string(int(op));
        run_test<float>(name.c_str(), nranks, in, want,
                        [=](std::shared_ptr<Communicator> comm, int port, int rank, std::vector<float>& input,
                            std::vector<float>& output) {
                            enter_rank(comm, port);
                            hipStream_t stream;
                            auto ctx = make_context(&stream);
                            void* in_ptr = upload(input);
                            void* out_ptr = reinterpret_cast<void*>(0x1);  // meaningless off the root (:501-505)
                            if (rank == root) out_ptr = dev_alloc(len * sizeof(float));
                            REQUIRE(comm->reduce(in_ptr, out_ptr, len, MegRay::MEGRAY_FLOAT32, op, root, ctx) == 0);
                            REQUIRE(hipStreamSynchronize(stream) == hipSuccess);
                            if (rank == root) download(output, out_ptr, stream);
                        });
    }
}

class FakeContext : public Context {
public:
    MegRay::ContextType type() const override { return MegRay::MEGRAY_CTX_CUDA; }
};

void test_errors() {
    // unknown backend: src/megray.cpp:56-57
    bool threw = false;
    try {
        MegRay::get_communicator(2, 0, MegRay::MEGRAY_NCCL);
    } catch (const MegRay::Exception& e) {
        threw = std::string(e.what()) == "unknown backend";
    }
    REQUIRE(threw);
    // unknown dtype: src/core/common.cpp:35-36
    threw = false;
    try {
        MegRay::get_dtype_size(MegRay::MEGRAY_DTYPE_COUNT);
    } catch (const MegRay::Exception& e) {
        threw = std::string(e.what()) == "unknown dtype";
    }
    REQUIRE(threw);
    // wrong context type: src/ucx/all_reduce.cpp:27-28
    int port = MegRay::get_free_port();
    REQUIRE(MegRay::create_server(1, port) == MegRay::MEGRAY_OK);
    auto comm = MegRay::get_communicator(1, 0, MegRay::MEGRAY_VRANK);
    REQUIRE(comm->init("localhost", port) == MegRay::MEGRAY_OK);
    void* buf = dev_alloc(64);
    threw = false;
    try {
        comm->all_reduce(buf, buf, 16, MegRay::MEGRAY_FLOAT32, MegRay::MEGRAY_SUM, std::make_shared<FakeContext>());
    } catch (const MegRay::Exception& e) {
        threw = std::string(e.what()) == "assertion failed";
    }
    REQUIRE(threw);
    // one rank is a valid group: all_reduce is a copy
    hipStream_t stream;
    auto ctx = make_context(&stream);
    std::vector<float> host{1, 2, 3, 4};
    void* in = upload(host);
    void* out = dev_alloc(16);
    REQUIRE(comm->all_reduce(in, out, 4, MegRay::MEGRAY_FLOAT32, MegRay::MEGRAY_SUM, ctx) == MegRay::MEGRAY_OK);
    std::vector<float> back(4);
    download(back, out, stream);
    REQUIRE(back == host);
    std::printf("ok   Errors\n");
}

}  // namespace

int main() {
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices < 1) {
        std::fprintf(stderr, "no GPU\n");
        return 2;
    }
    test_init();
    test_init_with_callback();
    test_send_recv();
    test_scatter_gather();
    test_all_to_all();
    test_all_gather();
    test_all_reduce();
    test_reduce_scatter();
    test_broadcast_and_reduce();
    test_errors();
    std::printf("all passed\n");
    return 0;
}
