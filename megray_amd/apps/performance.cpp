// megray_performance: the benchmark of the MegRay API for the MEGRAY_VRANK backend.
//
// Command line and table follow the reference's test/performance.cpp (options :443-496, table
// :342-362: bufsize / time(us) / speed(GB/s) / iters with speed = bufsize_bytes / avg_us / 1000, the
// per-rank payload over wall time), so numbers line up with anyone's MegRay runs.  Two columns are
// added: the HBM bytes the collective moves algorithmically per second, and that as a fraction of
// the 8 TB/s peak.  "-d" is the number of virtual ranks; all of them live on GPU 0 of this node,
// each driven by its own thread with its own stream, exactly like the reference's thread per device.
#include <hip/hip_runtime.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <functional>
#include <iomanip>
#include <iostream>
#include <memory>
#include <string>
#include <thread>
#include <vector>

#include "megray.h"
#include "megray_vrank.h"
#include "vrank_communicator.h"

namespace {

struct Arguments {
    std::string backends = "ALL";
    std::string master_ip = "127.0.0.1";
    int port = 2395;
    int n_nodes = 1;
    int node_rank = 0;
    int n_devs = 2;
    std::vector<size_t> sizes = {8, 1024, 512 * 1024, 1024 * 1024, 10 * 1024 * 1024};
    int send_dev = 0;
    int recv_dev = 1;
    int warmup_iters = 100;
    int iters = 100;
    std::string func_select = "ALL";
    size_t bufsize = 0, in_bufsize = 0, out_bufsize = 0;
    hipStream_t shared_stream = nullptr;  // -S: every rank enqueues on this one stream
    bool share = false;
    std::string json_path;  // -J: per-size results as JSON lines, with the spread of the per-call times
    bool random_fill = false;      // -R: inputs from the counter generator instead of zeros
    bool own_allocations = false;  // -M: every rank hipMallocs its own buffers, as the reference's harness does
    std::vector<void*> placed;     // otherwise: in buffers of ranks 0..N-1, then out buffers, in one allocation
};

// What rank 0's thread measured for one buffer size.
struct Timing {
    double avg_us = 0;     // wall time of all iterations including the final stream sync, per iteration
    double host_us = 0;    // the same without the final sync: what the calls cost the host, per iteration
    double drain_us = 0;   // the final stream sync: how far the device was behind the host when the last call returned
    // of the time from one call's return to the next call's return
    double median_us = 0, p90_us = 0, p99_us = 0, p999_us = 0, max_us = 0;
    uint64_t sleeps = 0;       // times a rank of the group went to sleep while waiting for the others (all iterations)
    uint64_t plans_built = 0;  // collectives that had to be planned (the rest came from the plan cache)
};

using Kernel = std::function<void(std::shared_ptr<MegRay::Communicator>, void*, void*, std::shared_ptr<MegRay::Context>)>;

struct Func {
    std::string name;
    int collective;  // MRV_* selector for the placement of the buffers (-1: none in particular)
    // buffer sizes per rank as multiples of bufsize (N = ranks), and HBM bytes moved per collective
    std::function<size_t(size_t, size_t)> in_bytes, out_bytes, hbm_bytes;
    std::function<Kernel(const Arguments&, int)> make;
};

#define CHECK_HIP(expr)                                                                    \
    do {                                                                                   \
        hipError_t e_ = (expr);                                                            \
        if (e_ != hipSuccess) {                                                            \
            std::fprintf(stderr, "hip error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__); \
            std::exit(1);                                                                  \
        }                                                                                  \
    } while (0)

// Inputs for -R: element i of rank r is uniform in [-1, 1), a pure function of (seed + r, i): the splitmix64 finaliser
// of ((seed + r) xor golden * i) + golden, its top 24 bits as float(u) * 2^-23 - 1.  All-zero buffers (what the
// reference's harness leaves in its buffers, test/performance.cpp:111) run a few points of the HBM peak faster
// than data.
__global__ void fill_uniform_kernel(float* p, uint64_t n, uint64_t key) {
    const uint64_t golden = 0x9E3779B97F4A7C15ull;
    for (uint64_t i = uint64_t(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += uint64_t(gridDim.x) * blockDim.x) {
        uint64_t z = (key ^ (i * golden)) + golden;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        p[i] = float(z >> 40) * (1.0f / 8388608.0f) - 1.0f;
    }
}

double now_us() {
    return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now().time_since_epoch()).count();
}

// worker() of test/performance.cpp:103-137
void worker(const Func& func, Arguments args, int dev, int port, Timing* res) {
    CHECK_HIP(hipSetDevice(0));
    hipStream_t stream = args.shared_stream;
    if (!args.share) CHECK_HIP(hipStreamCreate(&stream));
    auto context = MegRay::HipContext::make(stream);
    auto comm = MegRay::get_communicator(args.n_devs, dev, MegRay::MEGRAY_VRANK);
    if (comm->init(args.master_ip.c_str(), port) != MegRay::MEGRAY_OK) std::exit(1);
    void *in_ptr = nullptr, *out_ptr = nullptr;
    if (args.own_allocations) {
        CHECK_HIP(hipMalloc(&in_ptr, args.in_bufsize ? args.in_bufsize : 1));
        CHECK_HIP(hipMalloc(&out_ptr, args.out_bufsize ? args.out_bufsize : 1));
    } else {
        in_ptr = args.placed[size_t(dev)];
        out_ptr = args.placed[size_t(args.n_devs + dev)];
    }
    if (args.random_fill) {
        const uint64_t n = args.in_bufsize / 4;
        const uint64_t seed = 0x4D656752ull;  // "MegR"
        if (n) hipLaunchKernelGGL(fill_uniform_kernel, dim3(unsigned(std::min<uint64_t>((n + 255) / 256, 65536))), dim3(256), 0,
                                  stream, static_cast<float*>(in_ptr), n, seed + uint64_t(dev));
        CHECK_HIP(hipGetLastError());
        CHECK_HIP(hipStreamSynchronize(stream));
    } else {
        CHECK_HIP(hipMemset(in_ptr, 0, args.in_bufsize));
    }
    Kernel kernel = func.make(args, dev);
    for (int i = 0; i < args.warmup_iters; i++) kernel(comm, in_ptr, out_ptr, context);
    CHECK_HIP(hipStreamSynchronize(stream));
    std::vector<double> stamps;
    if (dev == 0) stamps.reserve(size_t(args.iters) + 1);
    const double t0 = now_us();
    if (dev == 0) stamps.push_back(t0);
    for (int i = 0; i < args.iters; i++) {
        kernel(comm, in_ptr, out_ptr, context);
        if (dev == 0) stamps.push_back(now_us());
    }
    const double t_issued = now_us();
    CHECK_HIP(hipStreamSynchronize(stream));
    const double t1 = now_us();
    if (args.own_allocations) {
        CHECK_HIP(hipFree(in_ptr));
        CHECK_HIP(hipFree(out_ptr));
    }
    if (!args.share) CHECK_HIP(hipStreamDestroy(stream));
    if (dev == 0) {
        std::vector<double> gaps;
        for (size_t i = 1; i < stamps.size(); ++i) gaps.push_back(stamps[i] - stamps[i - 1]);
        std::sort(gaps.begin(), gaps.end());
        const auto at = [&](double q) { return gaps[std::min(gaps.size() - 1, size_t(double(gaps.size()) * q))]; };
        res->avg_us = (t1 - t0) / args.iters;
        res->host_us = (t_issued - t0) / args.iters;
        res->drain_us = t1 - t_issued;
        res->median_us = at(0.5);
        res->p90_us = at(0.9);
        res->p99_us = at(0.99);
        res->p999_us = at(0.999);
        res->max_us = gaps.back();
        if (auto* vr = dynamic_cast<MegRay::VRankCommunicator*>(comm.get())) {
            const auto st = vr->stats();
            res->sleeps = st.sleeps;
            res->plans_built = st.plans_built;
        }
    }
}

Timing run_test(const Func& func, Arguments args) {
    Timing res;
    int port = MegRay::get_free_port();
    if (MegRay::create_server(args.n_devs, port) != MegRay::MEGRAY_OK) std::exit(1);
    void* base = nullptr;
    if (!args.own_allocations) {
        // all ranks' buffers in one allocation, at the distances the library recommends for buffers that
        // a collective walks through in step (the ranks share one HBM here)
        const size_t n = size_t(args.n_devs);
        std::vector<size_t> sizes(2 * n);
        for (size_t i = 0; i < n; ++i) {
            sizes[i] = args.in_bufsize ? args.in_bufsize : 1;
            sizes[n + i] = args.out_bufsize ? args.out_bufsize : 1;
        }
        args.placed.resize(2 * n);
        CHECK_HIP(hipSetDevice(0));
        std::vector<unsigned char> written(2 * n, 0);
        for (size_t i = 0; i < n; ++i) written[n + i] = 1;
        if (mrv_rank_buffers_alloc_for(func.collective, int(2 * n), sizes.data(), written.data(), args.placed.data(),
                                       &base) != 0) {
            std::fprintf(stderr, "mrv_rank_buffers_alloc_for: %s\n", mrv_last_error());
            std::exit(1);
        }
    }
    std::vector<std::thread> threads;
    for (int i = 0; i < args.n_devs; i++) threads.emplace_back(worker, std::cref(func), args, i, port, &res);
    for (auto& t : threads) t.join();
    if (base && mrv_rank_buffers_free(base) != 0) std::exit(1);
    return res;
}

std::vector<Func> all_funcs() {
    using A = const Arguments&;
    const auto f32 = MegRay::MEGRAY_FLOAT32;
    auto one = [](size_t b, size_t) { return b; };
    auto all = [](size_t b, size_t n) { return b * n; };
    std::vector<Func> f;
    f.push_back({"send_recv", -1, one, one, [](size_t b, size_t) { return 2 * b; }, [=](A a, int dev) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         if (dev == a.send_dev) comm->send(in, a.bufsize / 4, f32, a.recv_dev, ctx);
                         if (dev == a.recv_dev) comm->recv(out, a.bufsize / 4, f32, a.send_dev, ctx);
                     };
                 }});
    f.push_back({"all_reduce_sum", MRV_ALL_REDUCE, one, one, [](size_t b, size_t n) { return 2 * n * b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->all_reduce(in, out, a.bufsize / 4, f32, MegRay::MEGRAY_SUM, ctx);
                     };
                 }});
    f.push_back({"scatter", MRV_SCATTER, all, one, [](size_t b, size_t n) { return 2 * n * b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->scatter(in, out, a.bufsize / 4, f32, 0, ctx);
                     };
                 }});
    f.push_back({"gather", MRV_GATHER, one, all, [](size_t b, size_t n) { return 2 * n * b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->gather(in, out, a.bufsize / 4, f32, 0, ctx);
                     };
                 }});
    f.push_back({"all_to_all", MRV_ALL_TO_ALL, all, all, [](size_t b, size_t n) { return 2 * n * n * b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->all_to_all(in, out, a.bufsize / 4, f32, ctx);
                     };
                 }});
    f.push_back({"all_gather", MRV_ALL_GATHER, one, all, [](size_t b, size_t n) { return n * b + n * n * b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->all_gather(in, out, a.bufsize / 4, f32, ctx);
                     };
                 }});
    f.push_back({"reduce_scatter_sum", MRV_REDUCE_SCATTER, all, one, [](size_t b, size_t n) { return n * n * b + n * b; },
                 [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->reduce_scatter(in, out, a.bufsize / 4, f32, MegRay::MEGRAY_SUM, ctx);
                     };
                 }});
    f.push_back({"broadcast", MRV_BROADCAST, one, one, [](size_t b, size_t n) { return b + n * b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->broadcast(in, out, a.bufsize / 4, f32, 0, ctx);
                     };
                 }});
    f.push_back({"reduce_sum", MRV_REDUCE, one, one, [](size_t b, size_t n) { return n * b + b; }, [=](A a, int) -> Kernel {
                     return [=](auto comm, void* in, void* out, auto ctx) {
                         comm->reduce(in, out, a.bufsize / 4, f32, MegRay::MEGRAY_SUM, 0, ctx);
                     };
                 }});
    return f;
}

void show_help(const char* argv0) {
    std::cout << argv0
              << " {OPTIONS}\n\n    Benchmark of the MegRay API on the MEGRAY_VRANK backend.\n\n  OPTIONS:\n"
                 "      -h          this help\n"
                 "      -d[int]     number of devs = virtual ranks on GPU 0 (default 2, at most 32)\n"
                 "      -I[string]  master IP (default 127.0.0.1)\n"
                 "      -P[int]     master port (accepted; every run draws a free port)\n"
                 "      -n[int]     number of nodes: only 1 (all ranks share one GPU)\n"
                 "      -r[int]     rank of node: only 0\n"
                 "      -e[string]  backend: ALL or VRANK\n"
                 "      -f[string]  function: ALL, all_reduce, send_recv, scatter, gather, all_to_all,\n"
                 "                  all_gather, reduce_scatter, broadcast, reduce\n"
                 "      -s[int,..]  packet size(s) in bytes per rank (default: 8, 1 KiB, 512 KiB, 1 MiB, 10 MiB)\n"
                 "      -w[int]     warm-up iterations (default 100)\n"
                 "      -i[int]     timed iterations (default 100)\n"
                 "      -J[path]    also append one JSON line per size to this file: average, median, 90 / 99 / 99.9th\n"
                 "                  percentile and maximum of the per-call time on rank 0, the final stream sync, and the\n"
                 "                  group's sleep and planning counts (not in the reference's harness)\n"
                 "      -R          fill the inputs with uniform random fp32 in [-1, 1) from a counter generator (seed + rank)\n"
                 "                  instead of zeros; the table is the same\n"
                 "      -M          every rank allocates its own buffers with hipMalloc, as the reference's harness\n"
                 "                  does; without it all buffers lie in one allocation, placed by the library for the\n"
                 "                  collective at hand (mrv_rank_buffers_alloc_for)\n"
                 "      -S          all ranks enqueue on ONE stream (not in the reference's harness: its ranks\n"
                 "                  are devices); without it every rank has a stream of its own\n"
                 "      -A -B       send/recv: sending node rank / dev (default 0 / 0)\n"
                 "      -C -D       send/recv: receiving node rank / dev (default 0 / 1)\n\n"
                 "    example: "
              << argv0 << " -d 8 -f all_reduce -s 1073741824 -w 5 -i 20\n";
}

template <typename T>
void print(T value) {
    std::cout << std::setw(16) << value;
}

}  // namespace

int main(int argc, char* argv[]) {
    Arguments args;
    int ch;
    while ((ch = getopt(argc, argv, "hSMRd:I:P:n:r:e:f:s:w:i:A:B:C:D:J:")) != EOF) {
        switch (ch) {
            case 'h': show_help(argv[0]); return 0;
            case 'S': args.share = true; break;
            case 'M': args.own_allocations = true; break;
            case 'R': args.random_fill = true; break;
            case 'J': args.json_path = optarg; break;
            case 'd': args.n_devs = std::atoi(optarg); break;
            case 'I': args.master_ip = optarg; break;
            case 'P': args.port = std::atoi(optarg); break;
            case 'n': args.n_nodes = std::atoi(optarg); break;
            case 'r': args.node_rank = std::atoi(optarg); break;
            case 'e': args.backends = optarg; break;
            case 'f': args.func_select = optarg; break;
            case 's': {  // one size, or several separated by commas
                args.sizes.clear();
                for (const char* p = optarg; *p;) {
                    char* end = nullptr;
                    args.sizes.push_back(size_t(std::strtoull(p, &end, 10)));
                    if (end == p) { std::cerr << "Error arguments\n"; return 1; }
                    p = *end == ',' ? end + 1 : end;
                }
                break;
            }
            case 'w': args.warmup_iters = std::atoi(optarg); break;
            case 'i': args.iters = std::atoi(optarg); break;
            case 'A': break;  // node ranks of the send/recv pair: one node only
            case 'C': break;
            case 'B': args.send_dev = std::atoi(optarg); break;
            case 'D': args.recv_dev = std::atoi(optarg); break;
            default: std::cerr << "Error arguments\n"; show_help(argv[0]); return 1;
        }
    }
    if (args.n_nodes != 1 || args.node_rank != 0) {
        std::cerr << "the vrank backend keeps all ranks on one GPU of one node: use -n 1 -r 0\n";
        return 1;
    }
    if (args.backends != "ALL" && args.backends != "VRANK") {
        std::cerr << "this build has one backend: VRANK\n";
        return 1;
    }
    if (args.n_devs < 1 || args.n_devs > 32 || args.iters < 1) {
        std::cerr << "need 1 <= -d <= 32 and -i >= 1\n";
        return 1;
    }
    int devices = 0;
    if (hipGetDeviceCount(&devices) != hipSuccess || devices < 1) {
        std::cerr << "no GPU\n";
        return 2;
    }
    if (args.share) {
        CHECK_HIP(hipSetDevice(0));
        CHECK_HIP(hipStreamCreate(&args.shared_stream));
    }
    std::ofstream json;
    if (!args.json_path.empty()) {
        json.open(args.json_path, std::ios::app);
        if (!json) {
            std::cerr << "cannot write " << args.json_path << "\n";
            return 1;
        }
    }
    const std::string want = args.func_select;
    for (const Func& func : all_funcs()) {
        if (want != "ALL" && func.name.rfind(want, 0) != 0) continue;
        if (func.name == "send_recv" && (args.n_devs < 2 || args.send_dev == args.recv_dev)) continue;
        std::cout << "\nTesting " << func.name << " on backend VRANK (" << args.n_devs << " virtual ranks)\n";
        print("bufsize");
        print("time(us)");
        print("speed(GB/s)");
        print("iters");
        print("hbm(GB/s)");
        print("hbm(%peak)");
        std::cout << std::endl;
        for (size_t size : args.sizes) {
            Arguments run = args;
            run.bufsize = size / 4 * 4;
            run.in_bufsize = func.in_bytes(run.bufsize, args.n_devs);
            run.out_bufsize = func.out_bytes(run.bufsize, args.n_devs);
            const Timing timing = run_test(func, run);
            const double avg_us = timing.avg_us;
            if (json.is_open()) {
                json << "{\"func\": \"" << func.name << "\", \"ranks\": " << args.n_devs << ", \"bufsize\": " << size
                     << ", \"streams\": \"" << (args.share ? "shared" : "own") << "\", \"iters\": " << args.iters
                     << ", \"fill\": \"" << (args.random_fill ? "random" : "zeros") << "\", \"buffers\": \""
                     << (args.own_allocations ? "own" : "placed") << "\", \"avg_us\": " << timing.avg_us
                     << ", \"host_us\": " << timing.host_us << ", \"drain_us\": " << timing.drain_us
                     << ", \"median_us\": " << timing.median_us << ", \"p90_us\": " << timing.p90_us
                     << ", \"p99_us\": " << timing.p99_us << ", \"p999_us\": " << timing.p999_us
                     << ", \"max_us\": " << timing.max_us << ", \"sleeps\": " << timing.sleeps
                     << ", \"plans_built\": " << timing.plans_built << "}" << std::endl;
            }
            double hbm = func.hbm_bytes(run.bufsize, args.n_devs) / avg_us / 1000.0;
            print(size);
            print(avg_us);
            print(1.0 * size / avg_us / 1000);
            print(args.iters);
            print(hbm);
            print(hbm / 80.0);
            std::cout << std::endl;
        }
    }
    return 0;
}
