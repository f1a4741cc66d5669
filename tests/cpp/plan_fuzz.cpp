// Random calls into the host planner, built with the host sanitizers (address, undefined): the planner is
// pure host code, so what it does with odd lengths, offsets and rank counts can be checked without a GPU.
// For every plan it returns, every launch descriptor must keep the kernels inside the callers' buffers:
//   - flat launches: runs tile [0, count) in order, outputs stay inside the output buffers, the tile count
//     is what the kernel's grid covers;
//   - general launches: every segment lies inside the input and output buffers, the tile table is the running
//     sum of the segments' tiles;
//   - pack launches: slices of a copy's tiles cover every tile once, block copies stay inside the buffers;
//   - one-pass plans (fused all_reduce, reduce_scatter, reduce) write every output element exactly once.
// Usage: plan_fuzz [cases] [seed]; prints "ok <cases> plans" or the first violated invariant.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <random>
#include <vector>

#include "vrank_plan.h"

using namespace MegRay;
using namespace MegRay::vrank;

namespace {

std::mt19937_64 rng;
uint64_t below(uint64_t n) { return n ? rng() % n : 0; }

[[noreturn]] void fail(const char* what, const char* where) {
    std::printf("FAILED: %s (%s)\n", what, where);
    std::exit(1);
}
#define CHECK(cond, where) \
    do {                   \
        if (!(cond)) fail(#cond, where); \
    } while (0)

struct Buffers {
    const void* send[kMaxRanks] = {};
    void* recv[kMaxRanks] = {};
    uint64_t send_elems = 0, recv_elems = 0;
};

// Synthetic addresses (never dereferenced): buffers far apart, at offsets drawn the way callers' views are.
Buffers make_buffers(uint32_t nranks, uint32_t elem, uint64_t send_elems, uint64_t recv_elems, bool inplace) {
    Buffers b;
    b.send_elems = send_elems;
    b.recv_elems = recv_elems;
    const int mode = int(below(5));
    const uint64_t common = below(2048 / elem) * elem;
    for (uint32_t r = 0; r < nranks; ++r) {
        auto offset = [&]() -> uint64_t {
            if (mode == 0 || mode == 1) return 0;
            if (mode == 2) return common % 16;
            if (mode == 3) return below(16 / elem ? 16 / elem : 1) * elem;
            return below(2048 / elem) * elem;
        };
        const uint64_t base = (uint64_t(r) + 1) << 40;
        b.send[r] = reinterpret_cast<const void*>(base + offset());
        b.recv[r] = inplace ? const_cast<void*>(b.send[r]) : reinterpret_cast<void*>(base + (uint64_t(1) << 39) + offset());
    }
    return b;
}

uint64_t draw_len() {
    switch (below(6)) {
        case 0: return below(40);
        case 1: return below(5000);
        case 2: return below(3000000);
        case 3: return (uint64_t(1) << (10 + below(20))) + below(7) - 3;
        case 4: return uint64_t(kThreads) * 16 * below(5000) + below(3);
        default: return below(uint64_t(1) << 33);
    }
}

// Per destination rank: how often each output interval is written.  Intervals are kept as +1 / -1 edges.
struct Coverage {
    std::map<uint64_t, int64_t> edges[kMaxRanks];
    void add(uint32_t rank, uint64_t begin, uint64_t count) {
        if (!count) return;
        edges[rank][begin] += 1;
        edges[rank][begin + count] -= 1;
    }
    // every element of [0, n) of `rank` written exactly once and nothing outside
    bool exact(uint32_t rank, uint64_t n) const {
        int64_t depth = 0;
        uint64_t at = 0;
        for (const auto& e : edges[rank]) {
            if (e.second == 0) continue;
            if (depth == 0 && e.first != at) return false;   // a gap (or a start beyond 0)
            depth += e.second;
            if (depth > 1 || depth < 0) return false;        // written twice
            at = e.first;
        }
        return depth == 0 && at == n;
    }
    bool empty(uint32_t rank) const {
        for (const auto& e : edges[rank])
            if (e.second) return false;
        return true;
    }
};

void check_steps(const Plan& plan, const Buffers& b, uint32_t nranks, uint32_t elem, Coverage* cov, const char* where) {
    for (const Step& step : plan.steps) {
        if (step.kind == Step::kFlat) {
            const FlatLaunch& L = step.flat;
            CHECK(L.nranks == nranks && L.nruns >= 1 && L.nruns <= kMaxFlatRuns, where);
            CHECK(L.count <= b.send_elems, where);
            CHECK(L.elem_size == elem, where);
            const uint64_t tile = uint64_t(kThreads) * (kVecBytes / elem);
            CHECK(L.total_tiles == (L.count + tile - 1) / tile, where);
            CHECK(L.waves == 1 || L.waves == kGroupWaves, where);
            uint64_t begin = 0;
            for (uint32_t i = 0; i < L.nruns; ++i) {
                CHECK(L.end[i] >= begin && L.end[i] <= L.count, where);
                CHECK(L.shift[i] <= begin || L.end[i] == begin, where);
                const uint64_t n = L.end[i] - begin, out_begin = begin - (n ? L.shift[i] : 0);
                CHECK(out_begin + n <= b.recv_elems, where);
                const uint32_t out_first = (L.meta[i] >> 16) & 0xffu, start = L.meta[i] & 0xffu;
                CHECK(start < nranks && out_first < nranks && L.nout >= 1 && L.nout <= nranks, where);
                if (cov)
                    for (uint32_t m = 0; m < L.nout; ++m) cov->add((out_first + m) % nranks, out_begin, n);
                begin = L.end[i];
            }
            CHECK(begin == L.count, where);
            for (uint32_t i = L.nruns; i < kMaxFlatRuns; ++i) CHECK(L.end[i] == 0, where);  // the kernel scans in eights
        } else if (step.kind == Step::kFold) {
            const FoldLaunch& L = step.fold;
            CHECK(L.nseg >= 1 && L.nseg <= kMaxSegments, where);
            CHECK(L.nfold >= 1 && L.nfold <= nranks && L.nout >= 1 && L.nout <= nranks, where);
            CHECK(L.waves == 1 || L.waves == kGroupWaves, where);
            uint64_t tiles = 0;
            for (uint32_t s = 0; s < L.nseg; ++s) {
                const FoldSegment& sg = L.seg[s];
                CHECK(sg.count > 0, where);
                CHECK(sg.in_begin + sg.count <= b.send_elems || sg.in_begin + sg.count <= b.recv_elems, where);
                CHECK(sg.out_begin + sg.count <= b.recv_elems, where);
                CHECK(sg.start < nranks && sg.out_first < nranks && (sg.dir == 1 || sg.dir == -1), where);
                CHECK(L.first_tile[s] == tiles, where);
                if (sg.flags & kSegVector) CHECK(sg.count % (kVecBytes / elem) == 0 || L.waves == 1, where);
                tiles += segment_tiles(L, sg.flags & kSegVector, sg.count);
                CHECK(tiles <= 0x7fffffffull, where);
                if (cov)
                    for (uint32_t m = 0; m < L.nout; ++m) cov->add((sg.out_first + m) % nranks, sg.out_begin, sg.count);
            }
            CHECK(L.total_tiles == tiles, where);
        } else if (step.kind == Step::kTree) {
            const TreeLaunch& L = step.tree;
            CHECK(L.count <= b.send_elems && L.count <= b.recv_elems && L.root < nranks, where);
            // a lane takes a whole vector, or one element; the elements behind the last whole vector are the
            // work of the last workgroup's first lanes, so there is always at least one workgroup
            const uint64_t lanes = L.vector ? L.count / (kVecBytes / elem) : L.count;
            CHECK(uint64_t(L.total_tiles) * kThreads >= lanes && L.total_tiles >= 1, where);
            CHECK((uint64_t(L.total_tiles) - 1) * kThreads < (lanes ? lanes : 1), where);
            if (cov) cov->add(L.root, 0, L.count);
        } else {
            const PackLaunch& L = step.pack;
            CHECK(L.ncopies >= 1 && L.block_bytes > 0, where);
            CHECK(L.first_tile + L.tiles_per_copy <= pack_tiles(L.block_bytes), where);
            CHECK(L.waves == 1 || L.waves == kGroupWaves, where);
            if (L.waves == kGroupWaves) {
                CHECK(L.first_tile % (uint64_t(kGroupWaves) * kGroupStride) == 0, where);
                CHECK(L.groups_per_copy == group_grid(L.tiles_per_copy), where);
                CHECK(uint64_t(L.ncopies) * L.groups_per_copy <= 0x7fffffffull, where);
            } else {
                CHECK(uint64_t(L.ncopies) * L.tiles_per_copy <= 0x7fffffffull, where);
            }
            CHECK(L.width == 16 || L.width == 8 || L.width == 4 || L.width == 2 || L.width == 1, where);
            CHECK(L.block_bytes % L.width == 0, where);
        }
    }
}

// the slices of a block copy's tiles, over the pack launches of a plan, cover every tile once
void check_pack_slices(const Plan& plan, const char* where) {
    uint64_t next = 0, tiles = 0;
    for (const Step& step : plan.steps) {
        if (step.kind != Step::kPack) continue;
        tiles = pack_tiles(step.pack.block_bytes);
        CHECK(step.pack.first_tile == next, where);
        next += step.pack.tiles_per_copy;
    }
    CHECK(next == tiles, where);
}

}  // namespace

int main(int argc, char** argv) {
    const long cases = argc > 1 ? std::atol(argv[1]) : 20000;
    rng.seed(argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 20240611ull);
    const uint32_t elems[] = {1, 2, 4, 8};
    long planned = 0;
    for (long c = 0; c < cases; ++c) {
        const uint32_t nranks = 1 + uint32_t(below(kMaxRanks));
        const uint32_t elem = elems[below(4)];
        const int kind = int(below(8));
        const FoldOrder order = FoldOrder(below(kOrderCount));
        const Schedule sched = Schedule(below(kSchedCount));
        uint64_t len = draw_len();
        if (below(4) == 0) len /= nranks;
        const uint32_t root = uint32_t(below(nranks));
        char where[200];
        std::snprintf(where, sizeof(where), "case %ld kind %d nranks %u elem %u len %" PRIu64 " order %d sched %d root %u", c,
                      kind, nranks, elem, len, int(order), int(sched), root);
        Plan plan;
        Status st;
        Coverage cov;
        if (kind == 0) {  // all_reduce
            const Buffers b = make_buffers(nranks, elem, len, len, below(4) == 0);
            st = plan_all_reduce(plan, b.send, b.recv, nranks, len, elem, order, sched);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, sched == kSchedFused ? &cov : nullptr, where);
            if (sched == kSchedFused)
                for (uint32_t r = 0; r < nranks; ++r) CHECK(cov.exact(r, len), where);
        } else if (kind == 1) {  // reduce_scatter
            const Buffers b = make_buffers(nranks, elem, len * nranks, len, false);
            st = plan_reduce_scatter(plan, b.send, b.recv, nranks, len, elem, order, kSchedFused);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, &cov, where);
            for (uint32_t r = 0; r < nranks; ++r) CHECK(cov.exact(r, len), where);
        } else if (kind == 2) {  // reduce to a root
            const Buffers b = make_buffers(nranks, elem, len, len, false);
            st = plan_reduce(plan, b.send, b.recv[root], nranks, len, elem, order, root);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, &cov, where);
            for (uint32_t r = 0; r < nranks; ++r) CHECK(r == root ? cov.exact(r, len) : cov.empty(r), where);
        } else if (kind == 3) {
            const Buffers b = make_buffers(nranks, elem, len, len * nranks, false);
            st = plan_all_gather(plan, b.send, b.recv, nranks, len, elem);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, nullptr, where);
            check_pack_slices(plan, where);
        } else if (kind == 4) {
            const Buffers b = make_buffers(nranks, elem, len * nranks, len * nranks, false);
            st = plan_all_to_all(plan, b.send, b.recv, nranks, len, elem);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, nullptr, where);
            check_pack_slices(plan, where);
        } else if (kind == 5) {
            const Buffers b = make_buffers(nranks, elem, len * nranks, len, false);
            st = plan_scatter(plan, b.send[root], b.recv, nranks, len, elem, root);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, nullptr, where);
            check_pack_slices(plan, where);
        } else if (kind == 6) {
            const Buffers b = make_buffers(nranks, elem, len, len * nranks, false);
            st = plan_gather(plan, b.send, b.recv[root], nranks, len, elem, root);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, nullptr, where);
            check_pack_slices(plan, where);
        } else {
            const Buffers b = make_buffers(nranks, elem, len, len, false);
            st = plan_broadcast(plan, b.send[root], b.recv, nranks, len, elem, root);
            if (st != MEGRAY_OK) continue;
            check_steps(plan, b, nranks, elem, nullptr, where);
            check_pack_slices(plan, where);
        }
        ++planned;
    }
    std::printf("ok %ld plans of %ld cases\n", planned, cases);
    return 0;
}
