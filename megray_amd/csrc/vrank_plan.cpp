#include "vrank_plan.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace MegRay {
namespace vrank {

// propagate a planner error without logging: the caller reports it
#define PLAN_TRY(expr)                              \
    do {                                            \
        Status plan_status_ = (expr);               \
        if (plan_status_ != MEGRAY_OK) return plan_status_; \
    } while (0)

namespace {

thread_local char g_plan_error[256] = "";

Status invalid(const char* what) {
    std::snprintf(g_plan_error, sizeof(g_plan_error), "%s", what);
    return MEGRAY_INVALID_ARGUMENT;
}

// MEGRAY_VRANK_PACE in the environment overrides the planner's choice of which group launches pace their accesses
// (kFlatPaced): "always", "never"; anything else leaves it to paced_launch().
int pace_override() {
    const char* text = std::getenv("MEGRAY_VRANK_PACE");  // read at every planning: tests switch it
    if (text && std::strcmp(text, "always") == 0) return 1;
    if (text && std::strcmp(text, "never") == 0) return 0;
    return -1;
}

// MEGRAY_VRANK_KEEP in the environment overrides set_store_policy(): "always", "never".
int keep_override() {
    const char* text = std::getenv("MEGRAY_VRANK_KEEP");  // read at every planning: tests switch it
    if (text && std::strcmp(text, "always") == 0) return 1;
    if (text && std::strcmp(text, "never") == 0) return 0;
    return -1;
}

// Should a flat group launch over these buffers (`bytes` each) keep two loads and two stores per wavefront in flight
// instead of all of them?  Pacing costs a short launch latency and gains a long one bandwidth, the more the worse
// the buffers lie relative to each other.  Measured on MI355X, fp32 SUM all_reduce, % of the HBM peak, all at once ->
// paced, per-rank buffer sizes 64 MiB / 128 MiB / 256 MiB / 512 MiB / 1 GiB:
//   8 ranks, separate allocations (1 GiB + 2 MiB apart)   80.6 -> 80.1 / 81.6 -> 81.7 / 80.2 -> 82.9 / 77.0 -> 81.1 / 78.3 -> 82.0
//   8 ranks, placed an odd multiple of 128 MiB apart       82.4 -> 81.0 / 84.6 -> 83.0 / 83.9 -> 82.9 / 82.8 -> 82.7 / 82.8 -> 83.1
//   4 ranks, separate allocations                          80.8 -> 81.2 / 82.6 -> 82.2 / 82.8 -> 82.9 / 80.1 -> 82.9 / 80.7 -> 83.8
//   4 ranks, placed                                        81.4 -> 81.2 / 83.5 -> 83.0 / 84.1 -> 84.0 / 84.1 -> 84.0 / 84.0 -> 83.1
//   3 ranks, separate allocations                          79.7 -> 80.4 / 83.4 -> 83.3 / 84.0 -> 83.7 / 82.1 -> 83.5 / 81.8 -> 84.2
// So: buffers that do not lie the way vrank_placement.h lays them out pace from 3 GiB over all of them; buffers
// that do, never (8 ranks x 1 GiB placed, interleaved in one process on three boxes: 84.2 -> 84.0, 83.7 -> 83.2, 83.4 -> 82.6).
// The general group kernel (other rank counts, buffers off the 16-byte grid) behaves alike on separate allocations
// (5 / 7 / 12 / 16 ranks x 512 MiB: 79.4 -> 82.9 / 79.2 -> 81.3 / 76.4 -> 79.3 / 74.8 -> 78.3; x 256 MiB + 1 throughout;
// x 64 MiB - 1) and loses half a point to a point on placed buffers, where it is left alone (`flat` false) - unless
// it folds into ONE output (`nout` 1: a reduce_scatter of 3, 5, 6, 7, 9 ... ranks, whose blocks start off the tile
// grid).  That shape gains wherever the buffers lie, placed / separate, per-rank buffers of 32 / 128 / 512 MiB:
//   5 ranks   75.6 -> 74.8 / 75.7 -> 74.3     79.1 -> 82.6 / 79.1 -> 82.6     79.9 -> 85.0 / 79.7 -> 84.6
//   6 ranks   76.7 -> 77.7 / 75.2 -> 76.3     78.1 -> 80.9 / 78.3 -> 80.8     79.8 -> 82.2 / 79.5 -> 81.2
//   7 ranks   74.4 -> 76.0 / 73.1 -> 76.6     77.8 -> 81.1 / 77.8 -> 81.2     79.4 -> 81.8 / 79.2 -> 81.3
// (3 / 10 / 12 ranks x 256 MiB placed: 81.0 -> 83.2 / 78.0 -> 81.0 / 77.4 -> 81.1; 16 ranks 83.4 -> 83.5), and paces from
// 1 GiB over all its buffers.
bool paced_launch(const void* const* in, const void* const* out, uint32_t nranks, uint64_t bytes, bool flat = true,
                  uint32_t nout = 0) {
    if (pace_override() >= 0) return pace_override() == 1;
    const void* seen[2 * kMaxRanks];
    uint32_t n = 0;
    for (uint32_t pass = 0; pass < 2; ++pass) {
        for (uint32_t r = 0; r < nranks; ++r) {
            const void* p = pass ? out[r] : in[r];
            bool known = p == nullptr;
            for (uint32_t i = 0; i < n && !known; ++i) known = seen[i] == p;
            if (!known) seen[n++] = p;
        }
    }
    // placed: all starts at the same offset within 128 MiB and pairwise different in address bits 27 - 31
    constexpr uintptr_t kUnit = uintptr_t(128) << 20;
    bool placed = n > 0;
    uint32_t keys = 0;
    for (uint32_t i = 0; i < n && placed; ++i) {
        const uintptr_t a = reinterpret_cast<uintptr_t>(seen[i]);
        const uint32_t key = uint32_t((a / kUnit) % 32);
        placed = (a % kUnit) == (reinterpret_cast<uintptr_t>(seen[0]) % kUnit) && !(keys >> key & 1u);
        keys |= 1u << key;
    }
    const uint64_t total = uint64_t(n) * bytes;
    constexpr uint64_t kGiB = uint64_t(1) << 30;
    if (!flat && nout == 1 && total >= kGiB) return true;
    return !placed && total >= 3 * kGiB;
}

bool overlaps(const void* a, uint64_t a_bytes, const void* b, uint64_t b_bytes) {
    if (!a || !b || !a_bytes || !b_bytes) return false;
    const uintptr_t a0 = reinterpret_cast<uintptr_t>(a), b0 = reinterpret_cast<uintptr_t>(b);
    return a0 < b0 + b_bytes && b0 < a0 + a_bytes;
}

// Collects runs of elements (one fold order, one destination set each) and turns them into
// launches: one flat launch where the runs tile a buffer in order and everything is vector aligned,
// general launches (runs split into an unaligned head, a body of whole 16-byte vectors and a tail,
// a new launch whenever a descriptor fills up) otherwise.
class FoldBuilder {
public:
    FoldBuilder(Plan& plan, const void* const* in, void* const* out, uint32_t nranks, uint32_t nfold,
                uint32_t nout, uint32_t elem_size, bool new_wins)
            : m_plan(plan), m_nranks(nranks), m_nfold(nfold), m_nout(nout), m_elem(elem_size),
              m_new_wins(new_wins) {
        // Vector access needs every buffer at the same offset from a 16-byte boundary (usually 0; a
        // common non-zero offset, in whole elements, only lengthens the scalar head of each run).
        // m_grid is the largest power of two up to one tile (1 KiB) modulo which all buffers still
        // agree: vector bodies start on that grid so that neighbouring wavefronts do not share
        // cache lines.
        uintptr_t differ = 0, first_ptr = 0;
        bool first = true;
        for (uint32_t r = 0; r < kMaxRanks; ++r) {
            m_in[r] = r < nranks ? in[r] : nullptr;
            m_out[r] = r < nranks ? out[r] : nullptr;
            for (const void* p : {m_in[r], static_cast<const void*>(m_out[r])}) {
                if (!p) continue;  // unused slot
                if (first) {
                    first_ptr = reinterpret_cast<uintptr_t>(p);
                    first = false;
                }
                differ |= first_ptr ^ reinterpret_cast<uintptr_t>(p);
            }
        }
        m_grid = kThreads * kVecBytes;
        while (m_grid > 1 && (differ & (m_grid - 1))) m_grid >>= 1;
        m_aligned = m_grid >= kVecBytes;
        m_misalign = uint32_t(first_ptr & (m_grid - 1));  // offset of every base from the grid
        if (m_misalign % elem_size) m_aligned = false;
        // Buffers whose offsets from a 16-byte boundary differ: the 128-bit accesses of gfx950 need
        // 4-byte alignment only, so element types of 4 and 8 bytes (in naturally aligned buffers)
        // still go 16 bytes per lane, every buffer at its own alignment.  Narrower types do not.
        // 1- and 2-byte elements go 16 bytes per lane as well (m_bytes), through the segment kernels only, whose
        // tiles may start at any byte address.
        if (!m_aligned) {
            bool natural = true;
            for (uint32_t r = 0; r < kMaxRanks; ++r)
                for (const void* p : {m_in[r], static_cast<const void*>(m_out[r])})
                    if (p && reinterpret_cast<uintptr_t>(p) % elem_size) natural = false;
            m_plain = natural && elem_size >= 4;
            m_bytes = natural && elem_size < 4;
        }
    }

    void add_run(uint64_t in_begin, uint64_t out_begin, uint64_t count, uint8_t start, int8_t dir,
                 uint8_t out_first) {
        if (!count) return;
        m_plan.bytes_read += count * m_elem * m_nfold;
        m_plan.bytes_written += count * m_elem * m_nout;
        m_runs.push_back(Run{in_begin, out_begin, count, start, dir, out_first});
    }

    void finish() {
        if (m_runs.empty()) return;
        if (!emit_flat()) emit_general();
        m_runs.clear();
    }

    // Tree combination towards rank `root` of one whole buffer: a flat launch if the shape allows.
    bool finish_tree(uint64_t count, uint8_t root) {
        add_run(0, 0, count, root, 1, root);
        m_tree = true;
        const bool ok = emit_flat();
        m_runs.clear();
        return ok;
    }

private:
    struct Run {
        uint64_t in_begin, out_begin, count;
        uint8_t start;
        int8_t dir;
        uint8_t out_first;
    };

    // Do tiles that start on the buffers' common grid cover whole cache lines of every buffer, inputs and outputs
    // (which lie `shift_bytes` before the inputs)?
    bool lines_shared(uint64_t shift_bytes) const {
        constexpr uint64_t kLine = 128;
        return m_aligned && m_grid >= kLine && shift_bytes % kLine == 0;
    }

    // The flat kernel folds exactly nranks inputs with the rank count known at compile time.
    static bool flat_width(uint32_t n) { return n == 2 || n == 3 || n == 4 || n == 8; }

    bool emit_flat() {
        const bool vectors = m_plain || (m_aligned && (m_misalign & (kVecBytes - 1)) == 0);
        if (!vectors || m_nfold != m_nranks || !flat_width(m_nranks) || m_runs.size() > kMaxFlatRuns) return false;
        const uint64_t epv = kVecBytes / m_elem;
        const uint64_t tile = uint64_t(kThreads) * epv;  // elements per tile
        uint64_t expect = 0;
        for (const Run& r : m_runs) {
            if (r.in_begin != expect) return false;  // runs must tile [0, count) in order
            if (r.out_begin > r.in_begin || (r.in_begin - r.out_begin) % epv) return false;
            expect = r.in_begin + r.count;
        }
        const uint64_t total = (expect + tile - 1) / tile;
        if (total > 0x7fffffffull) return false;
        Step step;
        std::memset(&step, 0, sizeof(step));
        step.kind = Step::kFlat;
        FlatLaunch& L = step.flat;
        for (uint32_t r = 0; r < kFlatMaxRanks; ++r) {  // flat_width(): at most eight ranks
            L.in[r] = m_in[r];
            L.out[r] = m_out[r];
        }
        for (size_t i = 0; i < m_runs.size(); ++i) {
            const Run& r = m_runs[i];
            L.end[i] = r.in_begin + r.count;
            L.meta[i] = flat_meta(r.start, r.dir, r.out_first);
            L.shift[i] = r.in_begin - r.out_begin;
        }
        L.count = expect;
        L.nranks = m_nranks;
        L.nout = m_nout;
        L.nruns = uint32_t(m_runs.size());
        L.total_tiles = uint32_t(total);
        L.new_wins_ties = m_new_wins ? 1 : 0;
        L.elem_size = m_elem;
        L.tree = m_tree ? 1 : 0;
        // launches of many tiles take the group form; all_reduce shapes (every rank an output, outputs at
        // the inputs' offsets) also exchange the results between the wavefronts of a group
        bool unshifted = true;
        for (const Run& r : m_runs) unshifted = unshifted && r.in_begin == r.out_begin;
        // tiles that do not sit on the cache lines of every buffer share lines with their neighbours
        const bool base_on_lines = lines_shared(0) && m_misalign % 128 == 0;  // flat tiles start at the buffers' first byte
        bool on_lines = base_on_lines;
        for (const Run& r : m_runs) on_lines = on_lines && lines_shared((r.in_begin - r.out_begin) * m_elem);
        // (large one-output folds whose INPUT tiles sit on line boundaries stay at one wavefront per tile, see
        // flat_one_out; the one output in nine streams may be shifted by a part of a line - a receive length that is no
        // multiple of 128 bytes: 82 - 84 % of the HBM peak against 79 - 80 in the group form - but with every buffer
        // off the lines the group form, which deals its workgroups to the XCDs, is 8 points ahead)
        const bool one_wave = total < flat_group_min_tiles(m_nranks) || (base_on_lines && flat_one_out(m_nranks, m_nout, total));
        L.waves = one_wave ? 1 : kGroupWaves;
        L.exchange = (L.waves == kGroupWaves && !m_tree && m_nout == m_nranks && unshifted) ? 1 : 0;
        if (L.waves == kGroupWaves && !on_lines) L.exchange |= 2u;
        if (L.waves == kGroupWaves && L.exchange == 1 && paced_launch(m_in, m_out, m_nranks, expect * m_elem))
            L.exchange |= kFlatPaced;
        L.unshifted = unshifted ? 1 : 0;
        m_plan.steps.push_back(step);
        return true;
    }

    void emit_general() {
        const uint64_t epv = kVecBytes / m_elem;
        // long vector bodies take the group form (four wavefronts per workgroup)
        // Elements go 16 bytes per lane whatever the offsets (gfx950 serves 128-bit accesses at any byte address):
        // buffers whose offsets from a 16-byte boundary differ (m_plain, m_bytes), and runs whose outputs are
        // shifted against their inputs by a part of a vector (reduce_scatter with a receive length that is no
        // multiple of 16 bytes, the copies of the two-phase and ring schedules).
        const bool natural = m_plain || m_bytes || m_aligned;
        auto same_phase = [&](const Run& r) { return m_aligned && r.in_begin % epv == r.out_begin % epv; };
        uint64_t vector_elems = 0;
        for (const Run& r : m_runs)
            if (natural || same_phase(r)) vector_elems += r.count;
        uint64_t all_elems = 0;
        for (const Run& r : m_runs) all_elems += r.count;
        // short launches keep one wavefront per tile, and small tiles; folds that are vectors throughout keep them
        // longer (short_vector_max_bytes)
        const uint64_t vector_tiles = vector_elems / (kThreads * epv);
        if (vector_elems == all_elems && m_nfold >= 2) {
            m_short = all_elems * m_elem <= short_vector_max_bytes(m_elem, m_nranks, m_nout);
            m_waves = !m_short && vector_tiles >= kGroupMinTiles ? kGroupWaves : 1;
        } else {
            m_waves = vector_tiles >= kGroupMinTiles ? kGroupWaves : 1;
            m_short = m_waves == 1 && all_elems * m_elem <= kShortTilesMaxBytes;
        }
        m_paced = m_waves == kGroupWaves && m_nfold >= 3 && paced_launch(m_in, m_out, m_nranks, vector_elems * m_elem, false, m_nout);
        open_launch();
        for (const Run& r : m_runs) {
            const bool vector = natural || same_phase(r);
            uint64_t head = 0, body = 0;
            if (m_plain || m_bytes) {
                // no grid that all buffers share: the body starts where the run's first output sits on a tile
                // boundary, so that at least the stores of the other outputs miss whole cache lines by a few
                // elements only instead of by the run's arbitrary offset
                const uint64_t tile_bytes = uint64_t(kThreads) * kVecBytes;
                const uint64_t at = (reinterpret_cast<uintptr_t>(m_out[r.out_first]) + r.out_begin * m_elem) & (tile_bytes - 1);
                head = std::min<uint64_t>(((tile_bytes - at) & (tile_bytes - 1)) / m_elem, r.count);
                body = (r.count - head) / epv * epv;
            } else if (same_phase(r)) {
                // the body starts where inputs and outputs both sit on the coarsest grid they share
                uint64_t grid = m_grid;
                const uint64_t skew = (r.in_begin - r.out_begin) * m_elem;  // unsigned wrap is fine mod 2^k
                while (grid > kVecBytes && (skew & (grid - 1))) grid >>= 1;
                const uint64_t at = (m_misalign + r.in_begin * m_elem) & (grid - 1);
                head = std::min<uint64_t>(((grid - at) & (grid - 1)) / m_elem, r.count);
                body = (r.count - head) / epv * epv;
            } else if (vector) {
                // shifted by a part of a vector: the body starts where the OUTPUTS sit on the grid, so the stores
                // are aligned and cover whole cache lines; the loads take the inputs as they lie
                const uint64_t at = (m_misalign + r.out_begin * m_elem) & (m_grid - 1);
                head = std::min<uint64_t>(((m_grid - at) & (m_grid - 1)) / m_elem, r.count);
                body = (r.count - head) / epv * epv;
            }
            if (!body) {
                add_segment(r.in_begin, r.out_begin, r.count, r, 0);
                continue;
            }
            const uint64_t tail = r.count - head - body;
            if (head) add_segment(r.in_begin, r.out_begin, head, r, 0);
            // (a body that starts on the common grid sits on the lines of inputs and outputs alike unless the
            // outputs are shifted by a part of a line)
            const bool on_lines = lines_shared((r.in_begin - r.out_begin) * m_elem) && same_phase(r);
            add_segment(r.in_begin + head, r.out_begin + head, body, r, kSegVector | (on_lines ? 0 : kSegDeal));
            if (tail) add_segment(r.in_begin + head + body, r.out_begin + head + body, tail, r, 0);
        }
        close_launch();
    }

    void open_launch() {
        std::memset(&m_launch, 0, sizeof(m_launch));
        for (uint32_t r = 0; r < kMaxRanks; ++r) {
            m_launch.in[r] = m_in[r];
            m_launch.out[r] = m_out[r];
        }
        for (uint32_t i = 0; i < kMaxSegments; ++i) m_launch.first_tile[i] = 0xffffffffu;
        m_launch.nranks = m_nranks;
        m_launch.nfold = m_nfold;
        m_launch.nout = m_nout;
        m_launch.new_wins_ties = m_new_wins ? 1 : 0;
        m_launch.elem_size = m_elem;
        m_launch.waves = m_waves;
        m_launch.paced = m_paced ? 1 : 0;
        m_launch.short_tiles = m_short ? 1 : 0;
    }

    void close_launch() {
        if (!m_launch.nseg) return;
        Step step;
        std::memset(&step, 0, sizeof(step));
        step.kind = Step::kFold;
        step.fold = m_launch;
        m_plan.steps.push_back(step);
    }

    void add_segment(uint64_t in_begin, uint64_t out_begin, uint64_t count, const Run& r, uint8_t flags) {
        const uint64_t per_tile = tile_elems(m_launch, flags & kSegVector);
        const uint64_t max_tiles = 0x7fffffffull;
        while (count) {
            if (m_launch.nseg == kMaxSegments || m_launch.total_tiles >= max_tiles) {
                close_launch();
                open_launch();
            }
            // a segment never takes more tiles than one launch's grid has left
            const uint64_t room = max_tiles - m_launch.total_tiles;
            uint64_t take = std::min(count, room * per_tile);
            if (take < count) take = take / per_tile * per_tile;  // cut between workgroups (room > 0: never empty)
            m_launch.first_tile[m_launch.nseg] = m_launch.total_tiles;
            FoldSegment& sg = m_launch.seg[m_launch.nseg++];
            sg.in_begin = in_begin;
            sg.out_begin = out_begin;
            sg.count = take;
            sg.start = r.start;
            sg.dir = r.dir;
            sg.out_first = r.out_first;
            sg.flags = flags;
            m_launch.total_tiles += uint32_t(segment_tiles(m_launch, flags & kSegVector, take));
            in_begin += take;
            out_begin += take;
            count -= take;
        }
    }

    Plan& m_plan;
    const void* m_in[kMaxRanks];
    void* m_out[kMaxRanks];
    uint32_t m_nranks, m_nfold, m_nout, m_elem;
    bool m_new_wins;
    bool m_aligned;
    bool m_plain = false;  // 16-byte accesses on buffers that are only element-aligned (4- and 8-byte types)
    bool m_bytes = false;  // the same for 1- and 2-byte types: tiles start at any byte address
    uint32_t m_misalign = 0;
    uint64_t m_grid = kVecBytes;
    bool m_tree = false;
    uint32_t m_waves = 1;
    bool m_short = false;
    bool m_paced = false;
    std::vector<Run> m_runs;
    FoldLaunch m_launch;
};

Status check_ranks(uint32_t nranks) {
    if (nranks < 1 || nranks > kMaxRanks) return invalid("nranks must be in [1, 32]");
    return MEGRAY_OK;
}

Status check_elem(uint32_t elem_size) {
    if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8)
        return invalid("element size must be 1, 2, 4 or 8");
    return MEGRAY_OK;
}

// A length whose byte count, times every rank, still fits 64 bits with room to spare.
Status check_len(uint64_t len) {
    if (len > (uint64_t(1) << 48)) return invalid("length beyond 2^48 elements");
    return MEGRAY_OK;
}

// Every buffer a launch will touch must be there: a null pointer would fault on the device.
Status check_present(const void* const* ptrs, uint32_t n, uint64_t bytes, const char* what) {
    if (!bytes) return MEGRAY_OK;
    for (uint32_t r = 0; r < n; ++r)
        if (!ptrs[r]) return invalid(what);
    return MEGRAY_OK;
}
Status check_present(void* const* ptrs, uint32_t n, uint64_t bytes, const char* what) {
    if (!bytes) return MEGRAY_OK;
    for (uint32_t r = 0; r < n; ++r)
        if (!ptrs[r]) return invalid(what);
    return MEGRAY_OK;
}
Status check_present(const void* ptr, uint64_t bytes, const char* what) {
    return (bytes && !ptr) ? invalid(what) : MEGRAY_OK;
}

// Buffers of different ranks must not overlap.  A rank's own receive buffer may overlap its send
// buffer only at the one offset where every element keeps its address (`recv == send + shift`).
Status check_overlap(const void* const* send, uint64_t send_bytes, void* const* recv, uint64_t recv_bytes,
                     uint32_t nranks, int64_t own_shift_bytes_per_rank) {
    for (uint32_t a = 0; a < nranks; ++a) {
        for (uint32_t b = a + 1; b < nranks; ++b)
            if (overlaps(recv[a], recv_bytes, recv[b], recv_bytes))
                return invalid("receive buffers of two ranks overlap");
        for (uint32_t b = 0; b < nranks; ++b) {
            if (!overlaps(recv[a], recv_bytes, send[b], send_bytes)) continue;
            const intptr_t shift = int64_t(a) * own_shift_bytes_per_rank;
            const bool in_place = a == b && reinterpret_cast<intptr_t>(recv[a]) ==
                                                    reinterpret_cast<intptr_t>(send[a]) + shift;
            if (!in_place) return invalid("a receive buffer overlaps a send buffer out of place");
        }
    }
    return MEGRAY_OK;
}

}  // namespace

const char* plan_error() {
    return g_plan_error;
}

void set_plan_error(const char* text) {
    std::snprintf(g_plan_error, sizeof(g_plan_error), "%s", text ? text : "");
}

void chunk_partition(uint64_t len, uint32_t nchunks, uint64_t* sizes, uint64_t* offsets) {
    const uint64_t quotient = len / nchunks, remainder = len % nchunks;
    uint64_t offset = 0;
    for (uint32_t i = 0; i < nchunks; ++i) {
        sizes[i] = quotient + (i < remainder ? 1 : 0);
        offsets[i] = offset;
        offset += sizes[i];
    }
}

uint32_t order_chunks(FoldOrder order, uint32_t nranks) {
    switch (order) {
        case kOrderUcx: return nranks;
        case kOrderShm: return 2 * nranks;  // k = 2 chunks per rank, src/shm/all_reduce.cpp:42-43
        default: return 1;
    }
}

bool order_new_wins_ties(Collective coll, FoldOrder order) {
    // src/ucx/reduce_scatter.cpp:50-51 calls reduce(incoming, local): the (i0 > i1) ? i0 : i1 of
    // src/ucx/kernel.cu:24-38 then keeps the local (new) operand.  Every other loop keeps the
    // accumulator: src/ucx/all_reduce.cpp:74-76 passes (local, incoming); std::max / std::min in
    // src/shm/utils.cpp:24-32 return their first argument, the accumulator.
    return order == kOrderUcx && coll == kReduceScatter;
}

void chunk_fold_order(Collective coll, FoldOrder order, uint32_t nranks, uint32_t chunk, uint8_t* start,
                      int8_t* dir, uint8_t* owner) {
    switch (order) {
        case kOrderUcx:
            *dir = 1;
            if (coll == kAllReduce) {
                // chunk c starts on rank c and is finished on rank c-1 (src/ucx/all_reduce.cpp:57-60)
                *start = uint8_t(chunk % nranks);
                *owner = uint8_t(ring_sub(chunk, 1, nranks));
            } else {
                // chunk c starts on rank c+1 and is finished on rank c (src/ucx/reduce_scatter.cpp:40-41)
                *start = uint8_t(ring_add(chunk, 1, nranks));
                *owner = uint8_t(chunk % nranks);
            }
            break;
        case kOrderShm:
            // chunk w belongs to rank w/2, whose copy seeds the arena; ranks w/2-1, w/2-2, ... add
            // theirs (src/shm/all_reduce.cpp:91-109, src/shm/communicator.cpp:56-68)
            *dir = -1;
            *start = uint8_t((chunk / 2) % nranks);
            *owner = *start;
            break;
        default:
            *dir = 1;
            *start = 0;
            *owner = 0;
            break;
    }
}

Status plan_all_reduce(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                       uint64_t len, uint32_t elem_size, FoldOrder order, Schedule sched) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    if (order < 0 || order >= kOrderCount) return invalid("unknown fold order");
    if (sched < 0 || sched >= kSchedCount) return invalid("unknown schedule");
    if (sched == kSchedRing && order != kOrderUcx) return invalid("the ring schedule exists for the ucx order only");
    PLAN_TRY(check_len(len));
    PLAN_TRY(check_present(send, nranks, len, "a send buffer is null"));
    PLAN_TRY(check_present(recv, nranks, len, "a receive buffer is null"));
    PLAN_TRY(check_overlap(send, len * elem_size, recv, len * elem_size, nranks, 0));
    const uint32_t nchunks = order_chunks(order, nranks);
    uint64_t sizes[kMaxChunks], offs[kMaxChunks];
    chunk_partition(len, nchunks, sizes, offs);
    const bool new_wins = order_new_wins_ties(kAllReduce, order);
    const void* recv_in[kMaxRanks];
    for (uint32_t r = 0; r < nranks; ++r) recv_in[r] = recv[r];

    if (sched == kSchedFused) {
        FoldBuilder fold(plan, send, recv, nranks, nranks, nranks, elem_size, new_wins);
        for (uint32_t c = 0; c < nchunks; ++c) {
            uint8_t start, owner;
            int8_t dir;
            chunk_fold_order(kAllReduce, order, nranks, c, &start, &dir, &owner);
            fold.add_run(offs[c], offs[c], sizes[c], start, dir, 0);
        }
        fold.finish();
        return MEGRAY_OK;
    }

    if (sched == kSchedTwoPhase) {
        {   // reduce-scatter: the finished chunk lands on the rank the ring would leave it on
            FoldBuilder fold(plan, send, recv, nranks, nranks, 1, elem_size, new_wins);
            for (uint32_t c = 0; c < nchunks; ++c) {
                uint8_t start, owner;
                int8_t dir;
                chunk_fold_order(kAllReduce, order, nranks, c, &start, &dir, &owner);
                fold.add_run(offs[c], offs[c], sizes[c], start, dir, owner);
            }
            fold.finish();
        }
        if (nranks > 1) {  // all-gather: read the owner's chunk once, write the other N-1 ranks
            FoldBuilder copy(plan, recv_in, recv, nranks, 1, nranks - 1, elem_size, false);
            for (uint32_t c = 0; c < nchunks; ++c) {
                uint8_t start, owner;
                int8_t dir;
                chunk_fold_order(kAllReduce, order, nranks, c, &start, &dir, &owner);
                copy.add_run(offs[c], offs[c], sizes[c], owner, 1, uint8_t(ring_add(owner, 1, nranks)));
            }
            copy.finish();
        }
        return MEGRAY_OK;
    }

    // kSchedRing: the reference's steps, one launch each, with "send + receive into the workspace"
    // replaced by reading the left neighbour's buffer in place.
    {   // src/ucx/all_reduce.cpp:44-45
        FoldBuilder copy(plan, send, recv, nranks, 1, 1, elem_size, false);
        for (uint32_t r = 0; r < nranks; ++r)
            if (send[r] != recv[r]) copy.add_run(0, 0, len, uint8_t(r), 1, uint8_t(r));
        copy.finish();
    }
    for (uint32_t i = 0; i + 1 < nranks; ++i) {  // :61-82
        FoldBuilder fold(plan, recv_in, recv, nranks, 2, 1, elem_size, false);
        for (uint32_t r = 0; r < nranks; ++r) {
            const uint32_t c = ring_sub(r, i + 1, nranks);
            // reduce(local, incoming): incoming (the left rank's chunk) is the accumulator
            fold.add_run(offs[c], offs[c], sizes[c], uint8_t(ring_sub(r, 1, nranks)), 1, uint8_t(r));
        }
        fold.finish();
    }
    for (uint32_t i = 0; i + 1 < nranks; ++i) {  // :88-101
        FoldBuilder copy(plan, recv_in, recv, nranks, 1, 1, elem_size, false);
        for (uint32_t r = 0; r < nranks; ++r) {
            const uint32_t c = ring_sub(r, i, nranks);
            copy.add_run(offs[c], offs[c], sizes[c], uint8_t(ring_sub(r, 1, nranks)), 1, uint8_t(r));
        }
        copy.finish();
    }
    return MEGRAY_OK;
}

Status plan_reduce_scatter(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                           uint64_t recvlen, uint32_t elem_size, FoldOrder order, Schedule sched) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    if (order < 0 || order >= kOrderCount) return invalid("unknown fold order");
    if (sched != kSchedFused) return invalid("reduce_scatter has the fused schedule only");
    PLAN_TRY(check_len(recvlen));
    PLAN_TRY(check_present(send, nranks, recvlen, "a send buffer is null"));
    PLAN_TRY(check_present(recv, nranks, recvlen, "a receive buffer is null"));
    const uint64_t total = recvlen * nranks;
    PLAN_TRY(check_overlap(send, total * elem_size, recv, recvlen * elem_size, nranks,
                               int64_t(recvlen * elem_size)));
    const uint32_t nchunks = order_chunks(order, nranks);
    uint64_t sizes[kMaxChunks], offs[kMaxChunks];
    chunk_partition(total, nchunks, sizes, offs);
    FoldBuilder fold(plan, send, recv, nranks, nranks, 1, elem_size, order_new_wins_ties(kReduceScatter, order));
    for (uint32_t c = 0; c < nchunks; ++c) {
        uint8_t start, owner;
        int8_t dir;
        chunk_fold_order(kReduceScatter, order, nranks, c, &start, &dir, &owner);
        // rank r receives elements [r * recvlen, (r + 1) * recvlen) whatever chunk they were folded in
        uint64_t begin = offs[c];
        const uint64_t end = offs[c] + sizes[c];
        while (begin < end) {
            const uint64_t r = begin / recvlen;
            const uint64_t stop = std::min(end, (r + 1) * recvlen);
            fold.add_run(begin, begin - r * recvlen, stop - begin, start, dir, uint8_t(r));
            begin = stop;
        }
    }
    fold.finish();
    return MEGRAY_OK;
}

namespace {
Status add_pack(Plan& plan, const void* const* in, void* const* out, uint32_t nranks, uint64_t block_bytes,
                uint32_t mode, uint32_t root, uint32_t ncopies);
}

Status plan_all_gather(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                       uint64_t sendlen, uint32_t elem_size) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    PLAN_TRY(check_len(sendlen));
    PLAN_TRY(check_present(send, nranks, sendlen, "a send buffer is null"));
    PLAN_TRY(check_present(recv, nranks, sendlen, "a receive buffer is null"));
    // in place: rank r's contribution already sits in its slot, send[r] == recv[r] + r * sendlen
    for (uint32_t a = 0; a < nranks; ++a) {
        for (uint32_t b = a + 1; b < nranks; ++b)
            if (overlaps(recv[a], sendlen * nranks * elem_size, recv[b], sendlen * nranks * elem_size))
                return invalid("receive buffers of two ranks overlap");
        for (uint32_t b = 0; b < nranks; ++b) {
            if (!overlaps(recv[a], sendlen * nranks * elem_size, send[b], sendlen * elem_size)) continue;
            const bool in_place = a == b && static_cast<const char*>(send[a]) ==
                                                    static_cast<const char*>(recv[a]) + a * sendlen * elem_size;
            if (!in_place) return invalid("a receive buffer overlaps a send buffer out of place");
        }
    }
    // one pack launch: block i is read once from rank i and written into slot i of every rank
    const uint64_t before = plan.steps.size();
    Status st = add_pack(plan, send, recv, nranks, sendlen * elem_size, kPackAllGather, 0, nranks);
    if (st == MEGRAY_OK && plan.steps.size() > before)
        plan.bytes_written += sendlen * elem_size * nranks * (nranks - 1);  // add_pack counted one copy per block
    return st;
}

namespace {

// Should the group pack kernel of an all_gather or a broadcast issue a wavefront's N stores one at a time
// (PackLaunch::paced)?  A paced wavefront lives N round trips, which costs a short launch and gains a long one: the
// memory serves N streams of stores better when they do not arrive N at a time.  Measured on MI355X, % of the HBM peak,
// all stores at once -> one at a time.
// all_gather, fp32, outputs of 32 / 128 / 512 MiB per rank (blocks of 1 / N of that), on outputs an odd multiple of
// 128 MiB apart | 128 MiB k + 32 MiB apart (the placement's all_gather rule) | allocated one by one:
//   4 ranks   81.8 -> 77.5 | 82.0 -> 77.1 | 81.2 -> 77.3     80.1 -> 82.4 | 84.5 -> 82.7 | 79.6 -> 82.3     82.6 -> 84.4 | 85.5 -> 84.5 | 82.6 -> 84.4
//   5 ranks   78.5 -> 75.6 | 78.9 -> 75.7 | 83.2 -> 76.0     83.1 -> 81.7 | 83.3 -> 82.2 | 81.8 -> 81.6     81.0 -> 83.7 | 81.6 -> 83.7 | 80.4 -> 83.6
//   6 ranks   78.6 -> 77.0 | 78.9 -> 76.6 | 83.4 -> 79.6     81.6 -> 82.6 | 82.6 -> 83.0 | 80.0 -> 82.3     79.3 -> 83.8 | 77.9 -> 84.0 | 80.9 -> 84.2
//   7 ranks   78.3 -> 77.8 | 79.3 -> 77.6 | 82.1 -> 80.3     81.4 -> 83.2 | 82.7 -> 83.4 | 80.1 -> 82.6     79.5 -> 83.9 | 77.3 -> 83.6 | 79.4 -> 84.3
//   8 ranks   84.1 -> 81.5 | 84.9 -> 81.1 | 84.0 -> 80.9     79.7 -> 84.0 | 84.1 -> 83.9 | 81.1 -> 83.2     83.2 -> 84.6 | 85.2 -> 84.8 | 81.1 -> 84.8
// all_gather, uint8, outputs 128 MiB k + 32 MiB apart, blocks of 1 / 4 / 16 / 64 MiB:
//   9 ranks     76.8 -> 76.8 / 82.5 -> 82.4 / 84.1 -> 84.2 / 84.6 -> 84.6      (allocated one by one, 16 / 64 MiB: 80.6 -> 83.4 / 80.9 -> 84.6)
//   12 ranks    79.6 -> 81.6 / 78.0 -> 81.3 / 82.5 -> 84.4 / 81.9 -> 84.6      (allocated one by one: 77.4 -> 83.7 / 75.1 -> 80.2 / 80.6 -> 83.1 / 79.8 -> 84.5)
//   16 ranks    79.6 -> 80.7 / 76.5 -> 81.8 / 78.0 -> 83.9 / 78.2 -> 82.9      (allocated one by one: 69.1 -> 81.5 / 75.0 -> 80.6 / 77.4 -> 84.5 / 76.2 -> 83.2)
// all_gather, fp32, 6 / 7 / 8 / 10 ranks, outputs of 48 / 64 / 96 MiB per rank, placed | placed for the all_gather | one by one:
//   6 ranks   77.0 -> 80.0 | 80.5 -> 79.7 | 79.7 -> 79.9     79.4 -> 81.8 | 82.6 -> 82.2 | 82.7 -> 82.2     80.1 -> 82.8 | 82.5 -> 82.4 | 80.8 -> 82.1
//   8 ranks   79.3 -> 80.5 | 80.5 -> 80.3 | 78.3 -> 80.0     80.1 -> 82.1 | 81.7 -> 81.8 | 77.6 -> 81.8     80.4 -> 82.9 | 83.0 -> 83.0 | 81.7 -> 82.5
//   10 ranks  76.2 -> 80.6 | 76.9 -> 80.7 | 76.7 -> 79.8     76.2 -> 80.9 | 76.9 -> 81.3 | 77.4 -> 81.9     76.8 -> 82.4 | 76.6 -> 82.8 | 77.3 -> 82.2
// So: twelve ranks and more from blocks of a MiB; six ranks and more from 384 MiB written in all; four and five ranks
// from 2 GiB written; where the outputs lie does not enter.
bool paced_gather(uint32_t nranks, uint64_t block_bytes) {
    if (pace_override() >= 0) return pace_override() == 1;
    constexpr uint64_t kMiB = uint64_t(1) << 20;
    const uint64_t written = block_bytes * nranks * nranks;
    if (nranks >= 12) return block_bytes >= kMiB;
    if (nranks >= 6) return written >= 384 * kMiB;
    return nranks >= 4 && written >= 2048 * kMiB;
}

// The same for a broadcast (one load, N stores per wavefront, to the same offset of every output).  fp32, blocks of
// 32 / 128 / 512 MiB, outputs an odd multiple of 128 MiB apart | allocated one by one:
//   4 ranks   81.8 -> 77.2 | 81.6 -> 77.0     84.9 -> 82.4 | 84.4 -> 82.3     82.6 -> 84.5 | 80.2 -> 84.3
//   5 ranks   83.8 -> 78.5 | 83.3 -> 78.5     85.0 -> 83.3 | 78.1 -> 82.8     79.9 -> 85.0 | 79.3 -> 85.0
//   6 ranks   84.5 -> 80.0 | 84.6 -> 79.8     84.3 -> 82.1 | 77.5 -> 82.2     80.3 -> 82.9 | 83.1 -> 85.3
//   7 ranks   84.8 -> 80.6 | 84.7 -> 80.3     80.5 -> 82.9 | 79.4 -> 82.8     81.6 -> 84.7 | 81.7 -> 84.4
//   8 ranks   84.1 -> 81.5 | 83.9 -> 80.9     85.5 -> 84.5 | 84.7 -> 83.4     80.5 -> 84.8 | 79.6 -> 84.3
// (blocks of 256 MiB, placed, 3 / 5 / 6 / 7 / 8 ranks: 86.3 -> 83.5 / 81.6 -> 84.2 / 79.2 -> 81.7 / 79.2 -> 83.7 / 82.6 -> 84.6);
// uint8 blocks of 4 / 16 / 64 MiB, placed | allocated one by one:
//   9 ranks     67.8 -> 67.8 | 67.8 -> 67.7     83.4 -> 85.3 | 82.7 -> 82.6     81.5 -> 81.9 | 78.4 -> 81.1
//   12 ranks    68.6 -> 67.6 | 67.5 -> 70.2     81.5 -> 83.7 | 80.2 -> 82.5     79.3 -> 82.1 | 76.6 -> 81.6
//   16 ranks    69.9 -> 72.1 | 71.0 -> 70.5     78.8 -> 82.2 | 78.7 -> 81.4     75.5 -> 81.2 | 74.0 -> 81.1
// So: nine ranks and more from blocks of 16 MiB, five and more from 256 MiB, four from 512 MiB.
bool paced_broadcast(uint32_t nranks, uint64_t block_bytes) {
    if (pace_override() >= 0) return pace_override() == 1;
    constexpr uint64_t kMiB = uint64_t(1) << 20;
    if (nranks >= 9) return block_bytes >= 16 * kMiB;
    if (nranks >= 5) return block_bytes >= 256 * kMiB;
    return nranks == 4 && block_bytes >= 512 * kMiB;
}

uint32_t common_width(uint64_t block_bytes, const void* const* a, const void* const* b, uint32_t n) {
    uintptr_t bits = uintptr_t(block_bytes);
    for (uint32_t r = 0; r < n; ++r) bits |= reinterpret_cast<uintptr_t>(a[r]) | reinterpret_cast<uintptr_t>(b[r]);
    uint32_t width = kVecBytes;
    while (width > 1 && (bits & (width - 1))) width >>= 1;
    return width;
}

Status add_pack(Plan& plan, const void* const* in, void* const* out, uint32_t nranks, uint64_t block_bytes,
                uint32_t mode, uint32_t root, uint32_t ncopies) {
    if (!block_bytes) return MEGRAY_OK;
    Step step;
    std::memset(&step, 0, sizeof(step));
    step.kind = Step::kPack;
    PackLaunch& L = step.pack;
    const void* out_c[kMaxRanks];
    for (uint32_t r = 0; r < nranks; ++r) {
        L.in[r] = in[r];
        L.out[r] = out[r];
        out_c[r] = out[r];
    }
    L.block_bytes = block_bytes;
    L.nranks = nranks;
    L.mode = mode;
    L.root = root;
    L.ncopies = ncopies;
    L.width = common_width(block_bytes, in, out_c, nranks);
    const uint64_t tiles = pack_tiles(block_bytes);
    // Long blocks take the group form.  An all_to_all of five ranks and more is a launch of 25 and more copies
    // whichever form it takes, and up to 4 MiB per block one wavefront per tile serves it better: the group form's
    // grid comes in runs of 32 workgroups per copy, half of them idle on a block of 129 tiles.  Measured on MI355X,
    // uint8, microseconds per all_to_all, group form -> one wavefront per tile, blocks of 128 KiB / 512 KiB / 2 MiB / 4 MiB:
    //   16 ranks 18.3 -> 12.3 / 45.5 -> 40.4 / 160 -> 159 / 314 -> 318;  8 ranks 6.2 -> 4.6 / 13.2 -> 12.1 / 41.1 -> 39.7 / 80.5 -> 81.0;
    //   5 ranks 4.4 -> 3.8 / 6.3 -> 6.1 / 17.8 -> 17.1 / 31.9 -> 31.4;  4 ranks 3.3 -> 3.4 / 4.9 -> 4.6 / 12.0 -> 12.1 / 21.4 -> 21.5 (left alone).
    // A broadcast is one copy with N destinations, and an all_gather N of them: as long as the launch is short, one
    // wavefront per tile is the shorter way for them as well.  Group form / one wavefront per tile, microseconds, device
    // in its steady state, by KiB per block:
    //   broadcast   4 ranks  128 3.10 / 2.78   512 3.10 / 2.81   1024 3.16 / 2.98   2048 3.45 / 3.42   4096 4.49 / 4.64
    //               8 ranks  128 3.74 / 3.05   512 3.74 / 3.07   1024 3.79 / 3.41   2048 4.35 / 4.40   4096 6.60 / 6.82
    //              16 ranks  128 5.56 / 4.71   512 5.69 / 4.71   1024 5.77 / 5.05   2048 6.39 / 6.69   4096 10.8 / 10.5
    //   all_gather  2 ranks  512 2.92 / 2.79   4096 5.22 / 4.84   8192 7.58 / 6.73   16384 15.5 / 16.4
    //               4 ranks  128 3.10 / 2.88   1024 4.76 / 4.56   4096 10.7 / 10.4   8192 24.5 / 29.5
    //               6 ranks  128 3.63 / 3.06   1024 7.26 / 6.71   3072 16.3 / 15.4   4096 24.6 / 26.3
    //               8 ranks  128 4.01 / 4.19   192 4.02 / 3.93   1024 11.6 / 10.1   2048 18.8 / 17.7   3072 34.3 / 35.2   4096 45.0 / 51.5
    //              12 ranks  128 5.69 / 6.59   256 8.07 / 6.81   512 12.0 / 10.9   1024 25.0 / 27.0   (16 ranks alike: left alone)
    // (blocks on 4-byte boundaries only cross earlier: fp32, 4 ranks x 5 MiB + 4 B 12.7 / 15.5, 3 ranks x 10 MiB + 4 B 17.9 / 21.9;
    // 9 and 11 ranks x 2 MiB 28.2 / 30.1 and 40.9 / 44.1, x 1 MiB 13.9 / 12.3 and 18.4 / 16.9.)
    // scatter, gather and send / recv keep the group form from 128 tiles on.
    uint64_t group_min = kGroupMinTiles / 4;
    if (mode == kPackAllToAll && nranks >= 5) group_min = 4096;
    if (mode == kPackBroadcast) group_min = 2048;
    if (mode == kPackAllGather && nranks < 12)
        group_min = nranks <= 3 ? 8192 : nranks == 4 ? 4096 : nranks <= 7 ? 3072 : nranks == 8 ? 2048 : 1280;
    L.waves = tiles >= group_min ? kGroupWaves : 1;
    // (eight ranks x 128 KiB, 1024 workgroups of one wavefront, is the one point below that where the group form is ahead:
    // 4.0 against 4.2 - 4.7 us, while 96 KiB and 160 KiB read 3.6 / 3.2 and 4.0 / 3.7)
    if (mode == kPackAllGather && nranks == 8 && tiles >= kGroupMinTiles / 4 && tiles < 160) L.waves = kGroupWaves;
    if (L.waves == kGroupWaves && mode == kPackAllGather) L.paced = paced_gather(nranks, block_bytes) ? 1 : 0;
    if (L.waves == kGroupWaves && mode == kPackBroadcast) L.paced = paced_broadcast(nranks, block_bytes) ? 1 : 0;
    // A grid holds 2^31 - 1 workgroups: blocks whose tiles, over all copies, outnumber that are cut into
    // slices of tiles, one launch each (the reference's per-peer copies have no such limit either).
    const uint64_t span = uint64_t(kGroupWaves) * kGroupStride;  // tiles a run of kGroupStride workgroups covers
    uint64_t slice = 0x7fffffffull / ncopies;                    // workgroups per copy that fit one grid
    if (L.waves == kGroupWaves) slice = slice / kGroupStride * span;  // in tiles, whole runs of workgroups
    else slice = slice / span * span;
    if (!slice) return invalid("too many block copies for one pack launch");
    for (uint64_t first = 0; first < tiles; first += slice) {
        const uint64_t take = std::min(slice, tiles - first);
        L.first_tile = first;
        L.tiles_per_copy = uint32_t(take);
        L.groups_per_copy = group_grid(L.tiles_per_copy);
        plan.steps.push_back(step);
    }
    plan.bytes_read += block_bytes * ncopies;
    plan.bytes_written += block_bytes * ncopies;
    return MEGRAY_OK;
}

}  // namespace

void set_store_policy(Plan& plan) {
    const bool keep = keep_override() >= 0 ? keep_override() == 1 : plan.bytes_written <= kKeepMaxBytes;
    for (Step& step : plan.steps) {
        switch (step.kind) {
            case Step::kFold: step.fold.keep = keep ? 1 : 0; break;
            case Step::kFlat: step.flat.exchange = keep ? step.flat.exchange | kFlatKeep : step.flat.exchange & ~kFlatKeep; break;
            case Step::kTree:
                step.tree.keep = keep ? 1 : 0;
                step.tree.batch = tree_batch(step.tree.nranks, step.tree.elem_size, keep, step.tree.total_tiles);
                break;
            case Step::kPack: step.pack.keep = keep ? 1 : 0; break;
        }
    }
}

int plan_overrides() { return (pace_override() + 1) + 4 * (keep_override() + 1); }

Status plan_all_to_all(Plan& plan, const void* const* send, void* const* recv, uint32_t nranks,
                       uint64_t len, uint32_t elem_size) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    PLAN_TRY(check_len(len));
    PLAN_TRY(check_present(send, nranks, len, "a send buffer is null"));
    PLAN_TRY(check_present(recv, nranks, len, "a receive buffer is null"));
    const uint64_t bytes = len * nranks * elem_size;
    for (uint32_t a = 0; a < nranks; ++a) {
        for (uint32_t b = 0; b < nranks; ++b) {
            if (a < b && overlaps(recv[a], bytes, recv[b], bytes)) return invalid("receive buffers of two ranks overlap");
            if (overlaps(recv[a], bytes, send[b], bytes)) return invalid("all_to_all cannot run in place");
        }
    }
    return add_pack(plan, send, recv, nranks, len * elem_size, kPackAllToAll, 0, nranks * nranks);
}

Status plan_scatter(Plan& plan, const void* send_root, void* const* recv, uint32_t nranks, uint64_t recvlen,
                    uint32_t elem_size, uint32_t root) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    if (root >= nranks) return invalid("root out of range");
    const uint64_t block = recvlen * elem_size;
    PLAN_TRY(check_len(recvlen));
    PLAN_TRY(check_present(send_root, recvlen, "the root's send buffer is null"));
    PLAN_TRY(check_present(recv, nranks, recvlen, "a receive buffer is null"));
    for (uint32_t a = 0; a < nranks; ++a) {
        for (uint32_t b = a + 1; b < nranks; ++b)
            if (overlaps(recv[a], block, recv[b], block)) return invalid("receive buffers of two ranks overlap");
        if (overlaps(recv[a], block, send_root, block * nranks)) {
            const bool in_place = a == root && static_cast<const char*>(recv[a]) ==
                                                       static_cast<const char*>(send_root) + root * block;
            if (!in_place) return invalid("a receive buffer overlaps the root's send buffer out of place");
        }
    }
    const void* in[kMaxRanks] = {};
    in[root] = send_root;
    return add_pack(plan, in, recv, nranks, block, kPackScatter, root, nranks);
}

Status plan_gather(Plan& plan, const void* const* send, void* recv_root, uint32_t nranks, uint64_t sendlen,
                   uint32_t elem_size, uint32_t root) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    if (root >= nranks) return invalid("root out of range");
    const uint64_t block = sendlen * elem_size;
    PLAN_TRY(check_len(sendlen));
    PLAN_TRY(check_present(send, nranks, sendlen, "a send buffer is null"));
    PLAN_TRY(check_present(recv_root, sendlen, "the root's receive buffer is null"));
    for (uint32_t b = 0; b < nranks; ++b) {
        if (overlaps(recv_root, block * nranks, send[b], block)) {
            const bool in_place = b == root && static_cast<const char*>(send[b]) ==
                                                       static_cast<const char*>(recv_root) + root * block;
            if (!in_place) return invalid("the root's receive buffer overlaps a send buffer out of place");
        }
    }
    void* out[kMaxRanks] = {};
    out[root] = recv_root;
    return add_pack(plan, send, out, nranks, block, kPackGather, root, nranks);
}

Status plan_broadcast(Plan& plan, const void* send_root, void* const* recv, uint32_t nranks, uint64_t len,
                      uint32_t elem_size, uint32_t root) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    if (root >= nranks) return invalid("root out of range");
    const uint64_t bytes = len * elem_size;
    PLAN_TRY(check_len(len));
    PLAN_TRY(check_present(send_root, len, "the root's send buffer is null"));
    PLAN_TRY(check_present(recv, nranks, len, "a receive buffer is null"));
    for (uint32_t a = 0; a < nranks; ++a) {
        for (uint32_t b = a + 1; b < nranks; ++b)
            if (overlaps(recv[a], bytes, recv[b], bytes)) return invalid("receive buffers of two ranks overlap");
        if (overlaps(recv[a], bytes, send_root, bytes) && !(a == root && recv[a] == send_root))
            return invalid("a receive buffer overlaps the root's send buffer out of place");
    }
    const void* in[kMaxRanks] = {};
    in[root] = send_root;
    // one pack copy, read once and written into every rank's buffer
    const uint64_t before = plan.steps.size();
    Status st = add_pack(plan, in, recv, nranks, bytes, kPackBroadcast, root, 1);
    if (st == MEGRAY_OK && plan.steps.size() > before) plan.bytes_written += bytes * (nranks - 1);
    return st;
}

Status plan_reduce(Plan& plan, const void* const* send, void* recv_root, uint32_t nranks, uint64_t len,
                   uint32_t elem_size, FoldOrder order, uint32_t root) {
    PLAN_TRY(check_ranks(nranks));
    PLAN_TRY(check_elem(elem_size));
    if (order < 0 || order >= kOrderCount) return invalid("unknown fold order");
    if (root >= nranks) return invalid("root out of range");
    const uint64_t bytes = len * elem_size;
    PLAN_TRY(check_len(len));
    PLAN_TRY(check_present(send, nranks, len, "a send buffer is null"));
    PLAN_TRY(check_present(recv_root, len, "the root's receive buffer is null"));
    for (uint32_t b = 0; b < nranks; ++b)
        if (overlaps(recv_root, bytes, send[b], bytes) && !(b == root && recv_root == send[b]))
            return invalid("the root's receive buffer overlaps a send buffer out of place");
    void* out[kMaxRanks] = {};
    out[root] = recv_root;
    if (order == kOrderUcx) {
        if (!len) return MEGRAY_OK;
        const uint64_t before_r = plan.bytes_read, before_w = plan.bytes_written;
        FoldBuilder fold(plan, send, out, nranks, nranks, 1, elem_size, false);
        if (fold.finish_tree(len, uint8_t(root))) return MEGRAY_OK;
        plan.bytes_read = before_r + bytes * nranks;
        plan.bytes_written = before_w + bytes;
        Step step;
        std::memset(&step, 0, sizeof(step));
        step.kind = Step::kTree;
        TreeLaunch& L = step.tree;
        for (uint32_t r = 0; r < nranks; ++r) L.in[r] = send[r];
        L.out = recv_root;
        L.count = len;
        L.nranks = nranks;
        L.root = root;
        L.elem_size = elem_size;
        // 16 bytes per lane wherever the buffers hold whole elements (128-bit accesses work at any byte address)
        uintptr_t bits = reinterpret_cast<uintptr_t>(recv_root);
        for (uint32_t r = 0; r < nranks; ++r) bits |= reinterpret_cast<uintptr_t>(send[r]);
        L.vector = (bits & (elem_size - 1)) == 0 ? 1 : 0;
        const uint64_t lanes = L.vector ? std::max<uint64_t>(len / (kVecBytes / elem_size), 1) : len;
        const uint64_t tiles = (lanes + kThreads - 1) / kThreads;
        if (tiles > 0x7fffffffull) return invalid("buffer too large for one tree launch");
        L.total_tiles = uint32_t(tiles);
        L.batch = tree_batch(nranks, elem_size, true, L.total_tiles);  // set_store_policy() has the last word
        plan.steps.push_back(step);
        return MEGRAY_OK;
    }
    const uint32_t nchunks = order_chunks(order, nranks);
    uint64_t sizes[kMaxChunks], offs[kMaxChunks];
    chunk_partition(len, nchunks, sizes, offs);
    FoldBuilder fold(plan, send, out, nranks, nranks, 1, elem_size, false);
    for (uint32_t c = 0; c < nchunks; ++c) {
        uint8_t start, owner;
        int8_t dir;
        chunk_fold_order(kAllReduce, order, nranks, c, &start, &dir, &owner);
        fold.add_run(offs[c], offs[c], sizes[c], start, dir, uint8_t(root));
    }
    fold.finish();
    return MEGRAY_OK;
}

Status plan_reduce2(Plan& plan, const void* i0, const void* i1, void* o, uint64_t len, uint32_t elem_size) {
    PLAN_TRY(check_elem(elem_size));
    PLAN_TRY(check_len(len));
    if (len && (!i0 || !i1 || !o)) return invalid("a buffer is null");
    const uint64_t bytes = len * elem_size;
    if ((overlaps(o, bytes, i0, bytes) && o != i0) || (overlaps(o, bytes, i1, bytes) && o != i1))
        return invalid("the output overlaps an input out of place");
    const void* in[kMaxRanks] = {i0, i1};
    void* out[kMaxRanks] = {o};
    // (i0 OP i1) with ties / unordered -> i1: i1 seeds the accumulator, i0 is folded in
    FoldBuilder fold(plan, in, out, 2, 2, 1, elem_size, false);
    fold.add_run(0, 0, len, 1, 1, 0);
    fold.finish();
    return MEGRAY_OK;
}

}  // namespace vrank
}  // namespace MegRay
