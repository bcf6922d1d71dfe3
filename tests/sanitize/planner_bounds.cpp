// Bounds harness of the multi-tensor planner, for the CPU (built with -fsanitize=address,undefined).
//
// It lays out random parameter lists with the library's own planner (csrc/gm_planner.cpp) and walks
// every descriptor the way the update kernels' grid does, through the same lane_share function the
// kernels index with, for every lane width, workgroup size and chunk size the library can launch.
// Checked for every case:
//   1. the chunks of a tensor tile it exactly once, in order, with no gap and no overlap;
//   2. every descriptor's range [p, p + count * elem) of every stream lies inside that stream's
//      allocation (views: inside the view's extent);
//   3. the lane shares of a chunk's workgroups tile [0, count) exactly once, and the grid
//      (chunks << slice shift) covers every chunk;
//   4. a vec-wide (grouped) access is aligned to its width in every stream;
//   5. for the lists that fit in memory, every share is really read and written through the
//      descriptor's pointers into exact-length heap blocks, under the address sanitizer.
// Two modes: "virtual" lists up to 2^28 elements per tensor live at made-up addresses (checks 1-4
// are pure arithmetic), "real" lists are small and allocated.
//
// usage: planner_bounds [cases] [seed]
#include "../../go-metal_amd/csrc/gm_planner.hpp"

#include <algorithm>
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <random>
#include <set>
#include <vector>

using namespace gm;

namespace {

struct Allocation {
    uintptr_t base;
    size_t bytes;
};
std::map<uintptr_t, size_t> g_registry;                 // what length_of reports (the library's own buffers)
size_t length_of(uintptr_t h)
{
    auto it = g_registry.find(h);
    return it == g_registry.end() ? 0 : it->second;
}

int g_failures = 0;
#define CHECK(cond, ...)                                                     \
    do {                                                                     \
        if (!(cond)) {                                                       \
            if (g_failures < 20) {                                           \
                std::fprintf(stderr, "FAIL %s:%d %s: ", __FILE__, __LINE__, #cond); \
                std::fprintf(stderr, __VA_ARGS__);                           \
                std::fprintf(stderr, "\n");                                  \
            }                                                                \
            g_failures++;                                                    \
        }                                                                    \
    } while (0)

struct Shape {
    int chunk, vec, block;     // chunk 0: the planner's choice
};

// (count, flags, chunk size, vec, block) combinations already walked lane by lane
std::set<std::tuple<uint32_t, uint32_t, int, int, int>> g_walked;

struct Case {
    int kind;
    uint32_t half_mask;
    int streams;                                   // slots in use: 0 .. streams-1 contiguous, plus weight16 for AMP
    std::vector<int> sizes;                        // bytes
    std::vector<uintptr_t> handle[kNumSlots];
    std::vector<size_t> extent[kNumSlots];         // bytes available behind each handle
    bool real = false;
};

bool slot_used(const Case &c, int k) { return !c.handle[k].empty(); }

void check_layout(const Case &c, const Shape &shape, const PlanLayout &L, const char *what)
{
    const int n = (int)c.sizes.size();
    CHECK(L.status == 0, "%s: status %d", what, L.status);
    CHECK(L.num_segments == 1 || L.num_segments == 2, "%s: %d segments", what, L.num_segments);
    CHECK(L.segment[0].first_chunk == 0 && L.segment[1].first_chunk == L.segment[0].num_chunks &&
              (size_t)L.segment[0].num_chunks + L.segment[1].num_chunks == L.chunks.size(),
          "%s: segments do not partition the table", what);

    // 1. tiling of every tensor
    std::vector<size_t> covered(n, 0);
    for (int s = 0; s < 2; s++) {
        const PlanSegment &seg = L.segment[s];
        for (uint32_t ci = seg.first_chunk; ci < seg.first_chunk + seg.num_chunks; ci++) {
            const Chunk &ch = L.chunks[ci];
            CHECK(ch.tensor < (uint32_t)n, "%s: chunk %u names tensor %u", what, ci, ch.tensor);
            if (ch.tensor >= (uint32_t)n) continue;
            const int t = (int)ch.tensor;
            const size_t numel = (size_t)c.sizes[t] / 4;
            CHECK(ch.count > 0 && ch.count <= (uint32_t)seg.chunk_elements, "%s: chunk %u count %u of %d", what, ci,
                  ch.count, seg.chunk_elements);
            for (int k = 0; k < kNumSlots; k++) {
                if (!slot_used(c, k) || c.handle[k][t] == 0) {
                    CHECK(ch.p[k] == nullptr, "%s: chunk %u has a pointer in unused stream %d", what, ci, k);
                    continue;
                }
                const size_t elem = (c.half_mask >> k) & 1 ? 2 : 4;
                const uintptr_t p = reinterpret_cast<uintptr_t>(ch.p[k]);
                // in order, no gap, no overlap: this chunk starts where the tensor's coverage so far ends
                CHECK(p == c.handle[k][t] + covered[t] * elem, "%s: chunk %u stream %d starts at +%zu, expected +%zu", what,
                      ci, k, (size_t)(p - c.handle[k][t]), covered[t] * elem);
                // 2. inside the allocation
                CHECK(p + (size_t)ch.count * elem <= c.handle[k][t] + c.extent[k][t],
                      "%s: chunk %u stream %d ends %zu bytes past its buffer", what, ci, k,
                      (size_t)(p + (size_t)ch.count * elem - c.handle[k][t] - c.extent[k][t]));
            }
            covered[t] += ch.count;
            CHECK(covered[t] <= numel, "%s: tensor %d covered %zu of %zu", what, t, covered[t], numel);
        }
    }
    uint64_t total = 0;
    for (int t = 0; t < n; t++) {
        const size_t numel = c.sizes[t] > 0 ? (size_t)c.sizes[t] / 4 : 0;
        bool short_buffer = false;
        for (int k = 0; k < kNumSlots; k++)
            if (slot_used(c, k) && c.handle[k][t] != 0) {
                const size_t elem = (c.half_mask >> k) & 1 ? 2 : 4;
                const size_t have = length_of(c.handle[k][t]);
                if (have != 0 && have < numel * elem) short_buffer = true;
            }
        if (short_buffer) CHECK(covered[t] == 0, "%s: tensor %d has a short buffer and must be skipped", what, t);
        else CHECK(covered[t] == numel, "%s: tensor %d covered %zu of %zu", what, t, covered[t], numel);
        total += covered[t];
    }
    CHECK(total == L.total_elements, "%s: total %" PRIu64 " vs %" PRIu64, what, total, L.total_elements);

    // 3 + 4 (+ 5): the grid's walk over every chunk
    for (int s = 0; s < L.num_segments; s++) {
        const PlanSegment &seg = L.segment[s];
        if (seg.num_chunks == 0) continue;
        uint32_t grid = 0, shift = 0;
        const bool fits = segment_grid(seg, shape.vec, shape.block, grid, shift);
        CHECK(fits, "%s: segment %d does not fit one launch", what, s);
        if (!fits) continue;
        CHECK((uint64_t)grid == (uint64_t)seg.num_chunks << shift, "%s: grid", what);
        CHECK(((uint64_t)shape.block * shape.vec << shift) >= (uint64_t)seg.chunk_elements,
              "%s: the slices of a chunk cover %llu of %d elements", what,
              (unsigned long long)((uint64_t)shape.block * shape.vec << shift), seg.chunk_elements);
        for (uint32_t ci = seg.first_chunk; ci < seg.first_chunk + seg.num_chunks; ci++) {
            const Chunk &ch = L.chunks[ci];
            const auto key = std::make_tuple(ch.count, ch.flags, seg.chunk_elements, shape.vec, shape.block);
            const bool repeat = ci > seg.first_chunk && ch.count == L.chunks[ci - 1].count && ch.flags == L.chunks[ci - 1].flags;
            const bool walk_shares = !repeat && g_walked.insert(key).second;
            if (!walk_shares && !c.real) continue;
            uint32_t next = 0;
            for (uint32_t slice = 0; slice < (1u << shift); slice++) {
                for (uint32_t lane = 0; lane < (uint32_t)shape.block; lane++) {
                    const LaneShare sh = lane_share(ch.count, ch.flags, slice, lane, shape.vec, shape.block);
                    if (sh.count == 0) {
                        CHECK((uint64_t)(slice * shape.block + lane) * shape.vec >= ch.count, "%s: idle lane inside the chunk", what);
                        continue;
                    }
                    CHECK(sh.first == next, "%s: chunk %u share starts at %u, expected %u", what, ci, sh.first, next);
                    CHECK(sh.count <= (uint32_t)shape.vec && sh.first + sh.count <= ch.count, "%s: share [%u, +%u) of %u", what,
                          sh.first, sh.count, ch.count);
                    CHECK(!sh.grouped || sh.count == (uint32_t)shape.vec, "%s: grouped share of %u", what, sh.count);
                    next = sh.first + sh.count;
                    for (int k = 0; k < kNumSlots; k++) {
                        if (ch.p[k] == nullptr) continue;
                        const size_t elem = (c.half_mask >> k) & 1 ? 2 : 4;
                        const uintptr_t a = reinterpret_cast<uintptr_t>(ch.p[k]) + (size_t)sh.first * elem;
                        if (sh.grouped) CHECK(a % (elem * shape.vec) == 0, "%s: grouped access of stream %d at %#zx is not %zu-byte aligned", what, k, (size_t)a, elem * shape.vec);
                        if (c.real) {
                            // the access itself, under the address sanitizer
                            volatile unsigned char *bytes = reinterpret_cast<volatile unsigned char *>(a);
                            for (size_t b = 0; b < sh.count * elem; b++) bytes[b] = (unsigned char)(bytes[b] + 1);
                        }
                    }
                }
            }
            CHECK(next == ch.count, "%s: chunk %u shares cover %u of %u", what, ci, next, ch.count);
        }
    }
}

// Every byte of every participating tensor was touched exactly once per walk (real cases).
void check_touch_counts(const Case &c, int walks, const char *what)
{
    for (int k = 0; k < kNumSlots; k++) {
        if (!slot_used(c, k)) continue;
        for (size_t t = 0; t < c.sizes.size(); t++) {
            if (c.handle[k][t] == 0) continue;
            const size_t elem = (c.half_mask >> k) & 1 ? 2 : 4;
            const size_t bytes = (size_t)c.sizes[t] / 4 * elem;
            const unsigned char *p = reinterpret_cast<const unsigned char *>(c.handle[k][t]);
            bool short_buffer = false;
            for (int j = 0; j < kNumSlots; j++)
                if (slot_used(c, j) && c.handle[j][t] != 0) {
                    const size_t e = (c.half_mask >> j) & 1 ? 2 : 4;
                    const size_t have = length_of(c.handle[j][t]);
                    if (have != 0 && have < (size_t)c.sizes[t] / 4 * e) short_buffer = true;
                }
            const size_t readable = std::min(bytes, c.extent[k][t]);
            const unsigned char want = short_buffer ? 0 : (unsigned char)walks;
            for (size_t b = 0; b < readable; b++) {
                if (p[b] != want) {
                    CHECK(false, "%s: stream %d tensor %zu byte %zu touched %u times, expected %u", what, k, t, b, p[b], want);
                    break;
                }
            }
        }
    }
}

const Shape kShapes[] = {
    {0, 1, 256}, {0, 2, 128}, {0, 1, 128}, {0, 2, 256}, {0, 4, 128}, {0, 4, 256}, {0, 2, 64}, {0, 1, 64},
    {256, 1, 128}, {256, 1, 256}, {1024, 4, 256}, {1024, 1, 64}, {4096, 2, 128}, {16384, 4, 128}, {65536, 1, 256},
    {65536, 4, 256}, {65536, 2, 64},
};

struct RuleShape {
    int kind;
    int fp32_states;
    bool amp;
};
const RuleShape kRules[] = {{kRuleSGD, 0, false},     {kRuleSGD, 1, false},     {kRuleAdam, 2, false}, {kRuleRMSProp, 3, false},
                            {kRuleAdaGrad, 1, false}, {kRuleAdaDelta, 2, false}, {kRuleAdamAMP, 2, true}};

void run_case(std::mt19937_64 &rng, bool real, int index)
{
    auto uniform = [&](uint64_t lo, uint64_t hi) { return lo + rng() % (hi - lo + 1); };
    Case c;
    c.real = real;
    const RuleShape rule = kRules[uniform(0, sizeof kRules / sizeof kRules[0] - 1)];
    c.kind = rule.kind;
    c.half_mask = rule.amp ? (1u << kSlotGrad) | (1u << kSlotWeight16) : 0;
    std::vector<int> slots = {kSlotWeight, kSlotGrad};
    for (int k = 0; k < rule.fp32_states; k++) slots.push_back(kSlotState0 + k);
    if (rule.amp) slots.push_back(kSlotWeight16);

    // sizes: a mix of edge values and log-uniform draws
    const uint64_t edge[] = {0, 1, 2, 3, 63, 64, 65, 127, 255, 256, 257, 511, 512, 513, 1023, 1024, 1025, 4095, 4096, 4097,
                             16383, 16384, 16385, 65535, 65536, 65537, 131071, 131073};
    const int n = (int)uniform(1, real ? 24 : 400);
    const uint64_t max_elems = real ? (1u << 16) : (1u << 28);
    uint64_t budget = real ? (1u << 17) : (1ull << 29) + 64;  // elements per stream (real cases allocate them)
    for (int t = 0; t < n; t++) {
        uint64_t numel;
        const uint64_t pick = uniform(0, 9);
        if (pick < 4) numel = edge[uniform(0, sizeof edge / sizeof edge[0] - 1)];
        else {
            const double lg = (double)uniform(0, 1000000) / 1e6 * std::log2((double)max_elems);
            numel = (uint64_t)std::exp2(lg);
        }
        if (!real && t == 0 && uniform(0, 3) == 0) numel = (1u << 28) + uniform(0, 5);   // the largest a C int of bytes allows is 2^29 - 1
        numel = std::min<uint64_t>(numel, (1u << 29) - 1);
        if (numel > budget) numel = budget;
        budget -= numel;
        c.sizes.push_back((int)(numel * 4));
    }

    // buffers: own allocation per tensor and stream, registered with its exact or a padded length; or a view at
    // an odd offset into a larger block (length unknown to the registry); now and then too short (skipped tensor)
    uintptr_t next_virtual = 0x7000'0000'0000ull;
    std::vector<void *> blocks;
    g_registry.clear();
    for (int k : slots) {
        c.handle[k].assign(n, 0);
        c.extent[k].assign(n, 0);
    }
    for (int t = 0; t < n; t++) {
        const size_t numel = (size_t)c.sizes[t] / 4;
        const bool make_short = numel > 8 && uniform(0, 24) == 0;
        for (int k : slots) {
            const size_t elem = (c.half_mask >> k) & 1 ? 2 : 4;
            size_t bytes = numel * elem;
            const uint64_t style = uniform(0, 9);            // 0-5 own exact, 6-7 own padded to 16, 8-9 view
            size_t misalign = 0;
            bool registered = true;
            if (style >= 8) {
                misalign = elem * uniform(1, 7);
                registered = false;
            } else if (style >= 6) {
                bytes = (bytes + 15) / 16 * 16;
            }
            if (make_short && k == slots.back()) {
                bytes = numel * elem - elem * uniform(1, std::min<size_t>(numel - 1, 300));
                registered = true;
                misalign = 0;
            }
            uintptr_t h;
            if (real) {
                unsigned char *block = static_cast<unsigned char *>(std::malloc(std::max<size_t>(bytes + misalign, 1)));
                std::memset(block, 0, bytes + misalign);
                blocks.push_back(block);
                h = reinterpret_cast<uintptr_t>(block) + misalign;
            } else {
                h = next_virtual + misalign;
                next_virtual += (bytes + misalign + 4095) / 4096 * 4096 + 4096;
            }
            c.handle[k][t] = h;
            c.extent[k][t] = bytes;
            if (registered) g_registry[h] = bytes;
        }
    }

    PlanRequest req{};
    req.kind = c.kind;
    req.num_tensors = n;
    for (int k : slots) req.slot[k] = c.handle[k].data();
    req.sizes = c.sizes.data();
    req.required_mask = (1u << kSlotWeight) | (1u << kSlotGrad);
    req.missing_code = -4;
    req.half_mask = c.half_mask;

    int walks = 0;
    uint64_t total_elements = 0;
    for (int t = 0; t < n; t++) total_elements += (uint64_t)c.sizes[t] / 4;
    for (const Shape &shape : kShapes) {
        if (shape.chunk != 0 && shape.chunk < shape.block * shape.vec) continue;     // gm_set_tuning refuses these
        if (shape.chunk != 0 && total_elements / (uint64_t)shape.chunk > (1u << 19)) continue;   // a table of over 32 MiB
        PlanLayout L;
        layout_plan(req, shape.chunk, length_of, L);
        char what[160];
        std::snprintf(what, sizeof what, "case %d (%s, rule %d, %d tensors) chunk %d vec %d block %d", index,
                      real ? "real" : "virtual", c.kind, n, shape.chunk, shape.vec, shape.block);
        check_layout(c, shape, L, what);
        walks++;
        if (shape.chunk == 0) {
            // the planner's own choices obey their stated rules
            uint64_t working = 0, launched = 0;
            for (int t = 0; t < n; t++) {
                const uint64_t numel = (uint64_t)c.sizes[t] / 4;
                working += (numel + 255) / 256;
                launched += (numel + L.chunk_elements - 1) / L.chunk_elements * (L.chunk_elements / 256);
            }
            if (L.chunk_elements > 256)
                CHECK(launched - working <= (uint64_t)(0.05 * (double)working), "%s: chunk %d idles %llu of %llu", what,
                      L.chunk_elements, (unsigned long long)(launched - working), (unsigned long long)working);
            if (L.num_segments == 2) CHECK(L.segment[1].chunk_elements < L.segment[0].chunk_elements && L.segment[1].chunk_elements >= 256, "%s: segment sizes", what);
        }
    }
    if (real) {
        char what[64];
        std::snprintf(what, sizeof what, "case %d touch counts", index);
        check_touch_counts(c, walks, what);
    }
    for (void *b : blocks) std::free(b);
}

// A list known to need two segments (the GPU guard test uses the same one).
void two_segment_case()
{
    std::vector<int> small = {1, 255, 256, 257, 1023, 1025, 4095, 4097, 5, 300, 77, 2049};
    std::vector<int> sizes;
    for (int i = 0; i < 40; i++) sizes.push_back(small[i % 12] * 4);
    sizes.push_back(120000001 * 4);
    for (int i = 40; i < 80; i++) sizes.push_back(small[i % 12] * 4);
    const int n = (int)sizes.size();
    std::vector<uintptr_t> w(n), g(n);
    uintptr_t next = 0x7000'0000'0000ull;
    for (int t = 0; t < n; t++) {
        w[t] = next;
        next += ((size_t)sizes[t] + 4095) / 4096 * 4096 + 4096;
        g[t] = next;
        next += ((size_t)sizes[t] + 4095) / 4096 * 4096 + 4096;
    }
    PlanRequest req{};
    req.num_tensors = n;
    req.slot[kSlotWeight] = w.data();
    req.slot[kSlotGrad] = g.data();
    req.sizes = sizes.data();
    PlanLayout L;
    g_registry.clear();
    layout_plan(req, 0, length_of, L);
    CHECK(L.num_segments == 2 && L.segment[0].chunk_elements == 65536 && L.segment[1].num_chunks >= 80,
          "two-segment list: %d segments, chunk %d, %u small chunks", L.num_segments, L.segment[0].chunk_elements,
          L.segment[1].num_chunks);
}

}  // namespace

int main(int argc, char **argv)
{
    const int cases = argc > 1 ? std::atoi(argv[1]) : 300;
    const uint64_t seed = argc > 2 ? std::strtoull(argv[2], nullptr, 0) : 0x6d657461;
    std::mt19937_64 rng(seed);
    two_segment_case();
    for (int i = 0; i < cases; i++) run_case(rng, /*real=*/i % 3 == 0, i);
    std::printf("planner_bounds: %d cases x %zu launch shapes, %zu distinct chunk walks, %d failures\n", cases,
                sizeof kShapes / sizeof kShapes[0], g_walked.size(), g_failures);
    return g_failures == 0 ? 0 : 1;
}
