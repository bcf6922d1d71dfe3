// Chunk-table layout of a multi-tensor launch (no HIP dependency: see gm_planner.hpp).
#include "gm_planner.hpp"

namespace gm {

constexpr double kMaxIdleFraction = 0.05;
// Tensors shorter than a quarter of the list's chunk leave three quarters and more of their chunk's
// workgroups idle.  An idle workgroup costs about 0.6 ns and a second launch about 5 us (measured on
// MI355X), so those tensors move to a segment of their own, with a smaller chunk, once they would
// idle this many workgroups.  The 1B-parameter transformer list qualifies (360 vectors of 4096
// elements in 65536-element chunks: 86k idle workgroups; the step is 4 to 11 us of 4.32 ms faster
// with the second segment, alternated with the single-launch plan in one process).
constexpr uint64_t kSplitMinIdleWorkgroups = 16384;

// Working and launched workgroups of the tensors in [lo, hi) elements under one chunk size.
static void count_workgroups(const PlanRequest &r, int candidate, size_t lo, size_t hi, uint64_t &working,
                             uint64_t &launched)
{
    const uint64_t per_chunk = (uint64_t)candidate / kPlanBlock;
    working = launched = 0;
    for (int i = 0; i < r.num_tensors; i++) {
        const uint64_t numel = tensor_elements(r, i);
        if (numel < lo || numel >= hi) continue;
        working += (numel + kPlanBlock - 1) / kPlanBlock;
        launched += (numel + candidate - 1) / candidate * per_chunk;
    }
}

// A chunk's descriptor is fetched once per workgroup, and that fetch is the only latency a
// workgroup cannot overlap, so large chunks (many workgroups sharing one cached descriptor) are
// faster; but every chunk launches a full set of slices, and the slices past a tensor's end are
// idle workgroups.  Lists of small tensors end up with small chunks, down to one descriptor per
// workgroup: measured on MI355X, Adam over 5000 tensors of 64 to 2048 elements takes 64 us per
// step with 4096-element chunks (15 of 16 workgroups idle for most tensors) and 26 us with
// 256-element chunks, while lists of large tensors lose 3 to 4 points of bandwidth below 4096.
int choose_chunk_elements(const PlanRequest &r)
{
    for (int candidate : kChunkCandidates) {
        uint64_t working, launched;
        count_workgroups(r, candidate, 1, (size_t)-1, working, launched);
        if (launched - working <= (uint64_t)(kMaxIdleFraction * (double)working)) return candidate;
    }
    return kChunkCandidates[kNumChunkCandidates - 1];
}

int choose_small_segment(const PlanRequest &r, int chunk, size_t &limit)
{
    limit = (size_t)chunk / 4;
    uint64_t working, launched;
    count_workgroups(r, chunk, 1, limit, working, launched);
    if (launched - working < kSplitMinIdleWorkgroups) return 0;
    int last = 0;
    for (int candidate : kChunkCandidates) {
        if (candidate >= chunk) continue;
        last = candidate;
        count_workgroups(r, candidate, 1, limit, working, launched);
        if (launched - working <= (uint64_t)(kMaxIdleFraction * (double)working)) return candidate;
    }
    return last;
}

TensorCheck check_tensor(const PlanRequest &r, int i, BufferLengthFn length_of)
{
    TensorCheck t;
    uintptr_t h[kNumSlots];
    for (int k = 0; k < kNumSlots; k++) h[k] = r.slot[k] ? r.slot[k][i] : 0;

    // 1. handles that must be present
    for (int k = 0; k < kNumSlots; k++) {
        if (h[k] != 0) continue;
        if (r.required_mask & (1u << k)) {
            if (r.missing_code != 0) {
                t.status = r.missing_code;
                return t;
            }
            t.skip = true;
        } else if (r.skip_if_zero_mask & (1u << k)) {
            t.skip = true;
        }
    }
    if (r.extra_check) {
        t.status = r.extra_check(r, i);
        if (t.status != 0) return t;
    }
    t.numel = tensor_elements(r, i);
    if (t.skip || t.numel == 0) {
        t.skip = true;
        return t;
    }

    // 2. an allocation of ours that is shorter than the tensor: skip it
    //    (bridge_optimizer.m:427-436)
    t.flags = kRecVec2Ok | kRecVec4Ok | kRecGrad16VectorOk;
    for (int k = 0; k < kNumSlots; k++) {
        if (h[k] == 0) continue;
        const bool half = (r.half_mask & (1u << k)) != 0;
        const size_t need = t.numel * (half ? 2 : 4);
        const size_t have = length_of ? length_of(h[k]) : 0;
        if (have != 0 && have < need) t.skip = true;
        if (h[k] % (half ? 4 : 8) != 0) t.flags &= ~kRecVec2Ok;
        if (h[k] % (half ? 8 : 16) != 0) t.flags &= ~kRecVec4Ok;
        if (half && k == kSlotGrad && h[k] % 16 != 0) t.flags &= ~kRecGrad16VectorOk;
    }
    return t;
}

void layout_plan(const PlanRequest &r, int requested_chunk, BufferLengthFn length_of, PlanLayout &out)
{
    out = PlanLayout{};
    const int chunk = requested_chunk > 0 ? requested_chunk : choose_chunk_elements(r);
    size_t small_limit = 0;
    const int small_chunk = requested_chunk > 0 ? 0 : choose_small_segment(r, chunk, small_limit);
    out.chunk_elements = chunk;

    std::vector<Chunk> small_chunks;
    for (int i = 0; i < r.num_tensors; i++) {
        const TensorCheck t = check_tensor(r, i, length_of);
        if (t.status != 0) {
            out.status = t.status;
            break;
        }
        if (t.skip) continue;
        out.kept_signature = (out.kept_signature ^ (uint64_t)(i + 1)) * 0x100000001B3ull;     // FNV-1a over indices
        const bool in_small_segment = small_chunk != 0 && t.numel < small_limit;
        const size_t step = (size_t)(in_small_segment ? small_chunk : chunk);
        std::vector<Chunk> &table = in_small_segment ? small_chunks : out.chunks;
        for (size_t off = 0; off < t.numel; off += step) {
            const size_t left = t.numel - off;
            Chunk c{};
            for (int k = 0; k < kNumSlots; k++) {
                const uintptr_t h = r.slot[k] ? r.slot[k][i] : 0;
                if (h == 0) continue;
                const size_t elem = (r.half_mask & (1u << k)) ? 2 : 4;
                c.p[k] = reinterpret_cast<void *>(h + off * elem);
            }
            c.count = (uint32_t)(left < step ? left : step);
            c.flags = t.flags;
            c.tensor = (uint32_t)i;
            table.push_back(c);
        }
        out.total_elements += t.numel;
    }
    if (out.status != 0) {
        out.chunks.clear();
        small_chunks.clear();
    }
    out.segment[0] = PlanSegment{0, (uint32_t)out.chunks.size(), chunk};
    out.segment[1] = PlanSegment{(uint32_t)out.chunks.size(), (uint32_t)small_chunks.size(), small_chunk};
    out.num_segments = small_chunks.empty() ? 1 : 2;
    out.chunks.insert(out.chunks.end(), small_chunks.begin(), small_chunks.end());
}

uint32_t slice_shift_for(int chunk_elements, int vec, int block)
{
    const uint32_t slices = (uint32_t)(chunk_elements / (block * vec));
    uint32_t shift = 0;
    while ((1u << shift) < slices) shift++;
    return shift;
}

bool segment_grid(const PlanSegment &seg, int vec, int block, uint32_t &grid, uint32_t &shift)
{
    shift = slice_shift_for(seg.chunk_elements, vec, block);
    const uint64_t blocks = (uint64_t)seg.num_chunks << shift;
    if (blocks > 0x7FFFFFFFull) return false;
    grid = (uint32_t)blocks;
    return true;
}

}  // namespace gm
