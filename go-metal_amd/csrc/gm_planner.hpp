// Chunk-table layout of a multi-tensor launch: plain C++ with no HIP dependency, so the same
// code that feeds the kernels also compiles for the CPU, where a bounds harness walks every
// descriptor the way the grid does and an address sanitizer watches the accesses.
//
// A step over a parameter list is one kernel launch per segment.  The host flattens the list
// into fixed-size chunks; a chunk is shared by a fixed number of consecutive workgroups (one
// slice each).  One table lives in HBM and is rebuilt only when the caller's handles change:
//
//   Chunk chunks[num_chunks]   the address of the chunk's first element in every stream, the
//                              element count and flags
//
// A descriptor is one 64-byte line, fetched by a single wave-uniform (scalar) load that hits
// in cache for all but the first workgroup of the chunk (64 bytes of table per 256..65536
// elements).
#pragma once

#include <cstddef>
#include <cstdint>
#include <vector>

namespace gm {

// Stream slots of a tensor record.
enum : int {
    kSlotWeight = 0,
    kSlotGrad = 1,     // fp32, or fp16 for the mixed-precision step
    kSlotState0 = 2,
    kSlotState1 = 3,
    kSlotState2 = 4,
    kSlotWeight16 = 5,
    kNumSlots = 6,
};

enum : uint32_t {
    kRecVec2Ok = 1u,         // every used stream is aligned for 2-element lanes (8 B fp32 / 4 B fp16)
    kRecVec4Ok = 2u,         // ... for 4-element lanes (16 B fp32 / 8 B fp16)
    kRecGrad16VectorOk = 4u, // the fp16 gradient is 16-byte aligned (overflow-check kernel)
};

struct alignas(64) Chunk {
    void *p[kNumSlots];   // first element of this chunk in each stream (nullptr: stream unused)
    uint32_t count;       // elements in this chunk (<= chunk_elements)
    uint32_t flags;
    uint32_t tensor;      // index into the caller's list (diagnostics only)
    uint32_t pad;
};
static_assert(sizeof(Chunk) == 64, "Chunk layout");

// Which update rule a plan (and its validation) was built for.
enum RuleKind : int {
    kRuleSGD = 0,
    kRuleAdam,
    kRuleRMSProp,
    kRuleAdaGrad,
    kRuleAdaDelta,
    kRuleNAdam,
    kRuleAdamAMP,
};

// A run of chunks of one size inside the table.  A list whose small tensors would leave many
// workgroups of the list's chunk size idle gets a second segment with a smaller chunk size for
// them; each segment is one launch of the update kernel.
struct PlanSegment {
    uint32_t first_chunk = 0;
    uint32_t num_chunks = 0;
    int chunk_elements = 0;
};

// What an entry point hands to the planner.  slot[k] is the caller's handle
// array for stream k (nullptr = stream unused by this rule: all zeros).
struct PlanRequest {
    int kind;
    int variant;
    int num_tensors;
    const uintptr_t *slot[kNumSlots];
    const int *sizes;            // bytes of the fp32 weight tensor
    uint32_t required_mask;      // slots whose handle must be non-zero ...
    int missing_code;            // ... else the step fails with this code (0: skip that tensor instead)
    uint32_t skip_if_zero_mask;  // slots whose zero handle makes the tensor be skipped (when missing_code == 0)
    uint32_t half_mask;          // slots holding fp16 elements (length and alignment checks)
    // Optional extra per-tensor check run on a cache miss; returns a non-zero
    // error code to fail the step.
    int (*extra_check)(const PlanRequest &req, int tensor);
};

// Allocation length in bytes of a buffer handle, 0 when the handle is not one of the library's.
typedef size_t (*BufferLengthFn)(uintptr_t handle);

constexpr int kPlanBlock = 256;                                        // lanes the chunk sizes are counted in
constexpr int kChunkCandidates[] = {65536, 16384, 4096, 1024, 256};    // largest first
constexpr int kNumChunkCandidates = (int)(sizeof(kChunkCandidates) / sizeof(int));

// Elements of tensor i (its byte size / 4; 0 for a non-positive size).
inline size_t tensor_elements(const PlanRequest &r, int i)
{
    return r.sizes[i] > 0 ? (size_t)r.sizes[i] / sizeof(float) : 0;
}

// Chunk size for a tensor list when the caller has not fixed one: the largest candidate whose
// idle workgroups stay below 5 % of the working ones.
int choose_chunk_elements(const PlanRequest &r);

// The chunk size for the tensors below `limit` elements when they are worth a segment of their
// own (0 otherwise): the largest candidate under the list's chunk size that keeps their idle
// workgroups below 5 % of their working ones.  `limit` is set to chunk / 4.
int choose_small_segment(const PlanRequest &r, int chunk, size_t &limit);

// The verdict on one tensor of a request.
struct TensorCheck {
    int status = 0;        // non-zero: the whole step fails with this code
    bool skip = false;     // the tensor takes no part in the step
    uint32_t flags = 0;    // kRec* alignment flags of its streams
    size_t numel = 0;
};
TensorCheck check_tensor(const PlanRequest &r, int i, BufferLengthFn length_of);

// The table of one request.
struct PlanLayout {
    int status = 0;                 // validation result: 0 or the entry point's error code
    int chunk_elements = 0;         // the size in force for the first segment
    PlanSegment segment[2];
    int num_segments = 0;
    uint64_t total_elements = 0;
    uint64_t kept_signature = 0;    // hash over the indices of the tensors that take part, in order: two
                                    // layouts of the same sizes pair chunk for chunk only if it is equal
    std::vector<Chunk> chunks;      // segment 0's, then segment 1's
};

// Lays the request out.  requested_chunk > 0 fixes one chunk size for the whole list.
void layout_plan(const PlanRequest &r, int requested_chunk, BufferLengthFn length_of, PlanLayout &out);

#if defined(__HIPCC__)
#define GM_HOST_DEVICE __host__ __device__
#else
#define GM_HOST_DEVICE
#endif

// One lane's share of a chunk: elements [first, first + count) of every stream.  `grouped`: the
// share is one aligned vec-wide access per stream; otherwise its elements are accessed one by one
// (a chunk's tail, or streams whose handles are not aligned for vec-wide lanes).  count == 0: the
// lane lies past the chunk's end.  The update kernels and the CPU bounds harness both index
// through this function.
struct LaneShare {
    uint32_t first;
    uint32_t count;
    bool grouped;
};
GM_HOST_DEVICE inline LaneShare lane_share(uint32_t chunk_count, uint32_t chunk_flags, uint32_t slice, uint32_t lane,
                                           uint32_t vec, uint32_t block)
{
    LaneShare s{(slice * block + lane) * vec, 0u, false};
    if (s.first >= chunk_count) return s;
    const uint32_t vec_flag = vec == 4 ? kRecVec4Ok : kRecVec2Ok;
    if (vec > 1 && (chunk_flags & vec_flag) != 0 && s.first + vec <= chunk_count) {
        s.count = vec;
        s.grouped = true;
    } else {
        const uint32_t left = chunk_count - s.first;
        s.count = left < vec ? left : vec;
    }
    return s;
}

// log2(slices per chunk) for a chunk size, lane width and workgroup size; chunk_elements is a
// power-of-two multiple of block * vec.
uint32_t slice_shift_for(int chunk_elements, int vec, int block);

// Workgroups and slice shift of one segment's launch; false when the segment needs more
// workgroups than one launch can address.
bool segment_grid(const PlanSegment &seg, int vec, int block, uint32_t &grid, uint32_t &shift);

}  // namespace gm
