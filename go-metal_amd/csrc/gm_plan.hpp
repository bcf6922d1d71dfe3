// Multi-tensor launch plan: the device-side tables one update launch walks.
//
// A step over a parameter list is ONE kernel launch.  The host flattens the
// list into fixed-size chunks; a chunk is shared by a fixed number of
// consecutive workgroups (one slice each).  One table lives in HBM and is
// rebuilt only when the caller's handles change:
//
//   Chunk chunks[num_chunks]   the address of the chunk's first element in
//                              every stream, the element count and flags
//
// A descriptor is one 64-byte line, fetched by a single wave-uniform (scalar)
// load that hits in cache for all but the first workgroup of the chunk
// (64 bytes of table per 4096..65536 elements).
#pragma once

#include "gm_context.hpp"

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

struct MultiTensorPlan {
    // ---- key ----
    int kind = 0;
    int variant = 0;             // rule-specific bits that change validation (e.g. which optional states are on)
    int num_tensors = 0;
    int requested_chunk_elements = 0;   // 0: chosen by the planner
    int chunk_elements = 0;             // the size in force for this plan's first segment
    uint64_t generation = 0;
    std::vector<uintptr_t> handles;   // kNumSlots * num_tensors, slot-major
    std::vector<int> sizes;
    // ---- result ----
    int status = 0;              // validation result: 0 or the entry point's error code
    Chunk *d_chunks = nullptr;
    uint32_t num_chunks = 0;     // all segments together
    PlanSegment segment[2];
    int num_segments = 0;
    uint64_t total_elements = 0;
    ~MultiTensorPlan();
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

// Returns the cached plan for this request or builds one (under ctx->mu, which
// the caller holds).  nullptr on a HIP failure (error already recorded).
MultiTensorPlan *get_plan(Context *ctx, const PlanRequest &req);

// Elements per chunk forced by the caller (tunable for sweeps); 0 = chosen per plan.
int current_chunk_elements();
// Whether streaming accesses carry the non-temporal hint.
bool current_nontemporal();
// fp32 elements per lane (1, 2 or 4).
int current_vec();

}  // namespace gm
