// Cached multi-tensor launch plans: a laid-out chunk table (gm_planner.hpp) resident in HBM,
// keyed by the caller's handle arrays.
#pragma once

#include "gm_context.hpp"
#include "gm_planner.hpp"

namespace gm {

// Device memory for one chunk table with its pinned host twin.  The host fills the pinned copy
// and enqueues one asynchronous upload; nothing waits for it but the kernels behind it on the
// stream.  Slots are recycled through the context's free list instead of being freed, so neither
// building nor dropping a plan allocates, frees or synchronises once the slots exist.
struct TableSlot {
    Chunk *d_chunks = nullptr;
    Chunk *h_chunks = nullptr;       // hipHostMalloc
    size_t capacity = 0;             // descriptors
    hipEvent_t uploaded = nullptr;   // completion of the last upload that read h_chunks
    bool upload_pending = false;
};

struct MultiTensorPlan {
    // ---- key ----
    int kind = 0;
    int variant = 0;             // rule-specific bits that change validation (e.g. which optional states are on)
    int num_tensors = 0;
    int requested_chunk_elements = 0;   // 0: chosen by the planner
    std::vector<uintptr_t> handles;   // kNumSlots * num_tensors, slot-major
    std::vector<int> sizes;
    // ---- result ----
    int status = 0;              // validation result: 0 or the entry point's error code
    int chunk_elements = 0;      // the size in force for this plan's first segment
    TableSlot table;
    Chunk *d_chunks = nullptr;   // table.d_chunks (nullptr for an empty plan)
    uint32_t num_chunks = 0;     // all segments together
    PlanSegment segment[2];
    int num_segments = 0;
    uint64_t total_elements = 0;
    uint64_t kept_signature = 0;  // PlanLayout::kept_signature
};

// Returns the cached plan for this request or builds one (under ctx->mu, which
// the caller holds).  nullptr on a HIP failure (error already recorded).
MultiTensorPlan *get_plan(Context *ctx, const PlanRequest &req);

// Drops every cached plan with a handle inside [begin, begin + bytes): called (under ctx->mu)
// when that allocation is freed, since the address may come back with another length.  Plans
// that do not touch the range stay valid.
void plans_forget_range(Context *ctx, uintptr_t begin, size_t bytes);

// The context's launch-shape settings.
// Elements per chunk forced by the caller (tunable for sweeps); 0 = chosen per plan.
int current_chunk_elements(const Context *ctx);
// Whether streaming accesses carry the non-temporal hint.
bool current_nontemporal(const Context *ctx);
// fp32 elements per lane (1, 2 or 4); 0 = chosen per launch.
int current_vec(const Context *ctx);
// Lanes per workgroup of the update kernels; 0 = chosen per launch.
int current_block(const Context *ctx);

}  // namespace gm
