// The Adam step for callers that cannot allocate: code under HIP graph capture, tight serving
// loops, harnesses that forbid hipMalloc.  Same arithmetic and the same update kernel as
// execute_adam_step_mpsgraph; what differs is where the chunk table lives and how it gets there.
//
// The table sits in a file-scope __device__ array (one copy per GPU, held until the process
// ends) instead of a cached hipMalloc allocation, and it is written by a small kernel from
// tensor records passed as kernel arguments, 64 tensors per launch, instead of being uploaded:
// the entry point calls no hipMalloc, no hipFree, no copy and no other allocating routine, and
// never waits for the device.  Every call on a GPU rewrites that GPU's one table, so calls that
// overlap on one GPU (other than back to back on the library's stream, where they are ordered)
// race.
#include "gm_launch.hpp"
#include "gm_update_kernels.hpp"

#include "../../include/gometal_hip.h"

namespace gm {

constexpr uint32_t kNoAllocMaxChunks = 32768;     // descriptors: 2 MiB of table per GPU
constexpr int kNoAllocMaxTensors = 4096;
constexpr int kNoAllocBatch = 64;                 // tensor records per table-kernel launch (3 KiB of arguments)

static __device__ __align__(256) unsigned char scratch[(size_t)kNoAllocMaxChunks * sizeof(Chunk)];

// In host code `scratch` is only a stand-in for the symbol; each GPU's copy has its own
// address, resolved here once per context and used everywhere else.
bool noalloc_bind_scratch(Context *ctx)
{
    void *ptr = nullptr;
    if (!hip_ok(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)), "hipGetSymbolAddress(scratch)")) return false;
    ctx->noalloc_scratch = ptr;
    return true;
}

struct NoAllocTensor {
    uintptr_t w, g, m, v;
    uint32_t numel;
    uint32_t first_chunk;     // position of the tensor's first descriptor in the table
    uint32_t flags;
    uint32_t index;           // position in the caller's list (diagnostics only)
};
struct NoAllocBatch {
    NoAllocTensor t[kNoAllocBatch];
};
static_assert(sizeof(NoAllocBatch) <= 3072, "the records travel as kernel arguments");

// One workgroup per tensor record: writes the tensor's descriptors, the same ones layout_plan
// produces on the host for a single segment of chunk_elements.
__global__ void __launch_bounds__(64)
noalloc_table_kernel(NoAllocBatch batch, uint32_t chunk_elements, Chunk *__restrict__ table)
{
    const NoAllocTensor t = batch.t[blockIdx.x];
    const uint32_t chunks = (t.numel + chunk_elements - 1) / chunk_elements;
    for (uint32_t c = threadIdx.x; c < chunks; c += 64) {
        const size_t off = (size_t)c * chunk_elements;
        const uint32_t left = t.numel - (uint32_t)off;
        Chunk d{};
        d.p[kSlotWeight] = reinterpret_cast<void *>(t.w + off * sizeof(float));
        d.p[kSlotGrad] = reinterpret_cast<void *>(t.g + off * sizeof(float));
        d.p[kSlotState0] = reinterpret_cast<void *>(t.m + off * sizeof(float));
        d.p[kSlotState1] = reinterpret_cast<void *>(t.v + off * sizeof(float));
        d.count = left < chunk_elements ? left : chunk_elements;
        d.flags = t.flags;
        d.tensor = t.index;
        table[t.first_chunk + c] = d;
    }
}

}  // namespace gm

using namespace gm;

extern "C" {

int execute_adam_step_noalloc(uintptr_t device, uintptr_t *weight_buffers, uintptr_t *gradient_buffers,
                              uintptr_t *momentum_buffers, uintptr_t *variance_buffers, int num_weights,
                              int *buffer_sizes, float learning_rate, float beta1, float beta2,
                              float epsilon, float weight_decay, int step_count)
try {
    clear_error();
    if (device == 0) {
        set_error("device handle is nil");
        return -1;
    }
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (num_weights < 0 || (num_weights > 0 && (!buffer_sizes || !weight_buffers || !gradient_buffers))) {
        set_error("weight, gradient and size arrays are required");
        return -6;
    }
    if (num_weights > kNoAllocMaxTensors) {
        set_error("the allocation-free step takes at most %d tensors (got %d); use execute_adam_step_mpsgraph",
                  kNoAllocMaxTensors, num_weights);
        return -17;
    }
    if (!make_current(ctx)) return -6;
    Chunk *table = static_cast<Chunk *>(ctx->noalloc_scratch);
    if (!table) {
        set_error("the descriptor table of the allocation-free step was not resolved on this GPU");
        return -6;
    }

    PlanRequest req{};
    req.kind = kRuleAdam;
    req.num_tensors = num_weights;
    req.slot[kSlotWeight] = weight_buffers;
    req.slot[kSlotGrad] = gradient_buffers;
    req.slot[kSlotState0] = momentum_buffers;
    req.slot[kSlotState1] = variance_buffers;
    req.sizes = buffer_sizes;
    req.required_mask = (1u << kSlotWeight) | (1u << kSlotGrad) | (1u << kSlotState0) | (1u << kSlotState1);
    req.missing_code = -4;

    std::lock_guard<std::mutex> lock(ctx->mu);

    // Pass 1, nothing launched yet: every tensor is validated (a failure must leave every buffer
    // untouched) and the verdicts are kept on the stack.
    unsigned char keep[kNoAllocMaxTensors];
    unsigned char flags[kNoAllocMaxTensors];
    for (int i = 0; i < num_weights; i++) {
        const TensorCheck t = check_tensor(req, i, registry_length);
        if (t.status != 0) {
            set_error("a required buffer handle is nil (code %d)", t.status);
            return t.status;
        }
        keep[i] = t.skip ? 0 : 1;
        flags[i] = (unsigned char)t.flags;
    }

    // The list's chunk size, as the caching entry point chooses it for a single segment; if the
    // table would not fit, the next larger sizes are tried (more idle workgroups, same results).
    int chunk = current_chunk_elements(ctx);
    const bool chunk_forced = chunk != 0;
    if (!chunk_forced) chunk = choose_chunk_elements(req);
    uint64_t total_chunks = 0;
    for (;;) {
        total_chunks = 0;
        for (int i = 0; i < num_weights; i++)
            if (keep[i]) total_chunks += (tensor_elements(req, i) + (size_t)chunk - 1) / (size_t)chunk;
        if (total_chunks <= kNoAllocMaxChunks || chunk_forced || chunk >= kChunkCandidates[0]) break;
        chunk *= 4;      // the candidate sizes are a factor of four apart
    }
    if (total_chunks > kNoAllocMaxChunks) {
        set_error("the allocation-free step holds %u chunk descriptors; this list needs %llu in chunks of %d "
                  "elements (about 2.1e9 parameters fit in chunks of 65536); use execute_adam_step_mpsgraph",
                  kNoAllocMaxChunks, (unsigned long long)total_chunks, chunk);
        return -17;
    }
    if (total_chunks == 0) return 0;

    int vec = current_vec(ctx), block = current_block(ctx);
    if (vec == 0) vec = auto_vec(7);
    if (block == 0) block = auto_block(7);
    const PlanSegment segment{0, (uint32_t)total_chunks, chunk};
    SegmentLaunch launch{table, 0, 0};
    if (!segment_grid(segment, vec, block, launch.grid, launch.shift)) {
        set_error("parameter list needs more workgroups than one launch can address");
        return -6;
    }

    // Pass 2: the table, 64 tensors per launch.
    hipStream_t st = ctx->stream;
    NoAllocBatch batch;
    int filled = 0;
    uint32_t next_chunk = 0;
    for (int i = 0; i < num_weights; i++) {
        if (keep[i]) {
            NoAllocTensor &t = batch.t[filled++];
            t.w = weight_buffers[i];
            t.g = gradient_buffers[i];
            t.m = momentum_buffers[i];
            t.v = variance_buffers[i];
            t.numel = (uint32_t)tensor_elements(req, i);
            t.first_chunk = next_chunk;
            t.flags = flags[i];
            t.index = (uint32_t)i;
            next_chunk += (uint32_t)((t.numel + (uint32_t)chunk - 1) / (uint32_t)chunk);
        }
        if (filled == kNoAllocBatch || (i == num_weights - 1 && filled > 0)) {
            noalloc_table_kernel<<<filled, 64, 0, st>>>(batch, (uint32_t)chunk, table);
            filled = 0;
        }
    }

    StepParams p = zero_params();
    p.lr = learning_rate;
    p.beta1 = beta1;
    p.beta2 = beta2;
    p.one_minus_beta1 = 1.0f - beta1;
    p.one_minus_beta2 = 1.0f - beta2;
    p.eps = epsilon;
    p.weight_decay = weight_decay;
    gm_bias_corrections(beta1, beta2, step_count, &p.bc1, &p.bc2);
    launch_update<AdamRule>(st, launch, p, vec, block, current_nontemporal(ctx));
    return hip_ok(hipGetLastError(), "allocation-free Adam launch") ? 0 : -6;
} catch (...) {
    note_exception();
    return -6;
}

}  // extern "C"
