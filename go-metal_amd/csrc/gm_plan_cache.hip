// Plan cache of the multi-tensor steps: chunk tables resident in HBM, keyed by the caller's
// handle arrays, plus the host helpers every multi-tensor entry point starts with.
//
// A plan is built when a list is first seen (or seen with other handles) and dropped when one
// of its buffers is freed or when 16 newer plans have pushed it out.  Neither event allocates,
// frees or waits once table slots exist: a dropped plan's slot (device table + pinned host twin)
// goes to the context's free list, a new plan takes one from there, fills the pinned twin and
// enqueues one asynchronous upload in front of its first launch.
#include "gm_launch.hpp"

#include "../../include/gometal_hip.h"

#include <algorithm>
#include <cstring>

namespace gm {

constexpr size_t kMaxCachedPlans = 16;
constexpr size_t kMaxFreeTables = 8;          // slots kept for reuse beyond the cached plans'
constexpr size_t kMinTableCapacity = 1024;    // descriptors (64 KiB)
constexpr int kAutoFewStreams = 5;

int auto_vec(int streams) { return streams <= kAutoFewStreams ? 2 : 1; }
int auto_block(int streams) { return streams <= kAutoFewStreams ? 128 : 256; }

int current_chunk_elements(const Context *ctx) { return ctx->chunk_elements.load(); }
bool current_nontemporal(const Context *ctx) { return ctx->nontemporal.load() != 0; }
int current_vec(const Context *ctx) { return ctx->vec.load(); }
int current_block(const Context *ctx) { return ctx->block.load(); }

StepParams zero_params()
{
    StepParams p;
    std::memset(&p, 0, sizeof p);
    return p;
}

// ----------------------------------------------------------- table slots ----
static void destroy_slot(TableSlot &s)
{
    if (s.d_chunks) (void)hipFree(s.d_chunks);
    if (s.h_chunks) (void)hipHostFree(s.h_chunks);
    if (s.uploaded) (void)hipEventDestroy(s.uploaded);
    s = TableSlot{};
}

// The smallest free slot that holds `count` descriptors, or a new one.
static bool acquire_slot(Context *ctx, size_t count, TableSlot &out)
{
    auto &pool = ctx->free_tables;
    size_t best = pool.size();
    for (size_t i = 0; i < pool.size(); i++)
        if (pool[i].capacity >= count && (best == pool.size() || pool[i].capacity < pool[best].capacity)) best = i;
    if (best != pool.size()) {
        out = pool[best];
        pool.erase(pool.begin() + best);
        return true;
    }
    size_t capacity = kMinTableCapacity;
    while (capacity < count) capacity *= 2;
    TableSlot s;
    if (!hip_ok(hipMalloc(&s.d_chunks, capacity * sizeof(Chunk)), "hipMalloc(chunk table)") ||
        !hip_ok(hipHostMalloc(&s.h_chunks, capacity * sizeof(Chunk), hipHostMallocDefault), "hipHostMalloc(chunk table)") ||
        !hip_ok(hipEventCreateWithFlags(&s.uploaded, hipEventDisableTiming), "hipEventCreate(chunk table)")) {
        destroy_slot(s);
        return false;
    }
    s.capacity = capacity;
    ctx->table_allocations.fetch_add(1);
    out = s;
    return true;
}

// A dropped plan's slot goes back to the free list.  Kernels still reading its device table are
// ahead of any later upload on the same stream; the pinned twin is guarded by its event.
static void release_slot(Context *ctx, TableSlot &s)
{
    if (!s.d_chunks) return;
    auto &pool = ctx->free_tables;
    pool.push_back(s);
    s = TableSlot{};
    if (pool.size() > kMaxFreeTables) {
        // more spare slots than a changing workload has shown to need: give the smallest back
        size_t smallest = 0;
        for (size_t i = 1; i < pool.size(); i++)
            if (pool[i].capacity < pool[smallest].capacity) smallest = i;
        (void)hipStreamSynchronize(ctx->stream);
        destroy_slot(pool[smallest]);
        pool.erase(pool.begin() + smallest);
    }
}

static void drop_plan(Context *ctx, size_t index)
{
    release_slot(ctx, ctx->plans[index]->table);
    ctx->plans.erase(ctx->plans.begin() + index);
}

// ------------------------------------------------------------------ plan ----
static bool plan_matches(const MultiTensorPlan &p, const PlanRequest &r, int chunk)
{
    if (p.kind != r.kind || p.variant != r.variant || p.num_tensors != r.num_tensors ||
        p.requested_chunk_elements != chunk)
        return false;
    const size_t n = (size_t)r.num_tensors;
    if (n == 0) return true;
    if (std::memcmp(p.sizes.data(), r.sizes, n * sizeof(int)) != 0) return false;
    for (int k = 0; k < kNumSlots; k++) {
        const uintptr_t *cached = p.handles.data() + (size_t)k * n;
        if (r.slot[k]) {
            if (std::memcmp(cached, r.slot[k], n * sizeof(uintptr_t)) != 0) return false;
        } else {
            for (size_t i = 0; i < n; i++)
                if (cached[i] != 0) return false;
        }
    }
    return true;
}

static std::unique_ptr<MultiTensorPlan> build_plan(Context *ctx, const PlanRequest &r, int requested_chunk)
{
    auto plan = std::make_unique<MultiTensorPlan>();
    const size_t n = (size_t)r.num_tensors;
    plan->requested_chunk_elements = requested_chunk;
    plan->kind = r.kind;
    plan->variant = r.variant;
    plan->num_tensors = r.num_tensors;
    plan->sizes.assign(r.sizes, r.sizes + n);
    plan->handles.assign((size_t)kNumSlots * n, 0);
    for (int k = 0; k < kNumSlots; k++)
        if (r.slot[k]) std::memcpy(plan->handles.data() + (size_t)k * n, r.slot[k], n * sizeof(uintptr_t));

    PlanLayout layout;
    layout_plan(r, requested_chunk, registry_length, layout);
    ctx->plan_builds.fetch_add(1);
    plan->status = layout.status;
    plan->chunk_elements = layout.chunk_elements;
    plan->segment[0] = layout.segment[0];
    plan->segment[1] = layout.segment[1];
    plan->num_segments = layout.num_segments;
    plan->total_elements = layout.total_elements;
    plan->kept_signature = layout.kept_signature;
    const size_t count = layout.chunks.size();
    if (plan->status != 0 || count == 0) return plan;
    if (count > 0x7FFFFFFFull) {
        set_error("parameter list needs %zu chunks, more than one launch can address", count);
        return nullptr;
    }

    TableSlot slot;
    if (!acquire_slot(ctx, count, slot)) return nullptr;
    // the last upload out of this pinned twin must have been read before it is overwritten
    if (slot.upload_pending && !hip_ok(hipEventSynchronize(slot.uploaded), "hipEventSynchronize(chunk table)")) {
        release_slot(ctx, slot);
        return nullptr;
    }
    std::memcpy(slot.h_chunks, layout.chunks.data(), count * sizeof(Chunk));
    if (!hip_ok(hipMemcpyAsync(slot.d_chunks, slot.h_chunks, count * sizeof(Chunk), hipMemcpyHostToDevice,
                               ctx->stream), "upload chunks") ||
        !hip_ok(hipEventRecord(slot.uploaded, ctx->stream), "hipEventRecord(chunk table)")) {
        (void)hipStreamSynchronize(ctx->stream);
        slot.upload_pending = false;
        release_slot(ctx, slot);
        return nullptr;
    }
    slot.upload_pending = true;
    plan->table = slot;
    plan->d_chunks = slot.d_chunks;
    plan->num_chunks = (uint32_t)count;
    return plan;
}

MultiTensorPlan *get_plan(Context *ctx, const PlanRequest &req)
{
    const int chunk = current_chunk_elements(ctx);
    auto &plans = ctx->plans;
    for (size_t i = 0; i < plans.size(); i++) {
        if (plan_matches(*plans[i], req, chunk)) {
            if (i != 0) std::rotate(plans.begin(), plans.begin() + i, plans.begin() + i + 1);
            return plans[0].get();
        }
    }
    auto plan = build_plan(ctx, req, chunk);
    if (!plan) return nullptr;
    if (plans.size() >= kMaxCachedPlans) drop_plan(ctx, plans.size() - 1);
    plans.insert(plans.begin(), std::move(plan));
    return plans[0].get();
}

void plans_forget_range(Context *ctx, uintptr_t begin, size_t bytes)
{
    auto &plans = ctx->plans;
    const uintptr_t end = begin + bytes;
    for (size_t i = plans.size(); i-- > 0;) {
        const std::vector<uintptr_t> &h = plans[i]->handles;
        // a handle is the address of its tensor's first byte: inside the freed allocation or not
        const bool touches = std::any_of(h.begin(), h.end(), [&](uintptr_t x) { return x >= begin && x < end; });
        if (touches) drop_plan(ctx, i);
    }
}

// ----------------------------------------------------------- host helpers ----
int prepare(uintptr_t device, const PlanRequest &req, int hip_error_code, Launch &out,
            std::unique_lock<std::mutex> &lock)
{
    clear_error();
    if (device == 0) {
        set_error("device handle is nil");
        return -1;
    }
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (req.num_tensors < 0 || (req.num_tensors > 0 && (!req.sizes || !req.slot[kSlotWeight] ||
                                                         !req.slot[kSlotGrad]))) {
        set_error("weight, gradient and size arrays are required");
        return hip_error_code;
    }
    if (!make_current(ctx)) return hip_error_code;
    lock = std::unique_lock<std::mutex>(ctx->mu);
    MultiTensorPlan *plan = get_plan(ctx, req);
    if (!plan) return hip_error_code;
    if (plan->status != 0) {
        set_error("a required buffer handle is nil (code %d)", plan->status);
        return plan->status;
    }
    out.ctx = ctx;
    out.plan = plan;
    return 0;
}

bool launch_geometry(const MultiTensorPlan &plan, int vec, int block, SegmentLaunch out[2], int &count)
{
    count = 0;
    for (int s = 0; s < plan.num_segments; s++) {
        const PlanSegment &seg = plan.segment[s];
        if (seg.num_chunks == 0) continue;
        uint32_t grid, shift;
        if (!segment_grid(seg, vec, block, grid, shift)) {
            set_error("parameter list needs %llu workgroups, more than one launch can address",
                      (unsigned long long)((uint64_t)seg.num_chunks << shift));
            return false;
        }
        out[count++] = SegmentLaunch{plan.d_chunks + seg.first_chunk, grid, shift};
    }
    return true;
}

}  // namespace gm

using namespace gm;

extern "C" {

int gm_set_tuning(uintptr_t device, int chunk_elements, int nontemporal, int vec)
{
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -2;
    const int v = vec == 0 ? 4 : vec;        // an automatic width may be 1 or 2: the chunk must suit both
    const int c = chunk_elements;
    if (vec != 0 && v != 1 && v != 2 && v != 4) return -1;
    if (c != 0) {
        // a chunk is a power-of-two number of 256 * vec element slices
        if (c < 256 * v || c % (256 * v) != 0) return -1;
        const int slices = c / (256 * v);
        if ((slices & (slices - 1)) != 0) return -1;
    }
    ctx->vec.store(vec);
    ctx->chunk_elements.store(c);
    ctx->nontemporal.store(nontemporal < 0 ? 1 : (nontemporal ? 1 : 0));
    return 0;
}

int gm_set_workgroup_lanes(uintptr_t device, int lanes)
{
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -2;
    if (lanes != 0 && lanes != 128 && lanes != 256) return -1;
    ctx->block.store(lanes);
    return 0;
}

int gm_plan_cache_stats(uintptr_t device, uint64_t *plan_builds, uint64_t *table_allocations, int *cached_plans)
try {
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    std::lock_guard<std::mutex> lk(ctx->mu);
    if (plan_builds) *plan_builds = ctx->plan_builds.load();
    if (table_allocations) *table_allocations = ctx->table_allocations.load();
    if (cached_plans) *cached_plans = (int)ctx->plans.size();
    return 0;
} catch (...) {
    note_exception();
    return -10;
}

}  // extern "C"
