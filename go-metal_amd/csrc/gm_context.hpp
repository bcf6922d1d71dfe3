// Process-wide state behind the C ABI: the device context (one HIP stream per
// GPU), the registry that remembers the byte length of every buffer handed out
// by allocate_metal_buffer, and the per-thread error message.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <memory>
#include <mutex>
#include <unordered_map>
#include <vector>

namespace gm {

void set_error(const char *fmt, ...) __attribute__((format(printf, 1, 2)));
void clear_error();
// For the catch (...) block of an entry point: records the exception in flight as the thread's
// last error.  No exception may cross the C boundary; the entry point then returns the code the
// reference returns from its own @catch block.
void note_exception() noexcept;

// true when the HIP call succeeded; otherwise records "what: <hip error>".
bool hip_ok(hipError_t e, const char *what);

struct MultiTensorPlan;
struct TableSlot;

// Large host <-> device copies of ordinary (pageable) host memory go through pinned staging
// slots, two lanes at a time: each lane owns a stream, two slots and their events, moves one
// half of the range and overlaps the host memcpy of one slot with the DMA of the other.
constexpr int kStageLanes = 2;
constexpr size_t kStageSlotBytes = 4u << 20;
struct StageLane {
    hipStream_t stream = nullptr;
    char *slot[2] = {nullptr, nullptr};          // pinned (hipHostMalloc), kStageSlotBytes each
    hipEvent_t ev[2] = {nullptr, nullptr};
};

struct Context {
    int device_id = 0;
    bool usable = false;
    hipStream_t stream = nullptr;
    hipEvent_t ev_start = nullptr, ev_stop = nullptr;
    std::atomic<int> refs{0};
    std::mutex mu;                                    // guards plans and launches
    std::vector<std::unique_ptr<MultiTensorPlan>> plans;  // most recently used first
    std::vector<TableSlot> free_tables;               // chunk-table slots of dropped plans, kept for reuse
    std::atomic<uint64_t> plan_builds{0};             // chunk tables laid out so far (diagnostics)
    std::atomic<uint64_t> table_allocations{0};       // table slots allocated so far (diagnostics)
    void *noalloc_scratch = nullptr;                  // this GPU's address of the allocation-free step's table
    // Launch-shape settings of this context (gm_set_tuning, gm_set_workgroup_lanes, gm_set_amp_check_order):
    // measurement switches, every combination gives bit-identical results.
    std::atomic<int> chunk_elements{0};               // elements per chunk; 0: chosen per plan
    std::atomic<int> nontemporal{1};                  // streaming accesses carry the non-temporal hint
    std::atomic<int> vec{0};                          // fp32 elements per lane; 0: chosen per launch
    std::atomic<int> block{0};                        // lanes per workgroup of the update kernels; 0: chosen per launch
    std::atomic<int> amp_check_nontemporal{1};        // cache policy of the in-place overflow check's loads
    std::atomic<int> amp_check_reverse{0};            // the in-place overflow check walks the table backwards
    std::mutex stage_mu;                              // one staged copy at a time
    bool stage_ready = false;
    StageLane stage[kStageLanes];                     // created on first use, kept until the process ends
    ~Context();
};

// The context of HIP device 0, created on first call; nullptr if no GPU works.
Context *default_context();

// Maps a device handle from the C ABI to a context.  Any non-zero handle
// resolves to the default context: as on Metal, every device handle aliases
// the one system GPU, and tests may pass placeholder handles.
Context *resolve_device(uintptr_t device);

// Makes ctx's GPU current on the calling thread (HIP's current device is
// thread-local and callers may hop threads between calls).
bool make_current(Context *ctx);

// ---- buffer registry: handle (device address) -> allocation length ----
// base: the address to hand back to hipFree when it differs from the handle (0: the handle itself)
void registry_add(uintptr_t buffer, size_t bytes, uintptr_t base = 0);
// Forgets the handle and returns the address to free (0 when the handle is unknown).
uintptr_t registry_remove(uintptr_t buffer);
// 0 when the handle is not one of ours.
size_t registry_length(uintptr_t buffer);

// A freed address may come back with a different length, so whatever was validated against the
// old allocation must be forgotten: deallocate_metal_buffer calls these (holding ctx->mu) with
// the freed range.  Only the cached plans that hold a handle inside the range are affected.
void plans_forget_range(Context *ctx, uintptr_t begin, size_t bytes);    // multi-tensor plans: dropped
void lbfgs_forget_range(uintptr_t begin, size_t bytes);                  // L-BFGS plans: handles revalidated

// Resolves this GPU's address of the allocation-free step's descriptor table (a __device__
// array) once, at context creation, with the device current.  false: error recorded.
bool noalloc_bind_scratch(Context *ctx);

}  // namespace gm
