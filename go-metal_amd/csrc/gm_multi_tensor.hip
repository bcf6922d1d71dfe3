// Multi-tensor-apply optimizer steps for gfx950: plan cache, update kernels and
// the execute_*_step entry points of the C ABI (the HIP counterpart of
// cgo_bridge/bridge_optimizer.m).
//
// One launch per step (two when the list's small tensors get a chunk size of their own).  The
// parameter list is cut into chunks of chunk_elements (256 to 65536,
// chosen per list) and each chunk into slices of BLOCK * VEC elements; workgroup b handles slice
// (b mod slices_per_chunk) of chunk (b div slices_per_chunk), one VEC-wide group per lane: load
// every stream once, apply the rule in registers, store every state once, exit.
//
// Lane width (VEC fp32 elements per lane) and workgroup size (BLOCK lanes) are chosen per launch
// by the number of streams the rule touches.  One element per lane (global_load_dword) in
// 256-lane workgroups is the choice for the seven-stream rules: measured on MI355X it sustains
// about 82 % of peak HBM bandwidth on the 4-read / 3-write Adam stream over 1B parameters,
// against about 77 % for 8-byte and 71 % for 16-byte lanes (global_load_dwordx4), whatever the
// unrolling.  The five-stream rules (SGD-momentum, AdaGrad, plain RMSProp) do best with two
// elements per lane in 128-lane workgroups (81-83 %).  Short single-pass waves keep reads and
// writes finely interleaved at the memory controllers; wide, unrolled lanes issue them in bursts.
// Every shape stays selectable (gm_set_tuning, gm_set_workgroup_lanes) so the comparison can be
// rerun.  The path is HBM-bound (about 20 flops per 28 bytes for Adam): no LDS staging, no MFMA.
#include "gm_context.hpp"
#include "gm_plan.hpp"
#include "gm_rules.hpp"

#include "../../include/gometal_hip.h"

#include <algorithm>
#include <cmath>
#include <cstring>

namespace gm {

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;
constexpr int kAutoChunkCandidates[] = {65536, 16384, 4096, 1024, 256};   // largest first
constexpr double kAutoChunkMaxIdleFraction = 0.05;
// Tensors shorter than a quarter of the list's chunk leave three quarters and more of their chunk's
// workgroups idle.  An idle workgroup costs about 0.6 ns and a second launch about 5 us (measured on
// MI355X), so those tensors move to a segment of their own, with a smaller chunk, once they would
// idle this many workgroups.  The 1B-parameter transformer list qualifies (360 vectors of 4096
// elements in 65536-element chunks: 86k idle workgroups; the step is 4 to 11 us of 4.32 ms faster
// with the second segment, alternated with the single-launch plan in one process).
constexpr uint64_t kSplitMinIdleWorkgroups = 16384;
// Launch shape when the caller has not fixed it (gm_set_tuning, gm_set_workgroup_lanes), measured on
// MI355X over lists of 25M, 125M and 1B parameters.  Rules with five streams (SGD-momentum, AdaGrad,
// plain RMSProp: 3 reads + 2 writes): 8-byte lanes in 128-lane workgroups, 81-83 % of peak, against
// 76-82 % in 256-lane workgroups and 71-77 % with 4-byte lanes.  Seven streams and more (Adam, NAdam,
// AdaDelta, the mixed-precision step): 4-byte lanes in 256-lane workgroups, 81-82 %, against 79-80 %
// in 128-lane workgroups and 76-79 % with 8-byte lanes.
constexpr int kAutoFewStreams = 5;

static int auto_vec(int streams) { return streams <= kAutoFewStreams ? 2 : 1; }
static int auto_block(int streams) { return streams <= kAutoFewStreams ? 128 : kBlock; }
constexpr int kCheckUnroll = 4;           // 16-byte loads in flight per lane in the overflow check
constexpr size_t kMaxCachedPlans = 16;

static std::atomic<int> g_chunk_elements{0};   // 0: chosen per plan
static std::atomic<int> g_nontemporal{1};
static std::atomic<int> g_vec{0};               // 0: chosen per launch by auto_vec
static std::atomic<int> g_block{0};             // lanes per workgroup of the update kernels; 0: auto_block

int current_chunk_elements() { return g_chunk_elements.load(); }
bool current_nontemporal() { return g_nontemporal.load() != 0; }
int current_vec() { return g_vec.load(); }
int current_block() { return g_block.load(); }

// log2(slices per chunk) for a chunk size and lane width; chunk_elements is a
// power-of-two multiple of 256 * vec (gm_set_tuning enforces it).
static uint32_t slice_shift_for(int chunk_elements, int vec, int block)
{
    uint32_t slices = (uint32_t)(chunk_elements / (block * vec));
    uint32_t shift = 0;
    while ((1u << shift) < slices) shift++;
    return shift;
}

// ------------------------------------------------------------------ plan ----
MultiTensorPlan::~MultiTensorPlan()
{
    if (d_chunks) (void)hipFree(d_chunks);
}

static bool plan_matches(const MultiTensorPlan &p, const PlanRequest &r, int chunk, uint64_t gen)
{
    if (p.kind != r.kind || p.variant != r.variant || p.num_tensors != r.num_tensors ||
        p.requested_chunk_elements != chunk || p.generation != gen)
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

// Chunk size for a tensor list when the caller has not fixed one.  A chunk's
// descriptor is fetched once per workgroup, and that fetch is the only
// latency a workgroup cannot overlap, so large chunks (many workgroups
// sharing one cached descriptor) are faster; but every chunk launches a full
// set of slices, and the slices past a tensor's end are idle workgroups.
// Take the largest candidate whose idle workgroups stay below 5 % of the
// working ones.  Lists of small tensors end up with small chunks, down to one
// descriptor per workgroup: measured on MI355X, Adam over 5000 tensors of 64 to
// 2048 elements takes 64 us per step with 4096-element chunks (15 of 16
// workgroups idle for most tensors) and 26 us with 256-element chunks, while
// lists of large tensors lose 3 to 4 points of bandwidth below 4096.
static int choose_chunk_elements(const PlanRequest &r)
{
    for (int candidate : kAutoChunkCandidates) {
        const uint64_t per_chunk = (uint64_t)candidate / kBlock;
        uint64_t working = 0, launched = 0;
        for (int i = 0; i < r.num_tensors; i++) {
            const uint64_t numel = r.sizes[i] > 0 ? (uint64_t)r.sizes[i] / sizeof(float) : 0;
            working += (numel + kBlock - 1) / kBlock;
            launched += (numel + candidate - 1) / candidate * per_chunk;
        }
        if (launched - working <= (uint64_t)(kAutoChunkMaxIdleFraction * (double)working)) return candidate;
    }
    return kAutoChunkCandidates[sizeof(kAutoChunkCandidates) / sizeof(int) - 1];
}

// The chunk size for the tensors below `limit` elements when they are worth a segment of their own
// (0 otherwise): the largest candidate under the list's chunk size that keeps their idle workgroups
// below 5 % of their working ones.
static int choose_small_segment(const PlanRequest &r, int chunk, size_t &limit)
{
    limit = (size_t)chunk / 4;
    const uint64_t per_chunk = (uint64_t)chunk / kBlock;
    uint64_t idle = 0;
    for (int i = 0; i < r.num_tensors; i++) {
        const uint64_t numel = r.sizes[i] > 0 ? (uint64_t)r.sizes[i] / sizeof(float) : 0;
        if (numel == 0 || numel >= limit) continue;
        idle += per_chunk - (numel + kBlock - 1) / kBlock;
    }
    if (idle < kSplitMinIdleWorkgroups) return 0;
    int last = 0;
    for (int candidate : kAutoChunkCandidates) {
        if (candidate >= chunk) continue;
        last = candidate;
        const uint64_t per = (uint64_t)candidate / kBlock;
        uint64_t working = 0, launched = 0;
        for (int i = 0; i < r.num_tensors; i++) {
            const uint64_t numel = r.sizes[i] > 0 ? (uint64_t)r.sizes[i] / sizeof(float) : 0;
            if (numel == 0 || numel >= limit) continue;
            working += (numel + kBlock - 1) / kBlock;
            launched += (numel + candidate - 1) / candidate * per;
        }
        if (launched - working <= (uint64_t)(kAutoChunkMaxIdleFraction * (double)working)) return candidate;
    }
    return last;
}

static std::unique_ptr<MultiTensorPlan> build_plan(Context *ctx, const PlanRequest &r, int requested_chunk,
                                                   uint64_t gen)
{
    auto plan = std::make_unique<MultiTensorPlan>();
    const size_t n = (size_t)r.num_tensors;
    const int chunk = requested_chunk > 0 ? requested_chunk : choose_chunk_elements(r);
    size_t small_limit = 0;
    const int small_chunk = requested_chunk > 0 ? 0 : choose_small_segment(r, chunk, small_limit);
    plan->requested_chunk_elements = requested_chunk;
    plan->kind = r.kind;
    plan->variant = r.variant;
    plan->num_tensors = r.num_tensors;
    plan->chunk_elements = chunk;
    plan->generation = gen;
    plan->sizes.assign(r.sizes, r.sizes + n);
    plan->handles.assign((size_t)kNumSlots * n, 0);
    for (int k = 0; k < kNumSlots; k++)
        if (r.slot[k]) std::memcpy(plan->handles.data() + (size_t)k * n, r.slot[k], n * sizeof(uintptr_t));

    std::vector<Chunk> chunks, small_chunks;
    for (size_t i = 0; i < n; i++) {
        uintptr_t h[kNumSlots];
        for (int k = 0; k < kNumSlots; k++) h[k] = plan->handles[(size_t)k * n + i];

        // 1. handles that must be present
        bool skip = false;
        for (int k = 0; k < kNumSlots && plan->status == 0; k++) {
            if (h[k] != 0) continue;
            if (r.required_mask & (1u << k)) {
                if (r.missing_code != 0) plan->status = r.missing_code;
                else skip = true;
            } else if (r.skip_if_zero_mask & (1u << k)) {
                skip = true;
            }
        }
        if (plan->status == 0 && r.extra_check) plan->status = r.extra_check(r, (int)i);
        if (plan->status != 0) break;

        const int size_bytes = r.sizes[i] > 0 ? r.sizes[i] : 0;
        const size_t numel = (size_t)size_bytes / sizeof(float);
        if (skip || numel == 0) continue;

        // 2. an allocation of ours that is shorter than the tensor: skip it
        //    (bridge_optimizer.m:427-436)
        uint32_t flags = kRecVec2Ok | kRecVec4Ok | kRecGrad16VectorOk;
        for (int k = 0; k < kNumSlots; k++) {
            if (h[k] == 0) continue;
            const bool half = (r.half_mask & (1u << k)) != 0;
            const size_t need = numel * (half ? 2 : 4);
            const size_t have = registry_length(h[k]);
            if (have != 0 && have < need) skip = true;
            if (h[k] % (half ? 4 : 8) != 0) flags &= ~kRecVec2Ok;
            if (h[k] % (half ? 8 : 16) != 0) flags &= ~kRecVec4Ok;
            if (half && k == kSlotGrad && h[k] % 16 != 0) flags &= ~kRecGrad16VectorOk;
        }
        if (skip) continue;

        const bool in_small_segment = small_chunk != 0 && numel < small_limit;
        const size_t step = (size_t)(in_small_segment ? small_chunk : chunk);
        std::vector<Chunk> &table = in_small_segment ? small_chunks : chunks;
        for (size_t off = 0; off < numel; off += step) {
            const size_t left = numel - off;
            Chunk c{};
            for (int k = 0; k < kNumSlots; k++) {
                if (h[k] == 0) continue;
                const size_t elem = (r.half_mask & (1u << k)) ? 2 : 4;
                c.p[k] = reinterpret_cast<void *>(h[k] + off * elem);
            }
            c.count = (uint32_t)(left < step ? left : step);
            c.flags = flags;
            c.tensor = (uint32_t)i;
            table.push_back(c);
        }
        plan->total_elements += numel;
    }
    plan->segment[0] = PlanSegment{0, (uint32_t)chunks.size(), chunk};
    plan->segment[1] = PlanSegment{(uint32_t)chunks.size(), (uint32_t)small_chunks.size(), small_chunk};
    plan->num_segments = small_chunks.empty() ? 1 : 2;
    chunks.insert(chunks.end(), small_chunks.begin(), small_chunks.end());
    if (plan->status != 0 || chunks.empty()) return plan;
    if (chunks.size() > 0x7FFFFFFFull) {
        set_error("parameter list needs %zu chunks, more than one launch can address", chunks.size());
        return nullptr;
    }

    if (!hip_ok(hipMalloc(&plan->d_chunks, chunks.size() * sizeof(Chunk)), "hipMalloc(chunks)") ||
        !hip_ok(hipMemcpyAsync(plan->d_chunks, chunks.data(), chunks.size() * sizeof(Chunk),
                               hipMemcpyHostToDevice, ctx->stream), "upload chunks") ||
        !hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))
        return nullptr;
    plan->num_chunks = (uint32_t)chunks.size();
    return plan;
}

MultiTensorPlan *get_plan(Context *ctx, const PlanRequest &req)
{
    const int chunk = current_chunk_elements();
    const uint64_t gen = registry_generation();
    auto &plans = ctx->plans;
    for (size_t i = 0; i < plans.size(); i++) {
        if (plan_matches(*plans[i], req, chunk, gen)) {
            if (i != 0) std::rotate(plans.begin(), plans.begin() + i, plans.begin() + i + 1);
            return plans[0].get();
        }
    }
    // Plans of an older registry generation can never match again.
    for (size_t i = plans.size(); i-- > 0;)
        if (plans[i]->generation != gen) plans.erase(plans.begin() + i);
    auto plan = build_plan(ctx, req, chunk, gen);
    if (!plan) return nullptr;
    if (plans.size() >= kMaxCachedPlans) plans.pop_back();
    plans.insert(plans.begin(), std::move(plan));
    return plans[0].get();
}

// --------------------------------------------------------------- kernels ----
// Tensor addresses reach the kernels through tables in memory, so the compiler
// only knows them as generic pointers and would emit flat_* instructions.  They
// are always HBM addresses: casting to the global address space yields
// global_load / global_store (one wait counter, no aperture check).
#define GM_GLOBAL __attribute__((address_space(1)))

template <bool NT, class T>
__device__ inline T stream_load(const T *p)
{
    const GM_GLOBAL T *gp = (const GM_GLOBAL T *)p;
    if (NT) return __builtin_nontemporal_load(gp);
    return *gp;
}

template <bool NT, class T>
__device__ inline void stream_store(T v, T *p)
{
    GM_GLOBAL T *gp = (GM_GLOBAL T *)p;
    if (NT) __builtin_nontemporal_store(v, gp);
    else *gp = v;
}

template <class T, int N>
struct VecOf {
    typedef T type __attribute__((ext_vector_type(N)));
};
template <class T>
struct VecOf<T, 1> {
    typedef T type;
};

template <int N, class V>
__device__ inline auto lane_of(const V &v, int c)
{
    if constexpr (N == 1) return v;
    else return v[c];
}

template <int N, class V, class T>
__device__ inline void set_lane(V &v, int c, T x)
{
    if constexpr (N == 1) v = x;
    else v[c] = x;
}

// One lane's share of a slice: elements [first, first + N) of the chunk's
// streams, N = VEC when the whole group is inside the chunk and the streams
// are aligned for it, else 1.
template <class Rule, int N, bool NT, bool AMP>
__device__ inline void update_group(const Chunk &ch, uint32_t first, const StepParams &prm,
                                    float inv_scale)
{
    constexpr int NS = Rule::NSTATE;
    constexpr int NSA = NS > 0 ? NS : 1;
    typedef typename VecOf<float, N>::type FV;
    typedef typename VecOf<_Float16, N>::type HV;

    FV *wp = reinterpret_cast<FV *>(reinterpret_cast<float *>(ch.p[kSlotWeight]) + first);
    FV W = stream_load<NT>(wp);
    FV G;
    if (AMP) {
        HV h = stream_load<NT>(reinterpret_cast<const HV *>(
            reinterpret_cast<const _Float16 *>(ch.p[kSlotGrad]) + first));
#pragma unroll
        for (int c = 0; c < N; c++) set_lane<N>(G, c, (float)lane_of<N>(h, c));
    } else {
        G = stream_load<NT>(reinterpret_cast<const FV *>(
            reinterpret_cast<const float *>(ch.p[kSlotGrad]) + first));
    }
    FV S[NSA];
    FV *sp[NSA];
#pragma unroll
    for (int k = 0; k < NS; k++) {
        sp[k] = reinterpret_cast<FV *>(reinterpret_cast<float *>(ch.p[kSlotState0 + k]) + first);
        S[k] = stream_load<NT>(sp[k]);
    }
#pragma unroll
    for (int c = 0; c < N; c++) {
        float wv = lane_of<N>(W, c);
        float gv = lane_of<N>(G, c);
        if (AMP) gv = gv * inv_scale;
        float sv[NSA];
#pragma unroll
        for (int k = 0; k < NS; k++) sv[k] = lane_of<N>(S[k], c);
        Rule::apply(wv, gv, sv, prm);
        set_lane<N>(W, c, wv);
#pragma unroll
        for (int k = 0; k < NS; k++) set_lane<N>(S[k], c, sv[k]);
    }
    stream_store<NT>(W, wp);
#pragma unroll
    for (int k = 0; k < NS; k++) stream_store<NT>(S[k], sp[k]);
    if (AMP && ch.p[kSlotWeight16]) {
        HV h;
#pragma unroll
        for (int c = 0; c < N; c++) set_lane<N>(h, c, (_Float16)lane_of<N>(W, c));
        stream_store<NT>(h, reinterpret_cast<HV *>(reinterpret_cast<_Float16 *>(ch.p[kSlotWeight16]) + first));
    }
}

// Workgroup b -> (chunk, slice).  slice_shift = log2(slices per chunk).
template <class Rule, int VEC, bool NT, bool AMP, int BLOCK>
__device__ inline void update_slice(const Chunk &ch, uint32_t slice_shift, const StepParams &prm,
                                    float inv_scale)
{
    const uint32_t slice = blockIdx.x & ((1u << slice_shift) - 1u);
    const uint32_t local = (slice * BLOCK + threadIdx.x) * VEC;   // first element of this lane within the chunk
    if (local >= ch.count) return;
    constexpr uint32_t vec_flag = VEC == 4 ? kRecVec4Ok : kRecVec2Ok;
    if (VEC > 1 && (ch.flags & vec_flag) && local + VEC <= ch.count) {
        update_group<Rule, VEC, NT, AMP>(ch, local, prm, inv_scale);
    } else {
        const uint32_t n = ch.count - local < (uint32_t)VEC ? ch.count - local : (uint32_t)VEC;
        for (uint32_t e = 0; e < n; e++) update_group<Rule, 1, NT, AMP>(ch, local + e, prm, inv_scale);
    }
}

template <class Rule, int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
multi_tensor_update_kernel(const Chunk *__restrict__ chunks, uint32_t slice_shift, StepParams prm)
{
    const Chunk ch = chunks[blockIdx.x >> slice_shift];
    update_slice<Rule, VEC, NT, false, BLOCK>(ch, slice_shift, prm, 1.0f);
}

// SGD: a tensor without a momentum buffer takes the vanilla rule.
template <int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
multi_tensor_sgd_kernel(const Chunk *__restrict__ chunks, uint32_t slice_shift, StepParams prm)
{
    const Chunk ch = chunks[blockIdx.x >> slice_shift];
    if (prm.momentum > 0.0f && ch.p[kSlotState0] != nullptr)
        update_slice<SgdMomentumRule, VEC, NT, false, BLOCK>(ch, slice_shift, prm, 1.0f);
    else
        update_slice<SgdVanillaRule, VEC, NT, false, BLOCK>(ch, slice_shift, prm, 1.0f);
}

// ---- mixed precision ----

// Loss-scale state machine, resident in HBM next to the tensors.
struct alignas(16) AmpDeviceState {
    // head: the 16 bytes every workgroup of the update kernel reads with one scalar load
    float scale;
    float inv_scale;        // 1.0f / scale, kept by whoever changes scale (IEEE division on host and device alike)
    int found_inf;          // set by the check kernel, consumed and cleared by the epilogue
    int applied_steps;      // steps applied so far (the optimizer's StepCount): +1 per clean step
    // tail
    int growth_tracker;
    int last_skipped;
    float growth_factor;
    float backoff_factor;
    int growth_interval;
    int skipped_steps;      // steps dropped so far
    int pad[2];
};

// Bias corrections for the asynchronous step.  The host does not know how many of the steps
// still in flight were applied, so it sends the corrections (glibc powf, like every other
// step) for each step count that is possible and the kernel picks by the device's count.
constexpr int kAmpMaxInFlight = 8;
struct AmpBiasTable {
    int base;               // step count of entry 0 minus one: entry j is for t = base + 1 + j
    int count;              // 1: use entry 0 whatever the device's count (synchronous step)
    float bc1[kAmpMaxInFlight];
    float bc2[kAmpMaxInFlight];
};

// Phase A: OR over every fp16 gradient element of "exponent field all ones"
// (+-inf or NaN).  Per lane OR -> wavefront ballot -> one LDS word per wave ->
// one atomic per workgroup that saw a hit.
template <bool NT>
__global__ void __launch_bounds__(kBlock)
amp_overflow_check_kernel(const Chunk *__restrict__ chunks, AmpDeviceState *__restrict__ state)
{
    __shared__ unsigned int wave_hit[kBlock / 64];
    const Chunk ch = chunks[blockIdx.x];
    const unsigned short *g = reinterpret_cast<const unsigned short *>(ch.p[kSlotGrad]);
    unsigned int bad = 0;
    uint32_t done = 0;
    if (ch.flags & kRecGrad16VectorOk) {
        const uint32_t n8 = ch.count >> 3;
        const uintx4 *g8 = reinterpret_cast<const uintx4 *>(g);
        for (uint32_t base = threadIdx.x; base < n8; base += kBlock * kCheckUnroll) {
            uintx4 v[kCheckUnroll];
#pragma unroll
            for (int u = 0; u < kCheckUnroll; u++) {
                const uint32_t i = base + u * kBlock;
                v[u] = (i < n8) ? stream_load<NT>(g8 + i) : uintx4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int u = 0; u < kCheckUnroll; u++) {
#pragma unroll
                for (int c = 0; c < 4; c++) {
                    const unsigned int e = v[u][c] & 0x7C007C00u;
                    bad |= ((e & 0xFFFFu) == 0x7C00u) | ((e >> 16) == 0x7C00u);
                }
            }
        }
        done = n8 << 3;
    }
    for (uint32_t i = done + threadIdx.x; i < ch.count; i += kBlock)
        bad |= ((stream_load<false>(g + i) & 0x7C00u) == 0x7C00u);

    const unsigned long long ballot = __ballot(bad != 0);
    if ((threadIdx.x & 63) == 0) wave_hit[threadIdx.x >> 6] = (ballot != 0ull);
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned int any = 0;
#pragma unroll
        for (int k = 0; k < kBlock / 64; k++) any |= wave_hit[k];
        if (any) atomicOr(&state->found_inf, 1);
    }
}

// Phase B: the Adam update on unscaled gradients, skipped as a whole when the
// flag is set.
template <int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
amp_adam_update_kernel(const Chunk *__restrict__ chunks, uint32_t slice_shift, StepParams prm,
                       const AmpDeviceState *__restrict__ state, AmpBiasTable bias)
{
    // The state's head (scale, its reciprocal, flag, applied steps) comes with one 16-byte scalar load
    // and the chunk descriptor with another, both issued before anything is decided; the bias
    // table sits in the kernel arguments and its entry is picked by scalar selects.  No load
    // waits for another except on the kernel-argument pointers themselves.
    const uintx4 head = *reinterpret_cast<const uintx4 *>(state);
    const Chunk ch = chunks[blockIdx.x >> slice_shift];
    const uint32_t first_lane_element = (blockIdx.x & ((1u << slice_shift) - 1u)) * BLOCK * VEC;
    // (the weight pointer is never null; testing it here makes the compiler fetch the whole
    // descriptor before the branch instead of the count first and the addresses after it)
    if ((head.z != 0u) | (first_lane_element >= ch.count) | (ch.p[kSlotWeight] == nullptr))
        return;                                                        // step dropped, or an idle slice
    const float inv_scale = __uint_as_float(head.y);
    const int applied = (int)head.w;
    int pick = bias.count > 1 ? applied - bias.base : 0;
    pick = pick < 0 ? 0 : (pick >= bias.count ? bias.count - 1 : pick);
    float bc1 = bias.bc1[0], bc2 = bias.bc2[0];
#pragma unroll
    for (int j = 1; j < kAmpMaxInFlight; j++) {
        if (pick == j) {
            bc1 = bias.bc1[j];
            bc2 = bias.bc2[j];
        }
    }
    prm.bc1 = bc1;
    prm.bc2 = bc2;
    update_slice<AdamRule, VEC, NT, true, BLOCK>(ch, slice_shift, prm, inv_scale);
}

// Epilogue (one lane, same stream, after phase B has drained): advances the
// loss-scale state machine and re-arms the flag.  A separate launch rather
// than a last-workgroup ticket: a single counter bumped by every workgroup of
// a 250k-workgroup grid serialises in the memory-side atomic unit.
__global__ void amp_finalize_kernel(AmpDeviceState *state, AmpDeviceState *host_mirror)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    AmpDeviceState st = *state;
    const int found = st.found_inf;
    if (found) {
        st.scale = st.scale * st.backoff_factor;
        st.growth_tracker = 0;
        st.skipped_steps += 1;
    } else {
        st.applied_steps += 1;
        st.growth_tracker += 1;
        if (st.growth_tracker == st.growth_interval) {
            st.scale = st.scale * st.growth_factor;
            st.growth_tracker = 0;
        }
    }
    st.inv_scale = 1.0f / st.scale;
    st.last_skipped = found ? 1 : 0;
    st.found_inf = 0;
    *state = st;
    // The post-state also goes straight into pinned host memory: the host reads it once the
    // stream (or the event recorded after this launch) has completed, without a copy launch.
    if (host_mirror) *host_mirror = st;
}

// ----------------------------------------------------------- host helpers ----
static StepParams zero_params()
{
    StepParams p;
    std::memset(&p, 0, sizeof p);
    return p;
}

struct Launch {
    Context *ctx;
    MultiTensorPlan *plan;
};

// Resolves the device, takes the context lock, finds the plan.  Returns the
// entry point's code on failure (hip_error_code for HIP trouble) or 0; when 0
// and out.plan->num_chunks == 0 there is nothing to launch.
static int prepare(uintptr_t device, const PlanRequest &req, int hip_error_code, Launch &out,
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

// One launch per segment.  Grid size: every chunk of a segment gets the same number of slices; the
// slices past the end of a short chunk exit at once.
struct SegmentLaunch {
    const Chunk *chunks;
    uint32_t grid, shift;
};

// Fills out[0 .. count) for the plan's non-empty segments; false (nothing may be launched) when a
// segment needs more workgroups than a launch can address.
static bool launch_geometry(const MultiTensorPlan &plan, int vec, int block, SegmentLaunch out[2], int &count)
{
    count = 0;
    for (int s = 0; s < plan.num_segments; s++) {
        const PlanSegment &seg = plan.segment[s];
        if (seg.num_chunks == 0) continue;
        const uint32_t shift = slice_shift_for(seg.chunk_elements, vec, block);
        const uint64_t blocks = (uint64_t)seg.num_chunks << shift;
        if (blocks > 0x7FFFFFFFull) {
            set_error("parameter list needs %llu workgroups, more than one launch can address",
                      (unsigned long long)blocks);
            return false;
        }
        out[count++] = SegmentLaunch{plan.d_chunks + seg.first_chunk, (uint32_t)blocks, shift};
    }
    return true;
}

template <class Rule, int VEC, int BLOCK>
static void launch_rule_vec(const Launch &l, const StepParams &prm, const SegmentLaunch &g)
{
    if (current_nontemporal())
        multi_tensor_update_kernel<Rule, VEC, true, BLOCK><<<g.grid, BLOCK, 0, l.ctx->stream>>>(g.chunks, g.shift, prm);
    else
        multi_tensor_update_kernel<Rule, VEC, false, BLOCK><<<g.grid, BLOCK, 0, l.ctx->stream>>>(g.chunks, g.shift, prm);
}

template <class Rule>
static int launch_rule(const Launch &l, const StepParams &prm, int hip_error_code)
{
    if (l.plan->num_chunks == 0) return 0;
    constexpr int streams = 3 + 2 * Rule::NSTATE;          // w, g, states read; w, states written
    int vec = current_vec(), block = current_block();
    if (vec == 0) vec = auto_vec(streams);
    if (block == 0) block = auto_block(streams);
    SegmentLaunch seg[2];
    int count;
    if (!launch_geometry(*l.plan, vec, block, seg, count)) return hip_error_code;
    for (int s = 0; s < count; s++) {
        if (block == 128) {
            if (vec == 4) launch_rule_vec<Rule, 4, 128>(l, prm, seg[s]);
            else if (vec == 2) launch_rule_vec<Rule, 2, 128>(l, prm, seg[s]);
            else launch_rule_vec<Rule, 1, 128>(l, prm, seg[s]);
        } else {
            if (vec == 4) launch_rule_vec<Rule, 4, kBlock>(l, prm, seg[s]);
            else if (vec == 2) launch_rule_vec<Rule, 2, kBlock>(l, prm, seg[s]);
            else launch_rule_vec<Rule, 1, kBlock>(l, prm, seg[s]);
        }
    }
    return hip_ok(hipGetLastError(), "update kernel launch") ? 0 : hip_error_code;
}

static int rmsprop_extra_check(const PlanRequest &req, int i)
{
    const bool momentum = (req.variant & 1) != 0, centered = (req.variant & 2) != 0;
    if (momentum && (!req.slot[kSlotState1] || req.slot[kSlotState1][i] == 0)) return -5;
    const int ga = momentum ? kSlotState2 : kSlotState1;
    if (centered && (!req.slot[ga] || req.slot[ga][i] == 0)) return -6;
    return 0;
}

static int adam_like_step(int kind, uintptr_t device, uintptr_t *w, uintptr_t *g, uintptr_t *m,
                          uintptr_t *v, int n, int *sizes, float lr, float beta1, float beta2,
                          float eps, float wd, int step_count)
{
    PlanRequest req{};
    req.kind = kind;
    req.num_tensors = n;
    req.slot[kSlotWeight] = w;
    req.slot[kSlotGrad] = g;
    req.slot[kSlotState0] = m;
    req.slot[kSlotState1] = v;
    req.sizes = sizes;
    req.required_mask = (1u << kSlotWeight) | (1u << kSlotGrad) | (1u << kSlotState0) | (1u << kSlotState1);
    req.missing_code = -4;
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = prepare(device, req, -6, l, lock)) return rc;

    StepParams p = zero_params();
    p.lr = lr;
    p.beta1 = beta1;
    p.beta2 = beta2;
    p.one_minus_beta1 = 1.0f - beta1;
    p.one_minus_beta2 = 1.0f - beta2;
    p.eps = eps;
    p.weight_decay = wd;
    gm_bias_corrections(beta1, beta2, step_count, &p.bc1, &p.bc2);
    if (kind == kRuleNAdam) {
        p.mu = gm_nadam_mu_next(beta1, step_count);
        p.one_minus_mu = 1.0f - p.mu;
        return launch_rule<NAdamRule>(l, p, -6);
    }
    return launch_rule<AdamRule>(l, p, -6);
}

}  // namespace gm

using namespace gm;

// ================================================================= C ABI ====
extern "C" {

void gm_bias_corrections(float beta1, float beta2, int step_count, float *bc1, float *bc2)
{
    // bridge_optimizer.m:398-399
    *bc1 = 1.0f - powf(beta1, (float)step_count);
    *bc2 = 1.0f - powf(beta2, (float)step_count);
}

float gm_nadam_mu_next(float beta1, int step_count)
{
    // bridge_optimizer.m:2066
    const float exponent = (float)(step_count + 1) * 0.004f;
    const float decay = powf(0.96f, exponent);
    const float half_decay = 0.5f * decay;
    const float one_minus = 1.0f - half_decay;
    return beta1 * one_minus;
}

int gm_set_tuning(int chunk_elements, int nontemporal, int vec)
{
    const int v = vec == 0 ? 4 : vec;        // an automatic width may be 1 or 2: the chunk must suit both
    const int c = chunk_elements;
    if (vec != 0 && v != 1 && v != 2 && v != 4) return -1;
    if (c != 0) {
        // a chunk is a power-of-two number of 256 * vec element slices
        if (c < kBlock * v || c % (kBlock * v) != 0) return -1;
        const int slices = c / (kBlock * v);
        if ((slices & (slices - 1)) != 0) return -1;
    }
    g_vec.store(vec);
    g_chunk_elements.store(c);
    g_nontemporal.store(nontemporal < 0 ? 1 : (nontemporal ? 1 : 0));
    return 0;
}

int gm_set_workgroup_lanes(int lanes)
{
    if (lanes != 0 && lanes != 128 && lanes != kBlock) return -1;
    g_block.store(lanes);
    return 0;
}

int execute_sgd_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                              uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                              int num_weights, int *buffer_sizes, float learning_rate,
                              float momentum, float weight_decay, int nesterov, int step_count)
try {
    (void)step_count;   // unused by the reference as well
    PlanRequest req{};
    req.kind = kRuleSGD;
    req.num_tensors = num_weights;
    req.slot[kSlotWeight] = weight_buffers;
    req.slot[kSlotGrad] = gradient_buffers;
    req.slot[kSlotState0] = momentum > 0.0f ? momentum_buffers : nullptr;
    req.sizes = buffer_sizes;
    req.skip_if_zero_mask = (1u << kSlotWeight) | (1u << kSlotGrad);
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = prepare(device, req, -10, l, lock)) return rc;
    if (l.plan->num_chunks == 0) return 0;

    StepParams p = zero_params();
    p.lr = learning_rate;
    p.momentum = momentum;
    p.weight_decay = weight_decay;
    p.nesterov = nesterov;
    int vec = current_vec();
    if (vec == 0) vec = auto_vec(5);
    const bool nt = current_nontemporal();
    int block = current_block();
    // Without momentum every tensor takes the vanilla rule: two streams read, one written.  That mix
    // does best in single-wavefront workgroups (measured on MI355X: 8-byte lanes, 64 lanes per
    // workgroup 85-87 % of peak against 76-77 % in 128-lane workgroups).
    if (block == 0) block = momentum > 0.0f ? auto_block(5) : 64;
    SegmentLaunch seg[2];
    int count;
    if (!launch_geometry(*l.plan, vec, block, seg, count)) return -10;
    hipStream_t st = l.ctx->stream;
#define GM_LAUNCH_SGD(V, N, B) multi_tensor_sgd_kernel<V, N, B><<<g.grid, B, 0, st>>>(g.chunks, g.shift, p)
#define GM_LAUNCH_SGD_B(B)                                                              \
    if (vec == 4) { if (nt) GM_LAUNCH_SGD(4, true, B); else GM_LAUNCH_SGD(4, false, B); }        \
    else if (vec == 2) { if (nt) GM_LAUNCH_SGD(2, true, B); else GM_LAUNCH_SGD(2, false, B); }   \
    else { if (nt) GM_LAUNCH_SGD(1, true, B); else GM_LAUNCH_SGD(1, false, B); }
    for (int s = 0; s < count; s++) {
        const SegmentLaunch &g = seg[s];
        if (block == 64) { GM_LAUNCH_SGD_B(64) } else if (block == 128) { GM_LAUNCH_SGD_B(128) } else { GM_LAUNCH_SGD_B(kBlock) }
    }
#undef GM_LAUNCH_SGD_B
#undef GM_LAUNCH_SGD
    return hip_ok(hipGetLastError(), "sgd kernel launch") ? 0 : -10;
} catch (...) {
    note_exception();
    return -10;
}

int execute_adam_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                               uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                               uintptr_t *variance_buffers, int num_weights, int *buffer_sizes,
                               float learning_rate, float beta1, float beta2, float epsilon,
                               float weight_decay, int step_count)
try {
    return adam_like_step(kRuleAdam, device, weight_buffers, gradient_buffers, momentum_buffers,
                          variance_buffers, num_weights, buffer_sizes, learning_rate, beta1, beta2,
                          epsilon, weight_decay, step_count);
} catch (...) {
    note_exception();
    return -6;
}

int execute_adam_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                      uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                                      uintptr_t *variance_buffers, int num_weights,
                                      int *buffer_sizes, float learning_rate, float beta1,
                                      float beta2, float epsilon, float weight_decay,
                                      int step_count, uintptr_t command_pool)
try {
    if (device == 0) return -1;
    if (command_pool == 0) return -15;
    return adam_like_step(kRuleAdam, device, weight_buffers, gradient_buffers, momentum_buffers,
                          variance_buffers, num_weights, buffer_sizes, learning_rate, beta1, beta2,
                          epsilon, weight_decay, step_count);
} catch (...) {
    note_exception();
    return -13;
}

int execute_nadam_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                                uintptr_t *variance_buffers, int num_weights, int *buffer_sizes,
                                float learning_rate, float beta1, float beta2, float epsilon,
                                float weight_decay, int step_count)
try {
    return adam_like_step(kRuleNAdam, device, weight_buffers, gradient_buffers, momentum_buffers,
                          variance_buffers, num_weights, buffer_sizes, learning_rate, beta1, beta2,
                          epsilon, weight_decay, step_count);
} catch (...) {
    note_exception();
    return -6;
}

int execute_rmsprop_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                  uintptr_t *gradient_buffers,
                                  uintptr_t *squared_grad_avg_buffers,
                                  uintptr_t *momentum_buffers, uintptr_t *gradient_avg_buffers,
                                  int num_weights, int *buffer_sizes, float learning_rate,
                                  float alpha, float epsilon, float weight_decay, float momentum,
                                  bool centered, int step_count)
try {
    (void)step_count;
    const bool use_momentum = momentum > 0.0f;
    PlanRequest req{};
    req.kind = kRuleRMSProp;
    req.variant = (use_momentum ? 1 : 0) | (centered ? 2 : 0);
    req.num_tensors = num_weights;
    req.slot[kSlotWeight] = weight_buffers;
    req.slot[kSlotGrad] = gradient_buffers;
    req.slot[kSlotState0] = squared_grad_avg_buffers;
    // state order inside the kernel: squared average, [momentum], [gradient average]
    int next = kSlotState1;
    if (use_momentum) req.slot[next++] = momentum_buffers;
    if (centered) req.slot[next++] = gradient_avg_buffers;
    req.sizes = buffer_sizes;
    req.required_mask = (1u << kSlotWeight) | (1u << kSlotGrad) | (1u << kSlotState0);
    req.missing_code = -4;
    req.extra_check = rmsprop_extra_check;
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = prepare(device, req, -8, l, lock)) return rc;

    StepParams p = zero_params();
    p.lr = learning_rate;
    p.alpha = alpha;
    p.one_minus_alpha = 1.0f - alpha;
    p.eps = epsilon;
    p.weight_decay = weight_decay;
    p.momentum = momentum;
    if (use_momentum && centered) return launch_rule<RmsPropRule<true, true>>(l, p, -8);
    if (use_momentum) return launch_rule<RmsPropRule<true, false>>(l, p, -8);
    if (centered) return launch_rule<RmsPropRule<false, true>>(l, p, -8);
    return launch_rule<RmsPropRule<false, false>>(l, p, -8);
} catch (...) {
    note_exception();
    return -8;
}

int execute_adagrad_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                  uintptr_t *gradient_buffers,
                                  uintptr_t *squared_grad_avg_buffers, int num_weights,
                                  int *buffer_sizes, float learning_rate, float epsilon,
                                  float weight_decay)
try {
    PlanRequest req{};
    req.kind = kRuleAdaGrad;
    req.num_tensors = num_weights;
    req.slot[kSlotWeight] = weight_buffers;
    req.slot[kSlotGrad] = gradient_buffers;
    req.slot[kSlotState0] = squared_grad_avg_buffers;
    req.sizes = buffer_sizes;
    req.skip_if_zero_mask = (1u << kSlotWeight) | (1u << kSlotGrad) | (1u << kSlotState0);
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = prepare(device, req, -8, l, lock)) return rc;
    StepParams p = zero_params();
    p.lr = learning_rate;
    p.eps = epsilon;
    p.weight_decay = weight_decay;
    return launch_rule<AdaGradRule>(l, p, -8);
} catch (...) {
    note_exception();
    return -8;
}

int execute_adagrad_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                         uintptr_t *gradient_buffers,
                                         uintptr_t *squared_grad_avg_buffers, int num_weights,
                                         int *buffer_sizes, float learning_rate, float epsilon,
                                         float weight_decay, uintptr_t command_pool)
try {
    (void)command_pool;
    return execute_adagrad_step_mpsgraph(device, weight_buffers, gradient_buffers,
                                         squared_grad_avg_buffers, num_weights, buffer_sizes,
                                         learning_rate, epsilon, weight_decay);
} catch (...) {
    note_exception();
    return -8;
}

int execute_adadelta_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                   uintptr_t *gradient_buffers,
                                   uintptr_t *squared_grad_avg_buffers,
                                   uintptr_t *squared_update_avg_buffers, int num_weights,
                                   int *buffer_sizes, float rho, float epsilon, float weight_decay)
try {
    PlanRequest req{};
    req.kind = kRuleAdaDelta;
    req.num_tensors = num_weights;
    req.slot[kSlotWeight] = weight_buffers;
    req.slot[kSlotGrad] = gradient_buffers;
    req.slot[kSlotState0] = squared_grad_avg_buffers;
    req.slot[kSlotState1] = squared_update_avg_buffers;
    req.sizes = buffer_sizes;
    req.skip_if_zero_mask = (1u << kSlotWeight) | (1u << kSlotGrad) | (1u << kSlotState0) |
                            (1u << kSlotState1);
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = prepare(device, req, -8, l, lock)) return rc;
    StepParams p = zero_params();
    p.rho = rho;
    p.one_minus_rho = 1.0f - rho;
    p.eps = epsilon;
    p.weight_decay = weight_decay;
    return launch_rule<AdaDeltaRule>(l, p, -8);
} catch (...) {
    note_exception();
    return -8;
}

int execute_adadelta_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                          uintptr_t *gradient_buffers,
                                          uintptr_t *squared_grad_avg_buffers,
                                          uintptr_t *squared_update_avg_buffers, int num_weights,
                                          int *buffer_sizes, float rho, float epsilon,
                                          float weight_decay, uintptr_t command_pool)
try {
    (void)command_pool;
    return execute_adadelta_step_mpsgraph(device, weight_buffers, gradient_buffers,
                                          squared_grad_avg_buffers, squared_update_avg_buffers,
                                          num_weights, buffer_sizes, rho, epsilon, weight_decay);
} catch (...) {
    note_exception();
    return -8;
}

// ---------------------------------------------------------- mixed precision --
struct AmpState {
    uint64_t magic;
    Context *ctx;
    AmpDeviceState *d_state;
    AmpDeviceState *h_pinned;            // kAmpMaxInFlight + 1 slots: [0] synchronous read-backs, [1..] the ring
    hipEvent_t ring_event[kAmpMaxInFlight];
    // asynchronous steps: issue numbers count execute_adam_amp_step_async calls
    uint64_t issued;                     // steps issued so far
    uint64_t confirmed_issue;            // newest step whose post-state the host has seen
    int confirmed_applied;               // the device's applied_steps after that step
    int max_in_flight;                   // deepest run-ahead seen (diagnostics)
};
static const uint64_t kAmpMagic = 0x676D5F616D705F73ull;   // "gm_amp_s"

static AmpState *amp_from_handle(uintptr_t h)
{
    if (h == 0) return nullptr;
    auto *s = reinterpret_cast<AmpState *>(h);
    return s->magic == kAmpMagic ? s : nullptr;
}

static bool amp_upload(AmpState *s)
{
    return hip_ok(hipMemcpyAsync(s->d_state, s->h_pinned, sizeof(AmpDeviceState),
                                 hipMemcpyHostToDevice, s->ctx->stream), "amp state upload") &&
           hip_ok(hipStreamSynchronize(s->ctx->stream), "hipStreamSynchronize");
}

// Waits for everything on the stream and reads the state back: afterwards no step is in flight.
static bool amp_download(AmpState *s)
{
    if (!hip_ok(hipMemcpyAsync(s->h_pinned, s->d_state, sizeof(AmpDeviceState),
                               hipMemcpyDeviceToHost, s->ctx->stream), "amp state download") ||
        !hip_ok(hipStreamSynchronize(s->ctx->stream), "hipStreamSynchronize"))
        return false;
    s->confirmed_issue = s->issued;
    s->confirmed_applied = s->h_pinned->applied_steps;
    return true;
}

// Takes note of the asynchronous steps that have finished since the last look.  With
// must_free_slot, blocks until at most kAmpMaxInFlight - 2 steps are unconfirmed, so that the
// next step's bias table and ring slot are available.
static bool amp_poll(AmpState *s, bool must_free_slot)
{
    for (;;) {
        while (s->confirmed_issue < s->issued) {
            const uint64_t next = s->confirmed_issue + 1;
            const hipError_t q = hipEventQuery(s->ring_event[next % kAmpMaxInFlight]);
            if (q == hipErrorNotReady) {
                (void)hipGetLastError();     // "not ready" is an answer, not a failure to report later
                break;
            }
            if (!hip_ok(q, "hipEventQuery")) return false;
            s->confirmed_issue = next;
            s->confirmed_applied = s->h_pinned[1 + next % kAmpMaxInFlight].applied_steps;
        }
        if (!must_free_slot || s->issued - s->confirmed_issue <= (uint64_t)kAmpMaxInFlight - 2) return true;
        const uint64_t oldest = s->confirmed_issue + 1;
        if (!hip_ok(hipEventSynchronize(s->ring_event[oldest % kAmpMaxInFlight]), "hipEventSynchronize"))
            return false;
    }
}

static void amp_free(AmpState *s)
{
    if (s->d_state) (void)hipFree(s->d_state);
    if (s->h_pinned) (void)hipHostFree(s->h_pinned);
    for (hipEvent_t e : s->ring_event)
        if (e) (void)hipEventDestroy(e);
    s->magic = 0;
    delete s;
}

uintptr_t gm_amp_state_create(uintptr_t device, float init_scale, float growth_factor,
                              float backoff_factor, int growth_interval)
try {
    clear_error();
    if (device == 0) return 0;
    Context *ctx = resolve_device(device);
    if (!ctx || !make_current(ctx)) return 0;
    auto *s = new AmpState{};
    s->magic = kAmpMagic;
    s->ctx = ctx;
    bool ok = hip_ok(hipMalloc(&s->d_state, sizeof(AmpDeviceState)), "hipMalloc(amp state)") &&
              hip_ok(hipHostMalloc(&s->h_pinned, (kAmpMaxInFlight + 1) * sizeof(AmpDeviceState),
                                   hipHostMallocDefault), "hipHostMalloc(amp state)");
    for (int k = 0; ok && k < kAmpMaxInFlight; k++)
        ok = hip_ok(hipEventCreateWithFlags(&s->ring_event[k], hipEventDisableTiming), "hipEventCreate");
    if (ok) {
        std::memset(s->h_pinned, 0, (kAmpMaxInFlight + 1) * sizeof(AmpDeviceState));
        s->h_pinned->scale = init_scale;
        s->h_pinned->inv_scale = 1.0f / init_scale;
        s->h_pinned->growth_factor = growth_factor;
        s->h_pinned->backoff_factor = backoff_factor;
        s->h_pinned->growth_interval = growth_interval;
        std::lock_guard<std::mutex> lk(ctx->mu);
        ok = amp_upload(s);
    }
    if (!ok) {
        amp_free(s);
        return 0;
    }
    return reinterpret_cast<uintptr_t>(s);
} catch (...) {
    note_exception();
    return 0;
}

void gm_amp_state_destroy(uintptr_t amp_state)
try {
    AmpState *s = amp_from_handle(amp_state);
    if (!s) return;
    make_current(s->ctx);
    (void)hipStreamSynchronize(s->ctx->stream);     // ring copies may still be in flight
    amp_free(s);
} catch (...) {
    note_exception();
}

int gm_amp_state_get(uintptr_t amp_state, float *scale, int *growth_tracker)
{
    return gm_amp_state_query(amp_state, scale, growth_tracker, nullptr, nullptr);
}

int gm_amp_state_query(uintptr_t amp_state, float *scale, int *growth_tracker, int *applied_steps,
                       int *skipped_steps)
try {
    AmpState *s = amp_from_handle(amp_state);
    if (!s) return -16;
    if (!make_current(s->ctx)) return -6;
    std::lock_guard<std::mutex> lk(s->ctx->mu);
    if (!amp_download(s)) return -6;
    if (scale) *scale = s->h_pinned->scale;
    if (growth_tracker) *growth_tracker = s->h_pinned->growth_tracker;
    if (applied_steps) *applied_steps = s->h_pinned->applied_steps;
    if (skipped_steps) *skipped_steps = s->h_pinned->skipped_steps;
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

int gm_amp_state_max_in_flight(uintptr_t amp_state)
{
    AmpState *s = amp_from_handle(amp_state);
    return s ? s->max_in_flight : -16;
}

int gm_amp_state_set(uintptr_t amp_state, float scale, int growth_tracker)
try {
    AmpState *s = amp_from_handle(amp_state);
    if (!s) return -16;
    if (!make_current(s->ctx)) return -6;
    std::lock_guard<std::mutex> lk(s->ctx->mu);
    if (!amp_download(s)) return -6;
    s->h_pinned->scale = scale;
    s->h_pinned->inv_scale = 1.0f / scale;
    s->h_pinned->growth_tracker = growth_tracker;
    return amp_upload(s) ? 0 : -6;
} catch (...) {
    note_exception();
    return -6;
}

int gm_amp_state_set_step_count(uintptr_t amp_state, int applied_steps)
try {
    AmpState *s = amp_from_handle(amp_state);
    if (!s) return -16;
    if (applied_steps < 0) return -5;
    if (!make_current(s->ctx)) return -6;
    std::lock_guard<std::mutex> lk(s->ctx->mu);
    if (!amp_download(s)) return -6;
    s->h_pinned->applied_steps = applied_steps;
    if (!amp_upload(s)) return -6;
    s->confirmed_applied = applied_steps;
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

// Plan, parameters and the three launches shared by the synchronous and the asynchronous step.
static int amp_enqueue(uintptr_t device, AmpState *amp, uintptr_t *weight_buffers,
                       uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                       uintptr_t *variance_buffers, uintptr_t *weight16_buffers, int num_weights,
                       int *buffer_sizes, float learning_rate, float beta1, float beta2, float epsilon,
                       float weight_decay, int step_count, bool async, Launch &l,
                       std::unique_lock<std::mutex> &lock)
{
    PlanRequest req{};
    req.kind = kRuleAdamAMP;
    req.num_tensors = num_weights;
    req.slot[kSlotWeight] = weight_buffers;
    req.slot[kSlotGrad] = gradient16_buffers;
    req.slot[kSlotState0] = momentum_buffers;
    req.slot[kSlotState1] = variance_buffers;
    req.slot[kSlotWeight16] = weight16_buffers;
    req.sizes = buffer_sizes;
    req.required_mask = (1u << kSlotWeight) | (1u << kSlotGrad) | (1u << kSlotState0) | (1u << kSlotState1);
    req.missing_code = -4;
    req.half_mask = (1u << kSlotGrad) | (1u << kSlotWeight16);
    if (int rc = prepare(device, req, -6, l, lock)) return rc;
    if (l.ctx != amp->ctx) {
        set_error("the loss-scale state belongs to another device context");
        return -16;
    }

    StepParams p = zero_params();
    p.lr = learning_rate;
    p.beta1 = beta1;
    p.beta2 = beta2;
    p.one_minus_beta1 = 1.0f - beta1;
    p.one_minus_beta2 = 1.0f - beta2;
    p.eps = epsilon;
    p.weight_decay = weight_decay;

    // The context lock is held from here on: the issue counters of the loss-scale state are
    // only read and advanced under it.  An asynchronous step's post-state goes into the ring
    // slot of its issue number, a synchronous step's into slot 0.
    AmpDeviceState *host_mirror = amp->h_pinned;
    AmpBiasTable bias{};
    if (async) {
        if (!amp_poll(amp, true)) return -6;
        host_mirror = &amp->h_pinned[1 + (amp->issued + 1) % kAmpMaxInFlight];
        const int in_flight = (int)(amp->issued - amp->confirmed_issue);
        if (in_flight > amp->max_in_flight) amp->max_in_flight = in_flight;
        bias.base = amp->confirmed_applied;
        bias.count = in_flight + 1;
        for (int j = 0; j <= in_flight; j++)
            gm_bias_corrections(beta1, beta2, amp->confirmed_applied + 1 + j, &bias.bc1[j], &bias.bc2[j]);
    } else {
        bias.count = 1;
        gm_bias_corrections(beta1, beta2, step_count, &bias.bc1[0], &bias.bc2[0]);
    }

    const uint32_t chunks = l.plan->num_chunks;
    hipStream_t st = l.ctx->stream;
    if (chunks > 0) {
        int vec = current_vec();
        if (vec == 0) vec = auto_vec(8);
        const bool nt = current_nontemporal();
        int block = current_block();
        if (block == 0) block = auto_block(8);
        SegmentLaunch seg[2];
        int count;
        if (!launch_geometry(*l.plan, vec, block, seg, count)) return -6;
        // the check walks the whole table, one workgroup per chunk of either segment
        if (nt) amp_overflow_check_kernel<true><<<chunks, kBlock, 0, st>>>(l.plan->d_chunks, amp->d_state);
        else amp_overflow_check_kernel<false><<<chunks, kBlock, 0, st>>>(l.plan->d_chunks, amp->d_state);
#define GM_LAUNCH_AMP(V, N, B) amp_adam_update_kernel<V, N, B><<<g.grid, B, 0, st>>>(g.chunks, g.shift, p, amp->d_state, bias)
#define GM_LAUNCH_AMP_B(B)                                                              \
        if (vec == 4) { if (nt) GM_LAUNCH_AMP(4, true, B); else GM_LAUNCH_AMP(4, false, B); }        \
        else if (vec == 2) { if (nt) GM_LAUNCH_AMP(2, true, B); else GM_LAUNCH_AMP(2, false, B); }   \
        else { if (nt) GM_LAUNCH_AMP(1, true, B); else GM_LAUNCH_AMP(1, false, B); }
        for (int s = 0; s < count; s++) {
            const SegmentLaunch &g = seg[s];
            if (block == 128) { GM_LAUNCH_AMP_B(128) } else { GM_LAUNCH_AMP_B(kBlock) }
        }
#undef GM_LAUNCH_AMP_B
#undef GM_LAUNCH_AMP
    }
    amp_finalize_kernel<<<1, 64, 0, st>>>(amp->d_state, host_mirror);
    return hip_ok(hipGetLastError(), "mixed-precision kernel launch") ? 0 : -6;
}

int execute_adam_amp_step(uintptr_t device, uintptr_t *weight_buffers,
                          uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                          uintptr_t *variance_buffers, uintptr_t *weight16_buffers,
                          int num_weights, int *buffer_sizes, float learning_rate, float beta1,
                          float beta2, float epsilon, float weight_decay, int step_count,
                          uintptr_t amp_state, int *skipped, float *scale_out,
                          int *growth_tracker_out)
try {
    if (device == 0) return -1;
    AmpState *amp = amp_from_handle(amp_state);
    if (!amp) return -16;
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = amp_enqueue(device, amp, weight_buffers, gradient16_buffers, momentum_buffers,
                             variance_buffers, weight16_buffers, num_weights, buffer_sizes, learning_rate,
                             beta1, beta2, epsilon, weight_decay, step_count, false, l, lock))
        return rc;
    if (!hip_ok(hipStreamSynchronize(l.ctx->stream), "hipStreamSynchronize")) return -6;
    amp->confirmed_issue = amp->issued;
    amp->confirmed_applied = amp->h_pinned->applied_steps;
    if (skipped) *skipped = amp->h_pinned->last_skipped;
    if (scale_out) *scale_out = amp->h_pinned->scale;
    if (growth_tracker_out) *growth_tracker_out = amp->h_pinned->growth_tracker;
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

int execute_adam_amp_step_async(uintptr_t device, uintptr_t *weight_buffers,
                                uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                                uintptr_t *variance_buffers, uintptr_t *weight16_buffers,
                                int num_weights, int *buffer_sizes, float learning_rate, float beta1,
                                float beta2, float epsilon, float weight_decay, uintptr_t amp_state)
try {
    if (device == 0) return -1;
    AmpState *amp = amp_from_handle(amp_state);
    if (!amp) return -16;
    Launch l{};
    std::unique_lock<std::mutex> lock;
    if (int rc = amp_enqueue(device, amp, weight_buffers, gradient16_buffers, momentum_buffers,
                             variance_buffers, weight16_buffers, num_weights, buffer_sizes, learning_rate,
                             beta1, beta2, epsilon, weight_decay, 0, true, l, lock))
        return rc;
    // the event marks the arrival of this step's post-state in its ring slot
    const uint64_t issue = amp->issued + 1;
    const int slot = (int)(issue % kAmpMaxInFlight);
    if (!hip_ok(hipEventRecord(amp->ring_event[slot], l.ctx->stream), "hipEventRecord")) {
        // the step itself is enqueued; resynchronise the bookkeeping with the device
        (void)amp_download(amp);
        return -6;
    }
    amp->issued = issue;
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

}  // extern "C"
