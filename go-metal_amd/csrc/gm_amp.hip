// Mixed-precision (fp16-gradient) Adam step for gfx950: overflow check, update with fp16 weight
// copy, loss-scale state machine; synchronous and run-ahead entry points.
//
// An inf in the last tensor must suppress the write to the first, and the Adam update is not
// exactly invertible.  Two forms follow from that:
//
// in place (execute_adam_amp_step[_async]): weights and moments are updated where they lie, so
//   nothing may be written before every gradient has been checked: a check launch reads the fp16
//   gradients, an update launch reads them again (30 bytes move per parameter for 28 algorithmic
//   ones); one lane of the update launch advances the loss-scale state.
// ping-pong (execute_adam_amp_step_fused[_async]): weights and moments exist twice (sets A and B),
//   one of them current.  ONE launch reads the current set and the gradients, checks the
//   gradients as it goes, and writes the other set; the epilogue makes that set current only if
//   no gradient overflowed.  A dropped step leaves the current set untouched because it was
//   never written: every stream moves once, 28 bytes per parameter.  The fp16 weight copy has a
//   single consumer-visible buffer and is written speculatively; after a dropped step a repair
//   pass (which returns at once after an applied one) rewrites it from the current weights.
//
// The loss-scale state lives in HBM as two records and an overflow word.  A step reads one record
// (its pre-state) and one lane writes the advanced state into the other, which the next step
// reads: no kernel reads a record that the same launch writes.  The overflow word holds the
// stamp of the last step that saw an inf / NaN; every step carries its own 64-bit stamp, so the
// word needs no clearing and means "this step overflowed" only while it equals this step's stamp.
#include "gm_launch.hpp"
#include "gm_update_kernels.hpp"

#include "../../include/gometal_hip.h"

#include <chrono>
#include <cstddef>
#include <cstring>
#include <thread>

namespace gm {

constexpr float kMinLossScale = 1.17549435e-38f;   // FLT_MIN
constexpr float kMaxLossScale = 3.40282347e+38f;   // FLT_MAX
constexpr int kAmpSpinMicroseconds = 100;   // how long the host spins on a pinned stamp before it naps or blocks
constexpr int kCheckUnroll = 4;           // 16-byte loads in flight per lane in the overflow check

// Loss-scale state machine, resident in HBM next to the tensors.
struct alignas(16) AmpDeviceState {
    // head: the 16 bytes every workgroup of the update kernel reads with one scalar load
    int current_set;        // ping-pong step: 0 = set A holds the current weights and moments, 1 = set B
    float inv_scale;        // 1.0f / scale, kept by whoever changes scale (IEEE division on host and device alike)
    int skipped_steps;      // steps dropped so far
    int applied_steps;      // steps applied so far (the optimizer's StepCount): +1 per clean step
    // tail
    float scale;
    int growth_tracker;
    int last_skipped;
    float growth_factor;
    float backoff_factor;
    int growth_interval;
    unsigned long long stamp;   // the stamp of the step this record is the post-state of (0: set by the host).  In
                                // the pinned host copy it is written last: the host knows the record is complete
                                // when it reads the stamp it expects
};
static_assert(offsetof(AmpDeviceState, stamp) == 40, "AmpDeviceState layout");
static_assert(sizeof(AmpDeviceState) == 48, "AmpDeviceState layout");

// What a loss-scale state keeps on the device: the record the next step reads and the record it
// writes (they swap roles with every step), and the stamp of the last step that overflowed.
struct alignas(16) AmpDeviceBlock {
    AmpDeviceState slot[2];
    unsigned long long overflow;
    unsigned long long pad;
};
static_assert(sizeof(AmpDeviceBlock) == 112, "AmpDeviceBlock layout");

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
// one store of the step's stamp per workgroup that saw a hit.
template <bool NT>
__global__ void __launch_bounds__(kBlock)
amp_overflow_check_kernel(const Chunk *__restrict__ chunks, unsigned long long *__restrict__ overflow, int reverse,
                          unsigned long long stamp, uint32_t num_chunks, uint32_t split_shift)
{
    __shared__ unsigned int wave_hit[kBlock / 64];
    // A list of few chunks is checked by several workgroups per chunk (1 << split_shift of them, each taking
    // a run of whole 2048-element rows), so that a 1M-parameter tensor in sixteen 65536-element chunks is not
    // read by sixteen workgroups; lists of a thousand chunks and more take one workgroup per chunk.
    const uint32_t c = blockIdx.x >> split_shift;
    const uint32_t part = blockIdx.x & ((1u << split_shift) - 1u);
    // reverse: the table is walked from its end, so that the check finishes on the gradients the
    // update pass reads first (what is left of them in the memory-side cache is then the nearest)
    const Chunk ch = chunks[reverse ? num_chunks - 1u - c : c];
    const unsigned short *g = reinterpret_cast<const unsigned short *>(ch.p[kSlotGrad]);
    const uint32_t per_part = (((ch.count + (1u << split_shift) - 1u) >> split_shift) + 2047u) & ~2047u;
    const uint32_t lo = part * per_part < ch.count ? part * per_part : ch.count;
    const uint32_t hi = ch.count - lo < per_part ? ch.count : lo + per_part;
    unsigned int bad = 0;
    uint32_t done = lo;
    if (ch.flags & kRecGrad16VectorOk) {
        const uint32_t n8 = hi >> 3;
        const uintx4 *g8 = reinterpret_cast<const uintx4 *>(g);
        for (uint32_t base = (lo >> 3) + threadIdx.x; base < n8; base += kBlock * kCheckUnroll) {
            uintx4 v[kCheckUnroll];
#pragma unroll
            for (int u = 0; u < kCheckUnroll; u++) {
                const uint32_t i = base + u * kBlock;
                v[u] = (i < n8) ? stream_load<NT>(g8 + i) : uintx4{0u, 0u, 0u, 0u};
            }
#pragma unroll
            for (int u = 0; u < kCheckUnroll; u++) {
#pragma unroll
                for (int c4 = 0; c4 < 4; c4++) {
                    const unsigned int e = v[u][c4] & 0x7C007C00u;
                    bad |= ((e & 0xFFFFu) == 0x7C00u) | ((e >> 16) == 0x7C00u);
                }
            }
        }
        done = n8 << 3 > lo ? n8 << 3 : lo;
    }
    for (uint32_t i = done + threadIdx.x; i < hi; i += kBlock)
        bad |= ((stream_load<false>(g + i) & 0x7C00u) == 0x7C00u);

    const unsigned long long ballot = __ballot(bad != 0);
    if ((threadIdx.x & 63) == 0) wave_hit[threadIdx.x >> 6] = (ballot != 0ull);
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned int any = 0;
#pragma unroll
        for (int k = 0; k < kBlock / 64; k++) any |= wave_hit[k];
        if (any) __hip_atomic_store(overflow, stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
}

// Advances the loss-scale state machine after a step (one lane): reads the step's pre-state and
// writes its post-state into the record the next step reads.  found: this step's gradients held
// an inf / NaN.
__device__ inline void amp_advance(const AmpDeviceState *pre, AmpDeviceState *post, AmpDeviceState *host_mirror,
                                   bool found, int ping_pong, unsigned long long stamp)
{
    AmpDeviceState st = *pre;
    // The scale stays a normal, finite fp32 number whatever the run does: a growth that would
    // overflow to infinity (about 112 uninterrupted growth intervals from 65536) and a backoff
    // that would leave the normal range are not applied.  Unbounded, the scale would stick at
    // +inf (inf * 0.5 = inf) with a reciprocal of 0, or reach 0 with a reciprocal of +inf.
    if (found) {
        const float next = st.scale * st.backoff_factor;
        if (next >= kMinLossScale) st.scale = next;
        st.growth_tracker = 0;
        st.skipped_steps += 1;
    } else {
        st.applied_steps += 1;
        if (ping_pong) st.current_set ^= 1;      // the set just written is the current one from here on
        st.growth_tracker += 1;
        if (st.growth_tracker == st.growth_interval) {
            const float next = st.scale * st.growth_factor;
            if (next <= kMaxLossScale) st.scale = next;
            st.growth_tracker = 0;
        }
    }
    st.inv_scale = 1.0f / st.scale;
    st.last_skipped = found ? 1 : 0;
    st.stamp = stamp;
    *post = st;
    // The post-state also goes straight into pinned host memory, its stamp last and behind a
    // system-scope fence: the host reads the record without a copy launch, either after the stream
    // has completed or as soon as it sees the stamp of the step it is waiting for.
    if (host_mirror) {
        const unsigned long long *src = reinterpret_cast<const unsigned long long *>(&st);
        unsigned long long *dst = reinterpret_cast<unsigned long long *>(host_mirror);
#pragma unroll
        for (int k = 0; k < 5; k++) dst[k] = src[k];
        __threadfence_system();
        __hip_atomic_store(&host_mirror->stamp, stamp, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_SYSTEM);
    }
}

// The bias corrections of the step count the device has reached: entry (applied - base) of the
// table, clamped; entry 0 when the table has one entry.
__device__ inline void amp_pick_bias(StepParams &prm, const AmpBiasTable &bias, int applied)
{
    int pick = bias.count > 1 ? applied - bias.base : 0;
    pick = pick < 0 ? 0 : (pick >= bias.count ? bias.count - 1 : pick);
    // (the table sits in the kernel-argument segment: an indexed scalar load, no copy to scratch)
    prm.bc1 = bias.bc1[pick];
    prm.bc2 = bias.bc2[pick];
}

// Phase B: the Adam update on unscaled gradients, skipped as a whole when the check stored this
// step's stamp.  The launch also carries the step's epilogue: with `post` set, lane 0 of workgroup
// 0 advances the loss-scale state from the pre-state into the other record (the check has
// finished, so every workgroup of this launch sees the same decision; nothing it reads is written
// while it runs).
template <int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
amp_adam_update_kernel(const Chunk *__restrict__ chunks, uint32_t slice_shift, StepParams prm,
                       const AmpDeviceState *__restrict__ pre, const unsigned long long *__restrict__ overflow,
                       AmpBiasTable bias, unsigned long long stamp, AmpDeviceState *post, AmpDeviceState *host_mirror)
{
    // The pre-state's head (current set, reciprocal of the scale, applied steps) comes with one 16-byte scalar load,
    // the overflow word with another and the chunk descriptor with a third, all issued before anything is decided;
    // the bias table sits in the kernel arguments and its entry comes with an indexed scalar load.
    const uintx4 head = *reinterpret_cast<const uintx4 *>(pre);
    const unsigned long long seen = *overflow;
    const Chunk ch = chunks[blockIdx.x >> slice_shift];
    __builtin_amdgcn_sched_barrier(0);     // all three fetches are issued before the first of them is waited for
    const uint32_t first_lane_element = (blockIdx.x & ((1u << slice_shift) - 1u)) * BLOCK * VEC;
    const bool found = seen == stamp;
    // (the epilogue sits behind the update's loads and stores, not in front of them: a workgroup lives for a
    // microsecond or two, and whatever stands between its start and its first global load shows in the bandwidth)
    const bool epilogue = post != nullptr && blockIdx.x == 0;
    // (the weight pointer is never null; testing it here makes the compiler fetch the whole
    // descriptor before the branch instead of the count first and the addresses after it)
    if (found | (first_lane_element >= ch.count) | (ch.p[kSlotWeight] == nullptr)) {
        // step dropped, or an idle slice
        if (epilogue && threadIdx.x == 0) amp_advance(pre, post, host_mirror, found, 0, stamp);
        return;
    }
    const float inv_scale = __uint_as_float(head.y);
    amp_pick_bias(prm, bias, (int)head.w);
    update_slice<AdamRule, VEC, NT, true, BLOCK>(ch, slice_shift, prm, inv_scale);
    if (epilogue && threadIdx.x == 0) amp_advance(pre, post, host_mirror, found, 0, stamp);
}

// One lane's share in two halves, so that the kernel can issue its global loads, do its scalar
// bookkeeping (bias-correction pick) while they are in flight, and only then compute and store.
template <int N>
struct FusedLoaded {
    typename VecOf<float, N>::type W, M, V;
    typename VecOf<unsigned short, N>::type H;
};

template <int N, bool NT>
__device__ inline FusedLoaded<N> amp_fused_load(const Chunk &in, uint32_t first)
{
    typedef typename VecOf<float, N>::type FV;
    typedef typename VecOf<unsigned short, N>::type UV;
    FusedLoaded<N> x;
    x.W = stream_load<NT>(reinterpret_cast<const FV *>(reinterpret_cast<const float *>(in.p[kSlotWeight]) + first));
    x.H = stream_load<NT>(reinterpret_cast<const UV *>(reinterpret_cast<const unsigned short *>(in.p[kSlotGrad]) + first));
    x.M = stream_load<NT>(reinterpret_cast<const FV *>(reinterpret_cast<const float *>(in.p[kSlotState0]) + first));
    x.V = stream_load<NT>(reinterpret_cast<const FV *>(reinterpret_cast<const float *>(in.p[kSlotState1]) + first));
    return x;
}

// Computes the update of the loaded share and stores it into the other set (and the fp16 copy);
// true when one of its gradients is +-inf or NaN.
template <int N, bool NT>
__device__ inline bool amp_fused_finish(const FusedLoaded<N> &x, const Chunk &out, uint32_t first, const StepParams &prm,
                                        float inv_scale)
{
    typedef typename VecOf<float, N>::type FV;
    typedef typename VecOf<_Float16, N>::type HV;
    FV Wn, Mn, Vn;
    HV Hn;
    bool bad = false;
#pragma unroll
    for (int c = 0; c < N; c++) {
        const unsigned short bits = lane_of<N>(x.H, c);
        bad |= (bits & 0x7C00u) == 0x7C00u;
        float wv = lane_of<N>(x.W, c);
        float sv[2] = {lane_of<N>(x.M, c), lane_of<N>(x.V, c)};
        const float gv = (float)__builtin_bit_cast(_Float16, bits) * inv_scale;
        AdamRule::apply(wv, gv, sv, prm);
        set_lane<N>(Wn, c, wv);
        set_lane<N>(Mn, c, sv[0]);
        set_lane<N>(Vn, c, sv[1]);
        set_lane<N>(Hn, c, (_Float16)wv);
    }
    stream_store<NT>(Wn, reinterpret_cast<FV *>(reinterpret_cast<float *>(out.p[kSlotWeight]) + first));
    stream_store<NT>(Mn, reinterpret_cast<FV *>(reinterpret_cast<float *>(out.p[kSlotState0]) + first));
    stream_store<NT>(Vn, reinterpret_cast<FV *>(reinterpret_cast<float *>(out.p[kSlotState1]) + first));
    if (out.p[kSlotWeight16])
        stream_store<NT>(Hn, reinterpret_cast<HV *>(reinterpret_cast<_Float16 *>(out.p[kSlotWeight16]) + first));
    return bad;
}

// The ping-pong step: one pass.  Reads weights and moments of the current set and the fp16
// gradients, writes the other set and the fp16 weight copy, and stores the step's stamp when a
// gradient of its own is +-inf or NaN.  Its arithmetic never looks at the stamp: what it writes
// becomes current only if the epilogue finds that no workgroup stored it.  (The overflow word is
// accessed with atomic loads and stores only while this launch runs; the pre-state is read-only.)
// (The state pointer is the first argument and the early exit tests the head: both make the
// compiler fetch the state's head together with the two descriptors, straight after the kernel
// arguments, instead of behind the first branch; that shortens the chain of dependent scalar
// loads in front of the first global load from four to two.)
template <int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
amp_adam_fused_kernel(const AmpDeviceState *__restrict__ pre, const Chunk *__restrict__ set_a,
                      const Chunk *__restrict__ set_b, uint32_t slice_shift, StepParams prm, AmpBiasTable bias,
                      unsigned long long stamp, unsigned long long *__restrict__ overflow)
{
    const uintx4 head = *reinterpret_cast<const uintx4 *>(pre);
    const uint32_t c = blockIdx.x >> slice_shift;
    const Chunk a = set_a[c];
    const Chunk b = set_b[c];
    const uint32_t slice = blockIdx.x & ((1u << slice_shift) - 1u);
    // (a reciprocal scale of zero bits cannot occur: the scale is finite)
    // (an empty bias table cannot occur either; testing it here brings its size and base in together
    // with the descriptors, so the pick below is a dozen scalar instructions and not another
    // fetch-and-wait in front of the global loads)
    // (the dropped-step count is never negative either; testing it keeps all four words of the head alive up to
    // this point: with a dead word among them the compiler reuses its register for the chunk's element count while
    // the head is still in flight, and has to wait for the first descriptor before it may fetch the second)
    if ((slice * BLOCK * VEC >= a.count) | (a.p[kSlotWeight] == nullptr) | (b.p[kSlotWeight] == nullptr) | (head.y == 0u) |
        (bias.count < 1) | (bias.base < 0) | ((int)head.z < 0))
        return;
    const bool b_is_current = head.x != 0u;
    const Chunk &in = b_is_current ? b : a;
    const Chunk &out = b_is_current ? a : b;
    const float inv_scale = __uint_as_float(head.y);
    // vec-wide lanes need both sets aligned for them
    const LaneShare s = lane_share(a.count, a.flags & b.flags, slice, threadIdx.x, VEC, BLOCK);
    const bool whole = s.count != 0 && (VEC == 1 || s.grouped);
    FusedLoaded<VEC> loaded;
    if (whole) loaded = amp_fused_load<VEC, NT>(in, s.first);
    amp_pick_bias(prm, bias, (int)head.w);
    bool bad = false;
    if (whole) {
        bad = amp_fused_finish<VEC, NT>(loaded, out, s.first, prm, inv_scale);
    } else {
        for (uint32_t e = 0; e < s.count; e++)
            bad |= amp_fused_finish<1, NT>(amp_fused_load<1, NT>(in, s.first + e), out, s.first + e, prm, inv_scale);
    }
    // One store per wavefront that saw a hit, and none once the stamp is in (a tensor of nothing but
    // inf would otherwise send millions of stores to one address).  Every writer stores the same value.
    const unsigned long long hit = __ballot(bad);
    if (hit != 0ull && (threadIdx.x & 63u) == (unsigned int)(__ffsll((long long)hit) - 1) &&
        __hip_atomic_load(overflow, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != stamp)
        __hip_atomic_store(overflow, stamp, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Epilogue of a step over an empty list (one lane): there is no update launch to carry it.
__global__ void amp_finalize_kernel(const AmpDeviceState *pre, AmpDeviceState *post, AmpDeviceState *host_mirror,
                                    const unsigned long long *overflow, unsigned long long stamp, int ping_pong)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    amp_advance(pre, post, host_mirror, *overflow == stamp, ping_pong, stamp);
}

// Epilogue of the ping-pong step, and the repair of the fp16 weight copy, in one launch.  After a
// dropped step the copy holds what the discarded update wrote: it is rewritten from the current
// weights (the copy of an applied step is half(w) by construction, so this restores it bit for
// bit).  Small fixed grid; after an applied step every workgroup returns on its first load.
// Lane 0 of workgroup 0 writes the advanced state into the record the next step reads; what the
// workgroups of this launch read (the overflow word, the current set of the pre-state) is
// written by nobody while it runs.
__global__ void __launch_bounds__(kBlock)
amp_finalize_repair_kernel(const AmpDeviceState *pre, AmpDeviceState *post, AmpDeviceState *host_mirror,
                           const unsigned long long *overflow, unsigned long long stamp,
                           const Chunk *__restrict__ set_a, const Chunk *__restrict__ set_b, uint32_t num_chunks)
{
    const bool found = *overflow == stamp;
    if (blockIdx.x == 0 && threadIdx.x == 0) amp_advance(pre, post, host_mirror, found, 1, stamp);
    if (!found) return;
    const Chunk *current = pre->current_set != 0 ? set_b : set_a;      // a dropped step keeps the current set
    for (uint32_t c = blockIdx.x; c < num_chunks; c += gridDim.x) {
        const Chunk ch = current[c];
        if (ch.p[kSlotWeight16] == nullptr) continue;
        const float *w = reinterpret_cast<const float *>(ch.p[kSlotWeight]);
        _Float16 *h = reinterpret_cast<_Float16 *>(ch.p[kSlotWeight16]);
        for (uint32_t e = threadIdx.x; e < ch.count; e += kBlock) h[e] = (_Float16)w[e];
    }
}

}  // namespace gm

using namespace gm;

extern "C" {

// ---------------------------------------------------------- mixed precision --
struct AmpState {
    uint64_t magic;
    Context *ctx;
    AmpDeviceBlock *d_block;
    int slot;                            // which record of d_block the next step reads (the state as of now)
    AmpDeviceState *h_pinned;            // kAmpMaxInFlight + 1 slots: [0] synchronous read-backs, [1..] the ring
    unsigned long long ring_stamp[kAmpMaxInFlight];    // stamp of the asynchronous step whose post-state a ring slot awaits
    // asynchronous steps: issue numbers count execute_adam_amp_step_async calls
    uint64_t issued;                     // steps issued so far
    uint64_t confirmed_issue;            // newest step whose post-state the host has seen
    int confirmed_applied;               // the device's applied_steps after that step
    int max_in_flight;                   // deepest run-ahead seen (diagnostics)
    unsigned long long last_stamp;       // stamp of the newest step issued (either form); never 0, never repeats
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
    return hip_ok(hipMemcpyAsync(&s->d_block->slot[s->slot], s->h_pinned, sizeof(AmpDeviceState),
                                 hipMemcpyHostToDevice, s->ctx->stream), "amp state upload") &&
           hip_ok(hipStreamSynchronize(s->ctx->stream), "hipStreamSynchronize");
}

// Waits for everything on the stream and reads the state back: afterwards no step is in flight.
static bool amp_download(AmpState *s)
{
    if (!hip_ok(hipMemcpyAsync(s->h_pinned, &s->d_block->slot[s->slot], sizeof(AmpDeviceState),
                               hipMemcpyDeviceToHost, s->ctx->stream), "amp state download") ||
        !hip_ok(hipStreamSynchronize(s->ctx->stream), "hipStreamSynchronize"))
        return false;
    s->confirmed_issue = s->issued;
    s->confirmed_applied = s->h_pinned->applied_steps;
    return true;
}

// Waiting for a stamp in pinned memory: a spin for outcomes that are microseconds away, then naps
// whose length grows with the time already waited (an eighth of it, 20 us to 1 ms), so that the
// outcome is noticed within an eighth of the time it took to come and a long step costs the host
// few wake-ups.  A look at host memory is free for the device; asking the runtime whether the
// stream is still busy is not (65 queries in a 4.6 ms step cost the step 0.6 % of its bandwidth),
// so that happens every 50 ms only, to end the wait if the stream has drained or failed.
struct AmpWait {
    std::chrono::steady_clock::time_point start = std::chrono::steady_clock::now();
    std::chrono::steady_clock::time_point last_query = start;
    bool spinning() const { return std::chrono::steady_clock::now() - start < std::chrono::microseconds(kAmpSpinMicroseconds); }
};
// 1: the stream has drained (whatever was awaited has been written), 0: look again, -1: the stream failed.
static int amp_nap(AmpState *s, AmpWait &w)
{
    const auto now = std::chrono::steady_clock::now();
    if (now - w.last_query >= std::chrono::milliseconds(50)) {
        w.last_query = now;
        const hipError_t q = hipStreamQuery(s->ctx->stream);
        if (q == hipSuccess) return 1;
        if (q != hipErrorNotReady) return hip_ok(q, "hipStreamQuery") ? 1 : -1;
        (void)hipGetLastError();     // "not ready" is an answer, not a failure to report later
    }
    long long us = std::chrono::duration_cast<std::chrono::microseconds>(now - w.start).count() / 8;
    us = us < 20 ? 20 : (us > 1000 ? 1000 : us);
    std::this_thread::sleep_for(std::chrono::microseconds(us));
    return 0;
}

// Whether the post-state of asynchronous step `issue` has arrived in its ring slot.
static bool amp_arrived(const AmpState *s, uint64_t issue)
{
    const int slot = (int)(issue % kAmpMaxInFlight);
    return __atomic_load_n(&s->h_pinned[1 + slot].stamp, __ATOMIC_ACQUIRE) == s->ring_stamp[slot];
}

// Takes note of the asynchronous steps that have finished since the last look: a step has
// finished when its ring slot holds its stamp (the device writes the stamp last).  No HIP call
// in the common case.  With must_free_slot, waits until at most kAmpMaxInFlight - 2 steps are
// unconfirmed, so that the next step's bias table and ring slot are available: a short spin for
// steps of microseconds, then naps (amp_nap); a stream that has drained or failed ends the wait,
// so it cannot outlast the work it waits for.
static bool amp_poll(AmpState *s, bool must_free_slot)
{
    AmpWait wait;
    for (;;) {
        while (s->confirmed_issue < s->issued && amp_arrived(s, s->confirmed_issue + 1)) {
            s->confirmed_issue += 1;
            s->confirmed_applied = s->h_pinned[1 + s->confirmed_issue % kAmpMaxInFlight].applied_steps;
        }
        if (!must_free_slot || s->issued - s->confirmed_issue <= (uint64_t)kAmpMaxInFlight - 2) return true;
        if (wait.spinning()) continue;
        const int drained = amp_nap(s, wait);
        if (drained < 0) return false;
        if (drained == 0) continue;
        // the stream is empty: every step has written its slot
        if (!amp_arrived(s, s->issued)) {
            set_error("a mixed-precision step finished without reporting its state");
            return false;
        }
    }
}

// Waits until the post-state of the synchronous step with this stamp has arrived in pinned slot 0
// (the device writes the stamp last).  The in-place step reports from the first workgroup of its
// update launch, as soon as the check has finished, so its outcome is known long before the
// update has drained: the wait spins briefly, then naps (naps: true).  The one-pass step reports
// from its last launch, when the stream is about to drain: after the spin the stream's own wait
// is the cheaper one (naps: false).  A stream that has drained or failed ends either wait.
static bool amp_wait_outcome(AmpState *s, unsigned long long stamp, bool naps)
{
    const unsigned long long *word = &s->h_pinned->stamp;
    AmpWait wait;
    while (wait.spinning())
        if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == stamp) return true;
    for (;;) {
        if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == stamp) return true;
        if (!naps) {
            if (!hip_ok(hipStreamSynchronize(s->ctx->stream), "hipStreamSynchronize")) return false;
        } else {
            const int drained = amp_nap(s, wait);
            if (drained < 0) return false;
            if (drained == 0) continue;
        }
        // the stream is empty: the step has reported
        if (__atomic_load_n(word, __ATOMIC_ACQUIRE) == stamp) return true;
        set_error("a mixed-precision step finished without reporting its state");
        return false;
    }
}

static void amp_free(AmpState *s)
{
    if (s->d_block) (void)hipFree(s->d_block);
    if (s->h_pinned) (void)hipHostFree(s->h_pinned);
    s->magic = 0;
    delete s;
}

int gm_set_amp_check_order(uintptr_t device, int nontemporal, int reverse)
{
    if (device == 0) return -1;
    Context *ctx = resolve_device(device);
    if (!ctx) return -2;
    ctx->amp_check_nontemporal.store(nontemporal < 0 ? 1 : (nontemporal ? 1 : 0));
    ctx->amp_check_reverse.store(reverse < 0 ? 0 : (reverse ? 1 : 0));
    return 0;
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
    bool ok = hip_ok(hipMalloc(&s->d_block, sizeof(AmpDeviceBlock)), "hipMalloc(amp state)") &&
              hip_ok(hipMemsetAsync(s->d_block, 0, sizeof(AmpDeviceBlock), ctx->stream), "hipMemsetAsync(amp state)") &&
              // coherent whatever HIP_HOST_COHERENT says: the host reads stamps while the kernel that wrote them runs
              hip_ok(hipHostMalloc(&s->h_pinned, (kAmpMaxInFlight + 1) * sizeof(AmpDeviceState),
                                   hipHostMallocCoherent), "hipHostMalloc(amp state)");
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

// The next step's stamp (the context lock is held).  64 bits: it does not come round again.
static unsigned long long amp_next_stamp(AmpState *amp)
{
    return ++amp->last_stamp;
}

// The records of the step about to be enqueued: it reads `pre` and writes `post`, which the step
// after it reads (the context lock is held).
static void amp_take_records(AmpState *amp, AmpDeviceState *&pre, AmpDeviceState *&post)
{
    pre = &amp->d_block->slot[amp->slot];
    post = &amp->d_block->slot[amp->slot ^ 1];
    amp->slot ^= 1;
}

static StepParams amp_step_params(float learning_rate, float beta1, float beta2, float epsilon, float weight_decay)
{
    StepParams p = zero_params();
    p.lr = learning_rate;
    p.beta1 = beta1;
    p.beta2 = beta2;
    p.one_minus_beta1 = 1.0f - beta1;
    p.one_minus_beta2 = 1.0f - beta2;
    p.eps = epsilon;
    p.weight_decay = weight_decay;
    return p;
}

// Bias corrections and the pinned slot this step's post-state goes to.  The context lock is held:
// the issue counters of the loss-scale state are only read and advanced under it.  An asynchronous
// step's post-state goes into the ring slot of its issue number, a synchronous step's into slot 0.
static bool amp_bias_and_mirror(AmpState *amp, bool async, float beta1, float beta2, int step_count,
                                AmpBiasTable &bias, AmpDeviceState *&host_mirror)
{
    host_mirror = amp->h_pinned;
    bias = AmpBiasTable{};
    if (async) {
        if (!amp_poll(amp, true)) return false;
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
    return true;
}

static PlanRequest amp_request(uintptr_t *weight_buffers, uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                               uintptr_t *variance_buffers, uintptr_t *weight16_buffers, int num_weights,
                               int *buffer_sizes)
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
    return req;
}

// Plan, parameters and the launches (check, update with the epilogue) shared by the synchronous and the
// asynchronous in-place step.
static int amp_enqueue(uintptr_t device, AmpState *amp, uintptr_t *weight_buffers,
                       uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                       uintptr_t *variance_buffers, uintptr_t *weight16_buffers, int num_weights,
                       int *buffer_sizes, float learning_rate, float beta1, float beta2, float epsilon,
                       float weight_decay, int step_count, bool async, Launch &l,
                       std::unique_lock<std::mutex> &lock)
{
    const PlanRequest req = amp_request(weight_buffers, gradient16_buffers, momentum_buffers, variance_buffers,
                                        weight16_buffers, num_weights, buffer_sizes);
    if (int rc = prepare(device, req, -6, l, lock)) return rc;
    if (l.ctx != amp->ctx) {
        set_error("the loss-scale state belongs to another device context");
        return -16;
    }
    const StepParams p = amp_step_params(learning_rate, beta1, beta2, epsilon, weight_decay);
    const uint32_t chunks = l.plan->num_chunks;
    hipStream_t st = l.ctx->stream;
    int vec = current_vec(l.ctx);
    if (vec == 0) vec = auto_vec(8);
    const bool nt = current_nontemporal(l.ctx);
    int block = current_block(l.ctx);
    if (block == 0) block = auto_block(8);
    SegmentLaunch seg[2];
    int count = 0;
    if (chunks > 0 && !launch_geometry(*l.plan, vec, block, seg, count)) return -6;
    // nothing below fails before the launches: the step takes its stamp and its two records
    AmpDeviceState *host_mirror;
    AmpBiasTable bias;
    if (!amp_bias_and_mirror(amp, async, beta1, beta2, step_count, bias, host_mirror)) return -6;
    const unsigned long long stamp = amp_next_stamp(amp);
    if (async) amp->ring_stamp[(amp->issued + 1) % kAmpMaxInFlight] = stamp;
    AmpDeviceState *pre, *post;
    amp_take_records(amp, pre, post);
    unsigned long long *overflow = &amp->d_block->overflow;

    if (chunks > 0) {
        // the check walks the whole table: one workgroup per chunk of either segment, or several per chunk when
        // the list has few chunks (rows of 2048 elements are not split)
        const int reverse = l.ctx->amp_check_reverse.load();
        uint32_t split_shift = 0;
        {
            uint32_t smallest = 0;
            for (int k = 0; k < l.plan->num_segments; k++)
                if (l.plan->segment[k].num_chunks > 0 &&
                    (smallest == 0 || (uint32_t)l.plan->segment[k].chunk_elements < smallest))
                    smallest = (uint32_t)l.plan->segment[k].chunk_elements;
            while ((chunks << split_shift) < 1024u && (smallest >> (split_shift + 1)) >= 2048u) split_shift++;
        }
        const uint32_t check_grid = chunks << split_shift;
        if (nt && l.ctx->amp_check_nontemporal.load())
            amp_overflow_check_kernel<true><<<check_grid, kBlock, 0, st>>>(l.plan->d_chunks, overflow, reverse, stamp, chunks, split_shift);
        else
            amp_overflow_check_kernel<false><<<check_grid, kBlock, 0, st>>>(l.plan->d_chunks, overflow, reverse, stamp, chunks, split_shift);
        // the first update launch of the step carries the epilogue, so that the host learns the outcome as soon as
        // the check has finished (a second segment's launch reads the same pre-state, which nothing writes)
#define GM_LAUNCH_AMP(V, N, B) amp_adam_update_kernel<V, N, B><<<g.grid, B, 0, st>>>(g.chunks, g.shift, p, pre, overflow, bias, stamp, \
                                                                                 lead ? post : nullptr, lead ? host_mirror : nullptr)
#define GM_LAUNCH_AMP_B(B)                                                              \
        if (vec == 4) { if (nt) GM_LAUNCH_AMP(4, true, B); else GM_LAUNCH_AMP(4, false, B); }        \
        else if (vec == 2) { if (nt) GM_LAUNCH_AMP(2, true, B); else GM_LAUNCH_AMP(2, false, B); }   \
        else { if (nt) GM_LAUNCH_AMP(1, true, B); else GM_LAUNCH_AMP(1, false, B); }
        for (int s = 0; s < count; s++) {
            const SegmentLaunch &g = seg[s];
            const bool lead = s == 0;
            if (block == 128) { GM_LAUNCH_AMP_B(128) } else { GM_LAUNCH_AMP_B(kBlock) }
        }
#undef GM_LAUNCH_AMP_B
#undef GM_LAUNCH_AMP
    } else {
        amp_finalize_kernel<<<1, 64, 0, st>>>(pre, post, host_mirror, overflow, stamp, 0);
    }
    return hip_ok(hipGetLastError(), "mixed-precision kernel launch") ? 0 : -6;
}

// The ping-pong step: one plan per set (identical geometry: same sizes, same planner), one fused
// launch per segment, then the epilogue and the repair pass in one launch.
constexpr unsigned int kRepairGrid = 2048;
static int amp_enqueue_fused(uintptr_t device, AmpState *amp, uintptr_t *const set_a[3], uintptr_t *const set_b[3],
                             uintptr_t *gradient16_buffers, uintptr_t *weight16_buffers, int num_weights,
                             int *buffer_sizes, float learning_rate, float beta1, float beta2, float epsilon,
                             float weight_decay, int step_count, bool async, Launch &l,
                             std::unique_lock<std::mutex> &lock)
{
    for (int k = 0; k < 3; k++) {
        if (num_weights > 0 && (!set_a[k] || !set_b[k])) {
            set_error("both sets of weight, momentum and variance arrays are required");
            return -4;
        }
    }
    const PlanRequest req_a = amp_request(set_a[0], gradient16_buffers, set_a[1], set_a[2], weight16_buffers,
                                          num_weights, buffer_sizes);
    const PlanRequest req_b = amp_request(set_b[0], gradient16_buffers, set_b[1], set_b[2], weight16_buffers,
                                          num_weights, buffer_sizes);
    if (int rc = prepare(device, req_a, -6, l, lock)) return rc;
    if (l.ctx != amp->ctx) {
        set_error("the loss-scale state belongs to another device context");
        return -16;
    }
    MultiTensorPlan *plan_a = l.plan;
    // (the lock is held; the plan just found sits at the front of the cache and cannot be the one
    // pushed out by the second lookup)
    MultiTensorPlan *plan_b = get_plan(l.ctx, req_b);
    if (!plan_b) return -6;
    if (plan_b->status != 0) {
        set_error("a required buffer handle of set B is nil (code %d)", plan_b->status);
        return plan_b->status;
    }
    if (plan_a->num_chunks != plan_b->num_chunks || plan_a->num_segments != plan_b->num_segments ||
        plan_a->segment[0].num_chunks != plan_b->segment[0].num_chunks ||
        plan_a->segment[0].chunk_elements != plan_b->segment[0].chunk_elements ||
        plan_a->segment[1].chunk_elements != plan_b->segment[1].chunk_elements ||
        plan_a->total_elements != plan_b->total_elements || plan_a->kept_signature != plan_b->kept_signature) {
        // only a tensor skipped in one set and not the other (a buffer shorter than its size) gets here: chunk c of
        // set A must be the same tensor and range as chunk c of set B
        set_error("sets A and B do not hold the same tensors (a buffer of one set is shorter than its tensor)");
        return -4;
    }
    const StepParams p = amp_step_params(learning_rate, beta1, beta2, epsilon, weight_decay);
    AmpDeviceState *host_mirror;
    AmpBiasTable bias;
    if (!amp_bias_and_mirror(amp, async, beta1, beta2, step_count, bias, host_mirror)) return -6;
    const unsigned long long stamp = amp_next_stamp(amp);
    if (async) amp->ring_stamp[(amp->issued + 1) % kAmpMaxInFlight] = stamp;
    AmpDeviceState *pre, *post;
    amp_take_records(amp, pre, post);
    unsigned long long *overflow = &amp->d_block->overflow;

    hipStream_t st = l.ctx->stream;
    if (plan_a->num_chunks > 0) {
        int vec = current_vec(l.ctx);
        if (vec == 0) vec = auto_vec(8);
        const bool nt = current_nontemporal(l.ctx);
        int block = current_block(l.ctx);
        if (block == 0) block = auto_block(8);
        SegmentLaunch seg[2];
        int count;
        if (!launch_geometry(*plan_a, vec, block, seg, count)) return -6;
#define GM_LAUNCH_FUSED(V, N, B) \
        amp_adam_fused_kernel<V, N, B><<<g.grid, B, 0, st>>>(pre, g.chunks, plan_b->d_chunks + (g.chunks - plan_a->d_chunks), g.shift, p, bias, stamp, overflow)
#define GM_LAUNCH_FUSED_B(B)                                                              \
        if (vec == 4) { if (nt) GM_LAUNCH_FUSED(4, true, B); else GM_LAUNCH_FUSED(4, false, B); }        \
        else if (vec == 2) { if (nt) GM_LAUNCH_FUSED(2, true, B); else GM_LAUNCH_FUSED(2, false, B); }   \
        else { if (nt) GM_LAUNCH_FUSED(1, true, B); else GM_LAUNCH_FUSED(1, false, B); }
        for (int s = 0; s < count; s++) {
            const SegmentLaunch &g = seg[s];
            if (block == 128) { GM_LAUNCH_FUSED_B(128) } else { GM_LAUNCH_FUSED_B(kBlock) }
        }
#undef GM_LAUNCH_FUSED_B
#undef GM_LAUNCH_FUSED
    }
    // without an fp16 copy there is nothing to repair: one workgroup, for the epilogue alone
    const bool repair = plan_a->num_chunks > 0 && weight16_buffers;
    const unsigned int grid = !repair ? 1u : (plan_a->num_chunks < kRepairGrid ? plan_a->num_chunks : kRepairGrid);
    amp_finalize_repair_kernel<<<grid, kBlock, 0, st>>>(pre, post, host_mirror, overflow, stamp, plan_a->d_chunks,
                                                       plan_b->d_chunks, repair ? plan_a->num_chunks : 0u);
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
    // returns once the step's outcome is known; its update launch may still be running, and
    // everything that reads its results is ordered behind it on the library's stream
    if (!amp_wait_outcome(amp, amp->last_stamp, true)) return -6;
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
    amp->issued += 1;       // its post-state will arrive in the ring slot of this issue number, stamp last
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

int gm_amp_state_current_set(uintptr_t amp_state)
try {
    AmpState *s = amp_from_handle(amp_state);
    if (!s) return -16;
    if (!make_current(s->ctx)) return -6;
    std::lock_guard<std::mutex> lk(s->ctx->mu);
    if (!amp_download(s)) return -6;
    return s->h_pinned->current_set;
} catch (...) {
    note_exception();
    return -6;
}

int gm_amp_state_set_current_set(uintptr_t amp_state, int current_set)
try {
    AmpState *s = amp_from_handle(amp_state);
    if (!s) return -16;
    if (current_set != 0 && current_set != 1) return -5;
    if (!make_current(s->ctx)) return -6;
    std::lock_guard<std::mutex> lk(s->ctx->mu);
    if (!amp_download(s)) return -6;
    s->h_pinned->current_set = current_set;
    return amp_upload(s) ? 0 : -6;
} catch (...) {
    note_exception();
    return -6;
}

int execute_adam_amp_step_fused(uintptr_t device, uintptr_t *weight_a, uintptr_t *momentum_a, uintptr_t *variance_a,
                                uintptr_t *weight_b, uintptr_t *momentum_b, uintptr_t *variance_b,
                                uintptr_t *gradient16_buffers, uintptr_t *weight16_buffers, int num_weights,
                                int *buffer_sizes, float learning_rate, float beta1, float beta2, float epsilon,
                                float weight_decay, int step_count, uintptr_t amp_state, int *skipped,
                                float *scale_out, int *growth_tracker_out, int *current_set_out)
try {
    if (device == 0) return -1;
    AmpState *amp = amp_from_handle(amp_state);
    if (!amp) return -16;
    Launch l{};
    std::unique_lock<std::mutex> lock;
    uintptr_t *const a[3] = {weight_a, momentum_a, variance_a};
    uintptr_t *const b[3] = {weight_b, momentum_b, variance_b};
    if (int rc = amp_enqueue_fused(device, amp, a, b, gradient16_buffers, weight16_buffers, num_weights, buffer_sizes,
                                   learning_rate, beta1, beta2, epsilon, weight_decay, step_count, false, l, lock))
        return rc;
    if (!amp_wait_outcome(amp, amp->last_stamp, false)) return -6;
    amp->confirmed_issue = amp->issued;
    amp->confirmed_applied = amp->h_pinned->applied_steps;
    if (skipped) *skipped = amp->h_pinned->last_skipped;
    if (scale_out) *scale_out = amp->h_pinned->scale;
    if (growth_tracker_out) *growth_tracker_out = amp->h_pinned->growth_tracker;
    if (current_set_out) *current_set_out = amp->h_pinned->current_set;
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

int execute_adam_amp_step_fused_async(uintptr_t device, uintptr_t *weight_a, uintptr_t *momentum_a,
                                      uintptr_t *variance_a, uintptr_t *weight_b, uintptr_t *momentum_b,
                                      uintptr_t *variance_b, uintptr_t *gradient16_buffers,
                                      uintptr_t *weight16_buffers, int num_weights, int *buffer_sizes,
                                      float learning_rate, float beta1, float beta2, float epsilon,
                                      float weight_decay, uintptr_t amp_state)
try {
    if (device == 0) return -1;
    AmpState *amp = amp_from_handle(amp_state);
    if (!amp) return -16;
    Launch l{};
    std::unique_lock<std::mutex> lock;
    uintptr_t *const a[3] = {weight_a, momentum_a, variance_a};
    uintptr_t *const b[3] = {weight_b, momentum_b, variance_b};
    if (int rc = amp_enqueue_fused(device, amp, a, b, gradient16_buffers, weight16_buffers, num_weights, buffer_sizes,
                                   learning_rate, beta1, beta2, epsilon, weight_decay, 0, true, l, lock))
        return rc;
    amp->issued += 1;
    return 0;
} catch (...) {
    note_exception();
    return -6;
}

}  // extern "C"
