// L-BFGS step for gfx950: the HIP counterpart of execute_lbfgs_step_mpsgraph
// (cgo_bridge/bridge_optimizer.m:980-1321), which the reference runs as CPU
// loops over unified-memory buffers.
//
// The step is a fixed sequence of streaming launches over the whole tensor list
// on one stream.  Every element-wise statement of the reference is one fused
// pass; every dot product is accumulated by the pass that produces its operand,
// so a history pair costs two passes, not four:
//
//   prologue     gather rho[idx(j)], mark pairs with |rho| < 1e-10 invalid, alpha[j] = 0 for them
//   init         dot(s_j, q), q = -g, for the newest valid pair (q stays in registers)
//   backward     q -= alpha_j y_j             (+ dot with the next operand; the first one reads g for q)
//   forward      r += (alpha_j - beta) s_j    (+ dot with the next operand)
//   update       p = -r; x += a p; old_g = g; s_cur = a p; y_prev = g - old_g; rho_prev = 0
//
// The last line is the reference's curvature update as its own order of statements makes it
// come out.  It copies g into old_g (bridge_optimizer.m:1236-1239) before it forms
// y_prev = g - old_g (:1285-1288), so every element of y_prev is g - g: +0, or NaN for a
// non-finite g.  s_prev . y_prev is then a sum of zeros and NaNs, |s.y| > 1e-10 is false either
// way, and rho_prev = 0 (:1304-1310), whatever s_prev holds.  The update pass therefore writes
// y_prev = g - g from the gradient it already holds and rho_prev is set to 0 without reading
// s_prev or summing anything: the same bits as the reference's loop nest, 12 bytes per element
// less traffic than a curvature pass of its own (read g, old_g, s_prev; write y_prev), 4 less
// than a real dot product riding on the update pass.
//
// Which pairs are valid is read back once per step (history_count flags), so
// only the passes that do work are launched; with the history the reference's
// own optimizer produces (every rho it writes is 0) a step is the update pass alone.
//
// Dot products: exact fp64 products, summed in fp64 by a fixed radix-1024 tree
// (lane l of a 256-lane workgroup adds elements l, l+256, l+512, l+768 of a
// 1024-element slice in that order; lanes are combined by an adjacent-pair
// binary tree; slice sums are reduced by the same node, 1024 at a time, until
// one value is left) and rounded once to fp32.  The order is fixed by the data
// layout alone, so results are bit-reproducible and independent of the launch
// geometry.  The reference's running fp32 sum is inherently serial; this tree
// lies within that sum's own rounding-error bound of it.
#include "gm_context.hpp"

#include "../../include/gometal_hip.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <memory>
#include <vector>

namespace gm {

bool current_nontemporal(const Context *ctx);   // gm_plan_cache.hip

namespace {

constexpr int kLanes = 256;
constexpr int kPerLane = 4;
constexpr int kSlice = kLanes * kPerLane;            // 1024: the tree's radix and the slice length
constexpr int kChunkCandidates[] = {65536, 16384, 4096, 1024};
constexpr double kMaxIdleFraction = 0.05;
constexpr int kFusedReduceMaxGroups = 128;

struct alignas(16) LbChunk {
    uint32_t tensor;        // index into the handle rows
    uint32_t count;         // elements in this chunk
    uint32_t offset;        // first element, relative to the tensor
    uint32_t first_slice;   // ordinal of the chunk's first slice in the list-wide slice numbering
};

struct LbScalars {
    float coef;             // coefficient of the next axpy pass, written by a reduction epilogue
    float dot;              // last dot product, rounded to fp32
};

enum : int { kOpNone = 0, kOpAlpha, kOpBeta, kOpRho, kOpStore };

struct Epilogue {
    int op;
    const float *rho;       // rho of the pair (kOpAlpha, kOpBeta)
    float *alpha;           // &alpha[j] (kOpAlpha writes, kOpBeta reads)
    float *rho_out;         // kOpRho
    LbScalars *scalars;
};

struct Plan {
    // key
    std::vector<int> sizes;
    // geometry
    LbChunk *d_chunks = nullptr;
    uint32_t num_chunks = 0;
    uint32_t slice_shift = 0;          // log2(slices per chunk)
    uint64_t total_slices = 0;
    // handle rows: weights, gradients, old gradients, direction, s[h], y[h] (n each), then rho[h]
    int history_size = 0;
    std::vector<uintptr_t> handles;
    uintptr_t alpha_handle = 0;
    uintptr_t *d_handles = nullptr;
    size_t handles_capacity = 0;
    bool handles_valid = false;
    // scratch
    double *d_partial[2] = {nullptr, nullptr};
    LbScalars *d_scalars = nullptr;
    unsigned int *d_ticket = nullptr;  // workgroup counter of the fused reduction, zero between launches
    int *h_valid = nullptr;            // pinned host memory, written by the prologue kernel
    int valid_capacity = 0;

    ~Plan()
    {
        if (d_chunks) (void)hipFree(d_chunks);
        if (d_handles) (void)hipFree(d_handles);
        if (d_partial[0]) (void)hipFree(d_partial[0]);
        if (d_partial[1]) (void)hipFree(d_partial[1]);
        if (d_scalars) (void)hipFree(d_scalars);
        if (d_ticket) (void)hipFree(d_ticket);
        if (h_valid) (void)hipHostFree(h_valid);
    }
};

constexpr size_t kMaxPlans = 4;
// Never destroyed: plans own device memory, and static destructors may run after the HIP
// runtime has shut down.
std::vector<std::unique_ptr<Plan>> &plan_cache()
{
    static auto *cache = new std::vector<std::unique_ptr<Plan>>();
    return *cache;
}

int choose_chunk(const int *sizes, int n)
{
    for (int candidate : kChunkCandidates) {
        const uint64_t per_chunk = (uint64_t)candidate / kSlice;
        uint64_t working = 0, launched = 0;
        for (int i = 0; i < n; i++) {
            const uint64_t numel = sizes[i] > 0 ? (uint64_t)sizes[i] / sizeof(float) : 0;
            working += (numel + kSlice - 1) / kSlice;
            launched += (numel + candidate - 1) / candidate * per_chunk;
        }
        if (launched - working <= (uint64_t)(kMaxIdleFraction * (double)working)) return candidate;
    }
    return kSlice;
}

// ---------------------------------------------------------------- kernels ----
#define GM_GLOBAL __attribute__((address_space(1)))

template <bool NT>
__device__ inline float ld(const float *p)
{
    const GM_GLOBAL float *gp = (const GM_GLOBAL float *)p;
    if (NT) return __builtin_nontemporal_load(gp);
    return *gp;
}

template <bool NT>
__device__ inline void st(float v, float *p)
{
    GM_GLOBAL float *gp = (GM_GLOBAL float *)p;
    if (NT) __builtin_nontemporal_store(v, gp);
    else *gp = v;
}

// Adjacent-pair binary tree over the 256 lane values of a workgroup; the result is valid in
// thread 0.  The xor butterfly gives every lane of a pair the same sum (IEEE addition is
// commutative), so after the step with distance d every lane holds the sum of its aligned
// group of 2d lanes: exactly the adjacent-pair tree.
__device__ inline double workgroup_tree(double v)
{
    __shared__ double wave_sum[kLanes / 64];
#pragma unroll
    for (int d = 1; d < 64; d *= 2) v = v + __shfl_xor(v, d, 64);
    if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = v;
    __syncthreads();
    return (wave_sum[0] + wave_sum[1]) + (wave_sum[2] + wave_sum[3]);
}

enum : int { kModeAxpy = 0, kModeAxpyFirst };

struct StreamArgs {
    const LbChunk *chunks;
    uint32_t slice_shift;
    // rows of the handle table (one device address per tensor); meaning depends on the mode
    const uintptr_t *r0, *r1, *r2, *r3;
    double *partial;               // slice sums (modes with a dot product)
    const LbScalars *scalars;      // coefficient for kModeAxpy
    int subtract;                  // kModeAxpy: x - c v (backward loop) or x + c v (forward loop)
};

// One workgroup = one 1024-element slice: lane l handles elements l, l+256, l+512, l+768.
//   kModeAxpyFirst       r0 = g, r1 = v, r2 = dot operand, r3 = direction    x = (-g) - c v, stored as the direction
//   kModeAxpy            r0 = direction, r1 = v, r2 = dot operand        x = x -/+ c v
// The recursion starts from q = -g.  Nothing but its first axpy reads that q, so it is formed in
// registers twice (for the first dot product, lbfgs_dot_kernel, and by the first axpy, which reads
// g instead of the direction buffer) rather than written out and read back: 4 bytes per element
// less.
template <int MODE, bool DOT, bool NT>
__global__ void __launch_bounds__(kLanes) lbfgs_stream_kernel(StreamArgs a)
{
    const LbChunk ch = a.chunks[blockIdx.x >> a.slice_shift];
    const uint32_t slice = blockIdx.x & ((1u << a.slice_shift) - 1u);
    const uint32_t base = slice * kSlice;
    if (base >= ch.count) return;                       // the whole workgroup leaves together
    const uint32_t left = ch.count - base;
    const size_t first = (size_t)ch.offset + base + threadIdx.x;

    float *p0 = reinterpret_cast<float *>(a.r0[ch.tensor]) + first;
    float *p1 = reinterpret_cast<float *>(a.r1[ch.tensor]) + first;
    float *p2 = nullptr;
    constexpr bool kFusedDot = DOT;                                           // r2 = dot operand
    if (kFusedDot) p2 = reinterpret_cast<float *>(a.r2[ch.tensor]) + first;
    float *out = p0;                                                          // where an axpy stores x
    if (MODE == kModeAxpyFirst) out = reinterpret_cast<float *>(a.r3[ch.tensor]) + first;

    const float coef = a.scalars->coef;

    // Order of a lane's memory operations: element by element, all loads of the element, then
    // its store.  The compiler cannot prove that the streams do not overlap, so a store orders
    // the loads around it; a store placed between two loads of one element leaves a single load
    // in flight per lane (a pass ran at 53 % of peak that way, 75 % with loads first).
    // Hoisting the loads of all four elements above the first store is slower for the passes
    // that feed a dot product (68 % against 86 % of peak): reads and writes then reach the
    // memory controllers in bursts instead of finely interleaved.
    float v0[kPerLane], v1[kPerLane], v2[kPerLane];
    auto load_element = [&](int u) {
        const size_t o = (size_t)u * kLanes;
        const bool ok = threadIdx.x + u * kLanes < left;
        v0[u] = ok ? ld<NT>(p0 + o) : 0.0f;
        v1[u] = ok ? ld<NT>(p1 + o) : 0.0f;
        v2[u] = (kFusedDot && ok) ? ld<NT>(p2 + o) : 0.0f;
    };
    // arithmetic, stores, and the lane's running fp64 sum in element order
    double acc = 0.0;
#pragma unroll
    for (int u = 0; u < kPerLane; u++) {
        load_element(u);
        if (threadIdx.x + u * kLanes >= left) continue;
        const size_t o = (size_t)u * kLanes;
        const float from = MODE == kModeAxpyFirst ? -v0[u] : v0[u];
        const float cv = coef * v1[u];
        const float x = a.subtract ? from - cv : from + cv;
        const float d = v2[u];
        st<NT>(x, out + o);
        if (DOT) acc = acc + (double)d * (double)x;     // exact product, one fp64 rounding per addition
    }
    if (DOT) {
        const double total = workgroup_tree(acc);
        if (threadIdx.x == 0) a.partial[ch.first_slice + slice] = total;
    }
}

// The passes that only read (dot(s, -g) at the head of the recursion, gm_lbfgs_dot): the same sum
// as lbfgs_stream_kernel forms, with the memory side reshaped.  Nothing is stored, so what limits
// a pure read is the bytes each wave keeps in flight: lane l loads elements 4 l .. 4 l + 3 of the
// slice with one 16-byte load per operand, the four exact fp64 products go to LDS at their element
// positions, and after a barrier lane l adds products l, l + 256, l + 512, l + 768 in that order:
// the lane sum of the tree.  Slices that are ragged or not 16-byte aligned take 4-byte loads in
// the tree's own lane order.  Measured on MI355X over 1B parameters: 8 B/param in 1.61 ms (63 % of
// peak) with 4-byte loads throughout.
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <bool NEGATE, bool NT>
__global__ void __launch_bounds__(kLanes) lbfgs_dot_kernel(StreamArgs a)
{
    __shared__ double product[kSlice];
    const LbChunk ch = a.chunks[blockIdx.x >> a.slice_shift];
    const uint32_t slice = blockIdx.x & ((1u << a.slice_shift) - 1u);
    const uint32_t base = slice * kSlice;
    if (base >= ch.count) return;
    const uint32_t left = ch.count - base;
    const float *pa = reinterpret_cast<const float *>(a.r0[ch.tensor]) + ch.offset + base;
    const float *pb = reinterpret_cast<const float *>(a.r1[ch.tensor]) + ch.offset + base;
    double acc = 0.0;
    const bool wide = left >= (uint32_t)kSlice &&
                      ((reinterpret_cast<uintptr_t>(pa) | reinterpret_cast<uintptr_t>(pb)) & 15u) == 0;
    if (wide) {                                        // uniform over the workgroup
        const GM_GLOBAL floatx4 *ga = (const GM_GLOBAL floatx4 *)pa + threadIdx.x;
        const GM_GLOBAL floatx4 *gb = (const GM_GLOBAL floatx4 *)pb + threadIdx.x;
        const floatx4 x = NT ? __builtin_nontemporal_load(ga) : *ga;
        const floatx4 d = NT ? __builtin_nontemporal_load(gb) : *gb;
#pragma unroll
        for (int c = 0; c < 4; c++) {
            const float xv = NEGATE ? -x[c] : x[c];
            product[4 * threadIdx.x + c] = (double)d[c] * (double)xv;
        }
        __syncthreads();
#pragma unroll
        for (int u = 0; u < kPerLane; u++) acc = acc + product[threadIdx.x + u * kLanes];
    } else {
#pragma unroll
        for (int u = 0; u < kPerLane; u++) {
            const uint32_t i = threadIdx.x + u * kLanes;
            if (i >= left) continue;
            const float x0 = ld<NT>(pa + i);
            const float xv = NEGATE ? -x0 : x0;
            acc = acc + (double)ld<NT>(pb + i) * (double)xv;
        }
    }
    const double total = workgroup_tree(acc);
    if (threadIdx.x == 0) a.partial[ch.first_slice + slice] = total;
}

// The update pass: p = -r; x += a p; old_g = g; s_cur = a p; and, when the history is not empty,
// y_prev = g - old_g with old_g = g as just stored (+0, or NaN for a non-finite g).  It feeds no
// dot product, so it is free of the 1024-element slices of the summation tree: one element per
// lane, a workgroup per 256 elements.  Five of its seven or eight streams are written, and the
// write-heavy mix is the one that suffers most from long-lived workgroups: measured on MI355X over
// 2^29 elements, 81 % of peak HBM bandwidth in this shape against 70 % with four strided elements
// per lane (the shape of the passes above), 73-74 % with 8-byte lanes and 68-71 % with 16-byte lanes.
struct UpdateArgs {
    const LbChunk *chunks;
    uint32_t quarter_shift;        // log2(256-element workgroups per chunk)
    const uintptr_t *dir, *w, *g, *old_g, *s_cur, *y_prev;
    float step;
};

template <bool FROM_GRADIENT, bool WITH_Y, bool NT>
__global__ void __launch_bounds__(kLanes) lbfgs_update_kernel(UpdateArgs a)
{
    const LbChunk ch = a.chunks[blockIdx.x >> a.quarter_shift];
    const uint32_t local = (blockIdx.x & ((1u << a.quarter_shift) - 1u)) * kLanes + threadIdx.x;
    if (local >= ch.count) return;
    const size_t i = (size_t)ch.offset + local;
    float *dir = reinterpret_cast<float *>(a.dir[ch.tensor]) + i;
    float *w = reinterpret_cast<float *>(a.w[ch.tensor]) + i;
    const float g = ld<NT>(reinterpret_cast<const float *>(a.g[ch.tensor]) + i);
    const float x = ld<NT>(w);
    // r = -g when no pair is valid this step (formed in registers), else what the recursion left
    const float r = FROM_GRADIENT ? -g : ld<NT>(dir);
    const float p = -r;
    const float sp = a.step * p;
    st<NT>(p, dir);
    st<NT>(x + sp, w);
    st<NT>(g, reinterpret_cast<float *>(a.old_g[ch.tensor]) + i);
    st<NT>(sp, reinterpret_cast<float *>(a.s_cur[ch.tensor]) + i);
    if (WITH_Y) st<NT>(g - g, reinterpret_cast<float *>(a.y_prev[ch.tensor]) + i);
}

__device__ inline void run_epilogue(const Epilogue &e, double total)
{
    const float d = (float)total;
    e.scalars->dot = d;
    if (e.op == kOpAlpha) {
        const float v = d * *e.rho;          // alpha_j = rho_j (s_j . q)
        *e.alpha = v;
        e.scalars->coef = v;
    } else if (e.op == kOpBeta) {
        const float beta = d * *e.rho;       // beta = rho_j (y_j . r)
        e.scalars->coef = *e.alpha - beta;
    } else if (e.op == kOpRho) {
        *e.rho_out = fabs((double)d) > 1e-10 ? 1.0f / d : 0.0f;
    }
}

// One tree level: workgroup b reduces src[1024 b .. 1024 b + 1023] to dst[b].  The launch with
// a single workgroup is the last one and runs the scalar epilogue.
__global__ void __launch_bounds__(kLanes) lbfgs_reduce_kernel(const double *__restrict__ src, uint64_t count,
                                                             double *__restrict__ dst, Epilogue e)
{
    const uint64_t base = (uint64_t)blockIdx.x * kSlice;
    const uint64_t left = count - base;
    double acc = 0.0;
#pragma unroll
    for (int u = 0; u < kPerLane; u++) {
        const uint32_t i = threadIdx.x + u * kLanes;
        if (i < left) acc = acc + src[base + i];
    }
    const double total = workgroup_tree(acc);
    if (threadIdx.x != 0) return;
    dst[blockIdx.x] = total;
    if (gridDim.x == 1 && e.op != kOpNone) run_epilogue(e, total);
}

// The last two tree levels in one launch (2 .. kFusedReduceMaxGroups workgroups): every workgroup reduces its
// group to dst[b], publishes it and takes a ticket; the workgroup that draws the last ticket
// reduces dst[0 .. gridDim.x) with the same node and runs the scalar epilogue.  The order of
// the additions is that of two separate launches; only a 5 us launch is saved per dot product.
// Each workgroup's release makes its result visible device-wide, which costs a cache write-back:
// with 24 workgroups (25M parameters) the launch takes 5 us against 9 for two launches, with 966
// (1B parameters) it took 24 us, so lists with more groups use two plain launches.
__global__ void __launch_bounds__(kLanes) lbfgs_reduce_last_two_kernel(const double *__restrict__ src,
                                                                      uint64_t count, double *dst,
                                                                      unsigned int *ticket, Epilogue e)
{
    __shared__ bool is_last;
    const uint64_t base = (uint64_t)blockIdx.x * kSlice;
    const uint64_t left = count - base;
    double acc = 0.0;
#pragma unroll
    for (int u = 0; u < kPerLane; u++) {
        const uint32_t i = threadIdx.x + u * kLanes;
        if (i < left) acc = acc + src[base + i];
    }
    const double mine = workgroup_tree(acc);
    if (threadIdx.x == 0) {
        __hip_atomic_store(&dst[blockIdx.x], mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // release dst[b] to the device, acquire what the earlier ticket holders released
        const unsigned int drawn = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        is_last = drawn == gridDim.x - 1;
    }
    __syncthreads();      // also separates the two uses of workgroup_tree's shared words
    if (!is_last) return;
    double acc2 = 0.0;
#pragma unroll
    for (int u = 0; u < kPerLane; u++) {
        const uint32_t i = threadIdx.x + u * kLanes;
        if (i < gridDim.x) acc2 = acc2 + __hip_atomic_load(&dst[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const double total = workgroup_tree(acc2);
    if (threadIdx.x != 0) return;
    __hip_atomic_store(&dst[0], total, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);     // ready for the next launch
    if (e.op != kOpNone) run_epilogue(e, total);
}

// A list with zero or one slice has no tree level to run: the epilogue takes the value as is.
__global__ void lbfgs_epilogue_kernel(const double *src, uint64_t count, Epilogue e)
{
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    run_epilogue(e, count == 0 ? 0.0 : src[0]);
}

// rho of pair j of the recursion (slot idx(j) of the ring), validity flags, alpha[j] = 0 for
// invalid pairs (bridge_optimizer.m:1067-1070).
__global__ void lbfgs_prologue_kernel(const uintptr_t *rho_handles, int history_size, int history_count,
                                      int history_index, float *alpha, int *valid)
{
    for (int j = threadIdx.x; j < history_count; j += blockDim.x) {
        const int idx = (history_index - history_count + j + history_size) % history_size;
        const float rho = *reinterpret_cast<const float *>(rho_handles[idx]);
        const int ok = !(fabs((double)rho) < 1e-10);
        valid[j] = ok;
        if (!ok) alpha[j] = 0.0f;
    }
}

// ------------------------------------------------------------------- host ----
struct Rows {
    const uintptr_t *w, *g, *old_g, *dir, *rho;
    const uintptr_t *s(int h, int n) const { return s0 + (size_t)h * n; }
    const uintptr_t *y(int h, int n) const { return y0 + (size_t)h * n; }
    const uintptr_t *s0, *y0;
};

Rows rows_of(const uintptr_t *base, int n, int m)
{
    Rows r;
    r.w = base;
    r.g = base + (size_t)n;
    r.old_g = base + (size_t)2 * n;
    r.dir = base + (size_t)3 * n;
    r.s0 = base + (size_t)4 * n;
    r.y0 = r.s0 + (size_t)m * n;
    r.rho = r.y0 + (size_t)m * n;
    return r;
}

bool ensure_geometry(Context *ctx, Plan &p, const int *sizes, int n)
{
    const int chunk = choose_chunk(sizes, n);
    std::vector<LbChunk> chunks;
    uint64_t slice = 0;
    for (int i = 0; i < n; i++) {
        const size_t numel = sizes[i] > 0 ? (size_t)sizes[i] / sizeof(float) : 0;
        for (size_t off = 0; off < numel; off += (size_t)chunk) {
            const size_t left = numel - off;
            LbChunk c;
            c.tensor = (uint32_t)i;
            c.count = (uint32_t)(left < (size_t)chunk ? left : (size_t)chunk);
            c.offset = (uint32_t)off;
            c.first_slice = (uint32_t)slice;
            slice += (c.count + kSlice - 1) / kSlice;
            chunks.push_back(c);
        }
    }
    p.slice_shift = 0;
    while ((1u << p.slice_shift) < (uint32_t)(chunk / kSlice)) p.slice_shift++;
    if (slice > 0xFFFFFFFFull || ((uint64_t)chunks.size() << (p.slice_shift + 2)) > 0x7FFFFFFFull) {
        set_error("tensor list too large for one launch");
        return false;
    }
    p.total_slices = slice;
    p.num_chunks = (uint32_t)chunks.size();
    p.sizes.assign(sizes, sizes + n);
    if (!chunks.empty()) {
        if (!hip_ok(hipMalloc(&p.d_chunks, chunks.size() * sizeof(LbChunk)), "hipMalloc(lbfgs chunks)") ||
            !hip_ok(hipMemcpyAsync(p.d_chunks, chunks.data(), chunks.size() * sizeof(LbChunk),
                                   hipMemcpyHostToDevice, ctx->stream), "upload lbfgs chunks") ||
            !hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))
            return false;
    }
    const size_t level0 = (size_t)std::max<uint64_t>(slice, 1);
    const size_t level1 = (level0 + kSlice - 1) / kSlice;
    return hip_ok(hipMalloc(&p.d_partial[0], level0 * sizeof(double)), "hipMalloc(lbfgs partial sums)") &&
           hip_ok(hipMalloc(&p.d_partial[1], level1 * sizeof(double)), "hipMalloc(lbfgs partial sums)") &&
           hip_ok(hipMalloc(&p.d_scalars, sizeof(LbScalars)), "hipMalloc(lbfgs scalars)") &&
           hip_ok(hipMemsetAsync(p.d_scalars, 0, sizeof(LbScalars), ctx->stream), "clear lbfgs scalars") &&
           hip_ok(hipMalloc(&p.d_ticket, sizeof(unsigned int)), "hipMalloc(lbfgs ticket)") &&
           hip_ok(hipMemsetAsync(p.d_ticket, 0, sizeof(unsigned int), ctx->stream), "clear lbfgs ticket");
}

Plan *find_plan(Context *ctx, const int *sizes, int n)
{
    auto &cache = plan_cache();
    for (size_t i = 0; i < cache.size(); i++) {
        Plan &p = *cache[i];
        if ((int)p.sizes.size() == n && std::memcmp(p.sizes.data(), sizes, (size_t)n * sizeof(int)) == 0) {
            if (i != 0) std::rotate(cache.begin(), cache.begin() + i, cache.begin() + i + 1);
            return cache[0].get();
        }
    }
    auto plan = std::make_unique<Plan>();
    if (!ensure_geometry(ctx, *plan, sizes, n)) return nullptr;
    if (cache.size() >= kMaxPlans) {
        (void)hipStreamSynchronize(ctx->stream);    // an evicted plan's scratch may still be in use
        cache.pop_back();
    }
    cache.insert(cache.begin(), std::move(plan));
    return cache[0].get();
}

// Flattens the caller's handle arrays, validates them on change and uploads the table.
// Returns 0 or the entry point's error code.
int stage_handles(Context *ctx, Plan &p, int n, int m, const uintptr_t *w, const uintptr_t *g,
                  const uintptr_t *old_g, const uintptr_t *dir, const uintptr_t *s, const uintptr_t *y,
                  const uintptr_t *rho, uintptr_t alpha)
{
    const size_t total = (size_t)(4 + 2 * m) * n + (size_t)m;
    std::vector<uintptr_t> flat(total);
    Rows r = rows_of(flat.data(), n, m);
    const size_t row = (size_t)n * sizeof(uintptr_t);
    std::memcpy(const_cast<uintptr_t *>(r.w), w, row);
    std::memcpy(const_cast<uintptr_t *>(r.g), g, row);
    std::memcpy(const_cast<uintptr_t *>(r.old_g), old_g, row);
    std::memcpy(const_cast<uintptr_t *>(r.dir), dir, row);
    std::memcpy(const_cast<uintptr_t *>(r.s0), s, row * m);
    std::memcpy(const_cast<uintptr_t *>(r.y0), y, row * m);
    std::memcpy(const_cast<uintptr_t *>(r.rho), rho, (size_t)m * sizeof(uintptr_t));
    if (p.handles_valid && p.history_size == m && p.alpha_handle == alpha && p.handles == flat) return 0;

    for (int i = 0; i < n; i++) {
        const size_t need = p.sizes[i] > 0 ? (size_t)p.sizes[i] / sizeof(float) * sizeof(float) : 0;
        for (int k = 0; k < 4 + 2 * m; k++) {
            const uintptr_t h = flat[(size_t)k * n + i];
            if (h == 0) {
                set_error("L-BFGS buffer handle is nil (array %d, tensor %d)", k, i);
                return -8;
            }
            const size_t have = registry_length(h);
            if (have != 0 && have < need) {
                set_error("L-BFGS buffer shorter than its tensor (array %d, tensor %d)", k, i);
                return -8;
            }
        }
    }
    for (int h = 0; h < m; h++) {
        if (r.rho[h] == 0) {
            set_error("L-BFGS rho buffer %d is nil", h);
            return -8;
        }
    }
    const size_t alpha_len = registry_length(alpha);
    if (alpha == 0 || (alpha_len != 0 && alpha_len < (size_t)m * sizeof(float))) {
        set_error("L-BFGS alpha buffer is nil or shorter than history_size floats");
        return -8;
    }

    if (p.handles_capacity < total) {
        if (!hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize")) return -8;
        if (p.d_handles) (void)hipFree(p.d_handles);
        p.d_handles = nullptr;
        p.handles_capacity = 0;
        if (!hip_ok(hipMalloc(&p.d_handles, total * sizeof(uintptr_t)), "hipMalloc(lbfgs handles)")) return -8;
        p.handles_capacity = total;
    }
    if (p.valid_capacity < m) {
        if (!hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize")) return -8;
        if (p.h_valid) (void)hipHostFree(p.h_valid);
        p.h_valid = nullptr;
        p.valid_capacity = 0;
        if (!hip_ok(hipHostMalloc(&p.h_valid, (size_t)m * sizeof(int), hipHostMallocDefault),
                    "hipHostMalloc(lbfgs flags)"))
            return -8;
        p.valid_capacity = m;
    }
    // The staging vector dies with this call, so the upload is waited for.
    if (!hip_ok(hipMemcpyAsync(p.d_handles, flat.data(), total * sizeof(uintptr_t), hipMemcpyHostToDevice,
                               ctx->stream), "upload lbfgs handles") ||
        !hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize"))
        return -8;
    p.handles = std::move(flat);
    p.history_size = m;
    p.alpha_handle = alpha;
    p.handles_valid = true;
    return 0;
}

// dot(b, a) or dot(b, -a): a.r0 = a rows, a.r1 = b rows
void launch_dot(Context *ctx, const Plan &p, StreamArgs a, bool negate)
{
    if (p.num_chunks == 0) return;
    const uint32_t grid = p.num_chunks << p.slice_shift;
    a.chunks = p.d_chunks;
    a.slice_shift = p.slice_shift;
    const bool nt = current_nontemporal(ctx);
    if (negate) {
        if (nt) lbfgs_dot_kernel<true, true><<<grid, kLanes, 0, ctx->stream>>>(a);
        else lbfgs_dot_kernel<true, false><<<grid, kLanes, 0, ctx->stream>>>(a);
    } else {
        if (nt) lbfgs_dot_kernel<false, true><<<grid, kLanes, 0, ctx->stream>>>(a);
        else lbfgs_dot_kernel<false, false><<<grid, kLanes, 0, ctx->stream>>>(a);
    }
}

template <int MODE, bool DOT>
void launch_stream(Context *ctx, const Plan &p, StreamArgs a)
{
    if (p.num_chunks == 0) return;
    const uint32_t grid = p.num_chunks << p.slice_shift;
    a.chunks = p.d_chunks;
    a.slice_shift = p.slice_shift;
    if (current_nontemporal(ctx)) lbfgs_stream_kernel<MODE, DOT, true><<<grid, kLanes, 0, ctx->stream>>>(a);
    else lbfgs_stream_kernel<MODE, DOT, false><<<grid, kLanes, 0, ctx->stream>>>(a);
}

void launch_update(Context *ctx, const Plan &p, UpdateArgs a, bool from_gradient, bool with_y)
{
    if (p.num_chunks == 0) return;
    a.chunks = p.d_chunks;
    a.quarter_shift = p.slice_shift + 2;      // four 256-element workgroups to a 1024-element slice
    const uint32_t grid = p.num_chunks << a.quarter_shift;
    const bool nt = current_nontemporal(ctx);
    hipStream_t st = ctx->stream;
#define GM_LAUNCH_UPDATE(F, Y)                                                        \
    do {                                                                              \
        if (nt) lbfgs_update_kernel<F, Y, true><<<grid, kLanes, 0, st>>>(a);         \
        else lbfgs_update_kernel<F, Y, false><<<grid, kLanes, 0, st>>>(a);           \
    } while (0)
    if (from_gradient) { if (with_y) GM_LAUNCH_UPDATE(true, true); else GM_LAUNCH_UPDATE(true, false); }
    else { if (with_y) GM_LAUNCH_UPDATE(false, true); else GM_LAUNCH_UPDATE(false, false); }
#undef GM_LAUNCH_UPDATE
}

// Upper tree levels over the slice sums in d_partial[0], then the scalar epilogue.
void launch_reduction(Context *ctx, const Plan &p, const Epilogue &e)
{
    uint64_t count = p.total_slices;
    if (count <= 1) {
        lbfgs_epilogue_kernel<<<1, 64, 0, ctx->stream>>>(p.d_partial[0], count, e);
        return;
    }
    int src = 0;
    const Epilogue none{kOpNone, nullptr, nullptr, nullptr, nullptr};
    while (count > 1) {
        const uint64_t next = (count + kSlice - 1) / kSlice;
        if (next > 1 && next <= (uint64_t)kFusedReduceMaxGroups) {
            lbfgs_reduce_last_two_kernel<<<(uint32_t)next, kLanes, 0, ctx->stream>>>(
                p.d_partial[src], count, p.d_partial[src ^ 1], p.d_ticket, e);
            return;
        }
        lbfgs_reduce_kernel<<<(uint32_t)next, kLanes, 0, ctx->stream>>>(p.d_partial[src], count,
                                                                        p.d_partial[src ^ 1],
                                                                        next == 1 ? e : none);
        count = next;
        src ^= 1;
    }
}

struct Entry {
    Context *ctx = nullptr;
    Plan *plan = nullptr;
    std::unique_lock<std::mutex> lock;
};

int enter(uintptr_t device, const int *sizes, int n, Entry &out)
{
    clear_error();
    if (device == 0) {
        set_error("device handle is nil");
        return -1;
    }
    Context *ctx = resolve_device(device);
    if (!ctx) return -3;
    if (n <= 0 || !sizes) {
        set_error("L-BFGS needs at least one tensor and its size array");
        return -8;
    }
    if (!make_current(ctx)) return -8;
    out.lock = std::unique_lock<std::mutex>(ctx->mu);
    out.ctx = ctx;
    out.plan = find_plan(ctx, sizes, n);
    return out.plan ? 0 : -8;
}

}  // namespace

// A buffer of the library was freed: plans that hold a handle inside it validate and upload
// their handle table again on their next step (the address may come back with another length).
void lbfgs_forget_range(uintptr_t begin, size_t bytes)
{
    const uintptr_t end = begin + bytes;
    auto inside = [&](uintptr_t x) { return x >= begin && x < end; };
    for (auto &p : plan_cache())
        if (inside(p->alpha_handle) || std::any_of(p->handles.begin(), p->handles.end(), inside))
            p->handles_valid = false;
}

}  // namespace gm

using namespace gm;

extern "C" {

int execute_lbfgs_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers, uintptr_t *gradient_buffers,
                                uintptr_t *old_gradient_buffers, uintptr_t *search_dir_buffers,
                                uintptr_t *s_vectors_flat, uintptr_t *y_vectors_flat,
                                uintptr_t *rho_buffers, uintptr_t alpha_buffer, int num_weights,
                                int *buffer_sizes, int history_size, int history_count,
                                int history_index, float initial_step, float c1, float c2,
                                int max_line_search, float current_loss, float prev_loss,
                                float *step_size)
try {
    // The reference performs no line search: the Wolfe constants and the losses are accepted
    // and ignored (bridge_optimizer.m:1215-1216).
    (void)c1; (void)c2; (void)max_line_search; (void)current_loss; (void)prev_loss;
    Entry en;
    if (int rc = enter(device, buffer_sizes, num_weights, en)) return rc;
    if (!weight_buffers || !gradient_buffers || !old_gradient_buffers || !search_dir_buffers ||
        !s_vectors_flat || !y_vectors_flat || !rho_buffers) {
        set_error("L-BFGS buffer arrays are required");
        return -8;
    }
    if (history_size <= 0 || history_count < 0 || history_count > history_size || history_index < 0 ||
        history_index >= history_size) {
        set_error("L-BFGS history arguments out of range (size %d, count %d, index %d)", history_size,
                  history_count, history_index);
        return -5;
    }
    Context *ctx = en.ctx;
    Plan &p = *en.plan;
    const int n = num_weights, m = history_size;
    if (int rc = stage_handles(ctx, p, n, m, weight_buffers, gradient_buffers, old_gradient_buffers,
                               search_dir_buffers, s_vectors_flat, y_vectors_flat, rho_buffers, alpha_buffer))
        return rc;
    const Rows r = rows_of(p.d_handles, n, m);
    const Rows host = rows_of(p.handles.data(), n, m);
    float *alpha = reinterpret_cast<float *>(alpha_buffer);
    hipStream_t stream = ctx->stream;
    auto slot = [&](int j) { return (history_index - history_count + j + m) % m; };
    auto rho_ptr = [&](int idx) { return reinterpret_cast<float *>(host.rho[idx]); };

    // which pairs take part: one small read-back per step
    std::vector<int> valid;
    if (history_count > 0) {
        // the flags are written straight into pinned host memory: one wait, no copy launch
        lbfgs_prologue_kernel<<<1, 64, 0, stream>>>(r.rho, m, history_count, history_index, alpha, p.h_valid);
        if (!hip_ok(hipGetLastError(), "L-BFGS prologue launch") ||
            !hip_ok(hipStreamSynchronize(stream), "hipStreamSynchronize"))
            return -8;
        for (int j = 0; j < history_count; j++)
            if (p.h_valid[j]) valid.push_back(j);
    }

    StreamArgs base{};
    base.partial = p.d_partial[0];
    base.scalars = p.d_scalars;

    const int prev = (history_index - 1 + m) % m;

    if (!valid.empty()) {
        const int count = (int)valid.size();
        // q = -g (:1025-1038) stays in registers: the first dot product of the backward loop
        {
            StreamArgs a = base;
            a.r0 = r.g; a.r1 = r.s(slot(valid[count - 1]), n);
            launch_dot(ctx, p, a, true);
        }
        // backward loop, newest pair first (bridge_optimizer.m:1045-1130)
        for (int k = count - 1; k >= 0; k--) {
            const int j = valid[k], idx = slot(j);
            launch_reduction(ctx, p, Epilogue{kOpAlpha, rho_ptr(idx), alpha + j, nullptr, p.d_scalars});
            StreamArgs a = base;
            a.r0 = r.dir; a.r1 = r.y(idx, n); a.subtract = 1;
            // next dot: s of the next older valid pair, or y of the oldest one (first forward dot)
            a.r2 = k > 0 ? r.s(slot(valid[k - 1]), n) : r.y(slot(valid[0]), n);
            if (k == count - 1) {
                // the first axpy forms q = -g from the gradient and stores the result as the direction
                a.r0 = r.g; a.r3 = r.dir;
                launch_stream<kModeAxpyFirst, true>(ctx, p, a);
            } else {
                launch_stream<kModeAxpy, true>(ctx, p, a);
            }
        }
        // forward loop, oldest pair first (:1133-1201)
        for (int k = 0; k < count; k++) {
            const int j = valid[k], idx = slot(j);
            launch_reduction(ctx, p, Epilogue{kOpBeta, rho_ptr(idx), alpha + j, nullptr, p.d_scalars});
            StreamArgs a = base;
            a.r0 = r.dir; a.r1 = r.s(idx, n); a.subtract = 0;
            if (k + 1 < count) {
                a.r2 = r.y(slot(valid[k + 1]), n);
                launch_stream<kModeAxpy, true>(ctx, p, a);
            } else {
                launch_stream<kModeAxpy, false>(ctx, p, a);
            }
        }
    }
    // p = -r (r = -g when no pair took part); x += a p; old_g = g; s_cur = a p  (:1203-1259), and with a
    // non-empty history y_prev = g - old_g, rho_prev = 0  (:1262-1310)
    {
        UpdateArgs u{};
        u.dir = r.dir; u.w = r.w; u.g = r.g; u.old_g = r.old_g; u.s_cur = r.s(history_index, n);
        u.y_prev = r.y(prev, n);
        u.step = initial_step;
        launch_update(ctx, p, u, valid.empty(), history_count > 0);
    }
    if (step_size) *step_size = initial_step;
    if (history_count > 0)
        lbfgs_epilogue_kernel<<<1, 64, 0, stream>>>(nullptr, 0, Epilogue{kOpRho, nullptr, nullptr, rho_ptr(prev),
                                                                        p.d_scalars});
    return hip_ok(hipGetLastError(), "L-BFGS kernel launch") ? 0 : -8;
} catch (...) {
    note_exception();
    return -8;
}

int execute_lbfgs_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                       uintptr_t *gradient_buffers, uintptr_t *old_gradient_buffers,
                                       uintptr_t *search_dir_buffers, uintptr_t *s_vectors_flat,
                                       uintptr_t *y_vectors_flat, uintptr_t *rho_buffers,
                                       uintptr_t alpha_buffer, int num_weights, int *buffer_sizes,
                                       int history_size, int history_count, int history_index,
                                       float initial_step, float c1, float c2, int max_line_search,
                                       float current_loss, float prev_loss, uintptr_t command_pool,
                                       float *step_size)
{
    // With or without a pool the reference runs the same code (bridge_optimizer.m:1356-1392).
    (void)command_pool;
    return execute_lbfgs_step_mpsgraph(device, weight_buffers, gradient_buffers, old_gradient_buffers,
                                       search_dir_buffers, s_vectors_flat, y_vectors_flat, rho_buffers,
                                       alpha_buffer, num_weights, buffer_sizes, history_size,
                                       history_count, history_index, initial_step, c1, c2,
                                       max_line_search, current_loss, prev_loss, step_size);
}

int gm_lbfgs_dot(uintptr_t device, uintptr_t *a_buffers, uintptr_t *b_buffers, int num_tensors,
                 int *buffer_sizes, float *result)
try {
    Entry en;
    if (int rc = enter(device, buffer_sizes, num_tensors, en)) return rc;
    if (!a_buffers || !b_buffers || !result) {
        set_error("gm_lbfgs_dot: buffer arrays and result pointer are required");
        return -8;
    }
    Context *ctx = en.ctx;
    Plan &p = *en.plan;
    const int n = num_tensors;
    for (int i = 0; i < n; i++) {
        const size_t need = buffer_sizes[i] > 0 ? (size_t)buffer_sizes[i] / sizeof(float) * sizeof(float) : 0;
        for (uintptr_t h : {a_buffers[i], b_buffers[i]}) {
            const size_t have = registry_length(h);
            if (h == 0 || (have != 0 && have < need)) {
                set_error("gm_lbfgs_dot: buffer %d is nil or shorter than its tensor", i);
                return -8;
            }
        }
    }
    // a private two-row table; the step's cached table is left alone
    uintptr_t *d_rows = nullptr;
    LbScalars *h_result = nullptr;
    std::vector<uintptr_t> rows((size_t)2 * n);
    std::memcpy(rows.data(), a_buffers, (size_t)n * sizeof(uintptr_t));
    std::memcpy(rows.data() + n, b_buffers, (size_t)n * sizeof(uintptr_t));
    int rc = -8;
    if (hip_ok(hipMalloc(&d_rows, rows.size() * sizeof(uintptr_t)), "hipMalloc(dot rows)") &&
        hip_ok(hipHostMalloc(&h_result, sizeof(LbScalars), hipHostMallocDefault), "hipHostMalloc(dot result)") &&
        hip_ok(hipMemcpyAsync(d_rows, rows.data(), rows.size() * sizeof(uintptr_t), hipMemcpyHostToDevice,
                              ctx->stream), "upload dot rows")) {
        StreamArgs a{};
        a.partial = p.d_partial[0];
        a.scalars = p.d_scalars;
        a.r0 = d_rows;
        a.r1 = d_rows + n;
        launch_dot(ctx, p, a, false);
        launch_reduction(ctx, p, Epilogue{kOpStore, nullptr, nullptr, nullptr, p.d_scalars});
        if (hip_ok(hipGetLastError(), "dot kernel launch") &&
            hip_ok(hipMemcpyAsync(h_result, p.d_scalars, sizeof(LbScalars), hipMemcpyDeviceToHost, ctx->stream),
                   "read dot result") &&
            hip_ok(hipStreamSynchronize(ctx->stream), "hipStreamSynchronize")) {
            *result = h_result->dot;
            rc = 0;
        }
    }
    (void)hipStreamSynchronize(ctx->stream);
    if (d_rows) (void)hipFree(d_rows);
    if (h_result) (void)hipHostFree(h_result);
    return rc;
} catch (...) {
    note_exception();
    return -8;
}

}  // extern "C"
