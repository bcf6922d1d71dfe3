// Device side of the multi-tensor update: one lane's share of a slice for any update rule,
// and the kernels that walk a chunk table with it.  Shared by the fp32 entry points, the
// mixed-precision step and the allocation-free step (each translation unit instantiates the
// shapes it launches).
//
// Workgroup b handles slice (b mod slices_per_chunk) of chunk (b div slices_per_chunk), one
// VEC-wide group per lane: load every stream once, apply the rule in registers, store every
// state once, exit.
#pragma once

#include "gm_launch.hpp"
#include "gm_planner.hpp"
#include "gm_rules.hpp"

namespace gm {

typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;

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
    const LaneShare s = lane_share(ch.count, ch.flags, slice, threadIdx.x, VEC, BLOCK);
    if (s.count == 0) return;
    if (VEC > 1 && s.grouped) {
        update_group<Rule, VEC, NT, AMP>(ch, s.first, prm, inv_scale);
    } else {
        for (uint32_t e = 0; e < s.count; e++) update_group<Rule, 1, NT, AMP>(ch, s.first + e, prm, inv_scale);
    }
}

template <class Rule, int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
multi_tensor_update_kernel(const Chunk *__restrict__ chunks, uint32_t slice_shift, StepParams prm)
{
    const Chunk ch = chunks[blockIdx.x >> slice_shift];
    // An idle slice leaves here.  (The weight pointer is never null; testing it together with the
    // count makes the compiler fetch the whole descriptor with one wait, instead of the count
    // first and, behind the branch and a second wait, the addresses.)
    const uint32_t first_lane_element = (blockIdx.x & ((1u << slice_shift) - 1u)) * BLOCK * VEC;
    if ((first_lane_element >= ch.count) | (ch.p[kSlotWeight] == nullptr)) return;
    update_slice<Rule, VEC, NT, false, BLOCK>(ch, slice_shift, prm, 1.0f);
}

// SGD: a tensor without a momentum buffer takes the vanilla rule.
template <int VEC, bool NT, int BLOCK>
__global__ void __launch_bounds__(BLOCK)
multi_tensor_sgd_kernel(const Chunk *__restrict__ chunks, uint32_t slice_shift, StepParams prm)
{
    const Chunk ch = chunks[blockIdx.x >> slice_shift];
    const uint32_t first_lane_element = (blockIdx.x & ((1u << slice_shift) - 1u)) * BLOCK * VEC;
    if ((first_lane_element >= ch.count) | (ch.p[kSlotWeight] == nullptr)) return;     // as above
    if (prm.momentum > 0.0f && ch.p[kSlotState0] != nullptr)
        update_slice<SgdMomentumRule, VEC, NT, false, BLOCK>(ch, slice_shift, prm, 1.0f);
    else
        update_slice<SgdVanillaRule, VEC, NT, false, BLOCK>(ch, slice_shift, prm, 1.0f);
}

// Launches one segment of an fp32 rule in the requested shape.
template <class Rule, int VEC, int BLOCK>
inline void launch_update_shape(hipStream_t st, const SegmentLaunch &g, const StepParams &prm, bool nt)
{
    if (nt) multi_tensor_update_kernel<Rule, VEC, true, BLOCK><<<g.grid, BLOCK, 0, st>>>(g.chunks, g.shift, prm);
    else multi_tensor_update_kernel<Rule, VEC, false, BLOCK><<<g.grid, BLOCK, 0, st>>>(g.chunks, g.shift, prm);
}

template <class Rule>
inline void launch_update(hipStream_t st, const SegmentLaunch &g, const StepParams &prm, int vec, int block, bool nt)
{
    if (block == 128) {
        if (vec == 4) launch_update_shape<Rule, 4, 128>(st, g, prm, nt);
        else if (vec == 2) launch_update_shape<Rule, 2, 128>(st, g, prm, nt);
        else launch_update_shape<Rule, 1, 128>(st, g, prm, nt);
    } else {
        if (vec == 4) launch_update_shape<Rule, 4, kBlock>(st, g, prm, nt);
        else if (vec == 2) launch_update_shape<Rule, 2, kBlock>(st, g, prm, nt);
        else launch_update_shape<Rule, 1, kBlock>(st, g, prm, nt);
    }
}

}  // namespace gm
