// Multi-tensor-apply optimizer steps for gfx950: the execute_*_step entry points of the C ABI
// for the fp32 rules (the HIP counterpart of cgo_bridge/bridge_optimizer.m).
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
#include "gm_launch.hpp"
#include "gm_update_kernels.hpp"

#include "../../include/gometal_hip.h"

#include <cmath>

namespace gm {

template <class Rule>
static int launch_rule(const Launch &l, const StepParams &prm, int hip_error_code)
{
    if (l.plan->num_chunks == 0) return 0;
    constexpr int streams = 3 + 2 * Rule::NSTATE;          // w, g, states read; w, states written
    int vec = current_vec(l.ctx), block = current_block(l.ctx);
    if (vec == 0) vec = auto_vec(streams);
    if (block == 0) block = auto_block(streams);
    SegmentLaunch seg[2];
    int count;
    if (!launch_geometry(*l.plan, vec, block, seg, count)) return hip_error_code;
    for (int s = 0; s < count; s++) launch_update<Rule>(l.ctx->stream, seg[s], prm, vec, block, current_nontemporal(l.ctx));
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
    int vec = current_vec(l.ctx);
    if (vec == 0) vec = auto_vec(5);
    const bool nt = current_nontemporal(l.ctx);
    int block = current_block(l.ctx);
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

}  // extern "C"
