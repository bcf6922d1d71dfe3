// The six update rules as per-element device functions.
//
// Each statement is one node of the reference's MPSGraph op chain
// (cgo_bridge/bridge_optimizer.m) and rounds once to binary32: this file must
// be compiled with -ffp-contract=off (no FMA fusion) and hipcc's default
// correctly rounded fp32 division and square root, with fp32 denormals on.
// Scalars such as 1-beta and the bias corrections are computed on the host in
// binary32 and arrive in StepParams.
#pragma once

#include <hip/hip_runtime.h>

namespace gm {

struct StepParams {
    float lr;
    float beta1, beta2;         // Adam / NAdam
    float one_minus_beta1, one_minus_beta2;
    float bc1, bc2;             // 1 - beta^t
    float mu, one_minus_mu;     // NAdam momentum schedule at t+1
    float eps;
    float weight_decay;
    float momentum;             // SGD / RMSProp
    float alpha, one_minus_alpha;   // RMSProp
    float rho, one_minus_rho;       // AdaDelta
    int nesterov;
};

// bridge_optimizer.m:313-347 (no momentum buffer)
struct SgdVanillaRule {
    static constexpr int NSTATE = 0;
    __device__ static inline void apply(float &w, float g, float *, const StepParams &p)
    {
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            g = g + decay;
        }
        float upd = p.lr * g;
        w = w - upd;
    }
};

// bridge_optimizer.m:219-311
struct SgdMomentumRule {
    static constexpr int NSTATE = 1;
    __device__ static inline void apply(float &w, float g, float *s, const StepParams &p)
    {
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            g = g + decay;
        }
        float scaled = s[0] * p.momentum;
        float m = scaled + g;
        float upd;
        if (p.nesterov != 0) {
            float t1 = p.momentum * m;
            float t2 = t1 + g;
            upd = p.lr * t2;
        } else {
            upd = p.lr * m;
        }
        w = w - upd;
        s[0] = m;
    }
};

// bridge_optimizer.m:484-550
struct AdamRule {
    static constexpr int NSTATE = 2;
    __device__ static inline void apply(float &w, float g, float *s, const StepParams &p)
    {
        float m_scaled = s[0] * p.beta1;
        float g_scaled = g * p.one_minus_beta1;
        float m = m_scaled + g_scaled;
        float g_sq = g * g;
        float v_scaled = s[1] * p.beta2;
        float g_sq_scaled = g_sq * p.one_minus_beta2;
        float v = v_scaled + g_sq_scaled;
        float m_hat = m / p.bc1;
        float v_hat = v / p.bc2;
        float root = sqrtf(v_hat);
        float den = root + p.eps;
        float upd = m_hat / den;
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            upd = upd + decay;
        }
        float scaled = upd * p.lr;
        w = w - scaled;
        s[0] = m;
        s[1] = v;
    }
};

// bridge_optimizer.m:782-876.  State order: squared-gradient average, then
// the momentum buffer (if MOMENTUM), then the gradient average (if CENTERED).
template <bool MOMENTUM, bool CENTERED>
struct RmsPropRule {
    static constexpr int NSTATE = 1 + (MOMENTUM ? 1 : 0) + (CENTERED ? 1 : 0);
    __device__ static inline void apply(float &w, float g, float *s, const StepParams &p)
    {
        float g_sq = g * g;
        float s_scaled = s[0] * p.alpha;
        float g_sq_scaled = g_sq * p.one_minus_alpha;
        float sq = s_scaled + g_sq_scaled;
        float den;
        if (CENTERED) {
            constexpr int GA = MOMENTUM ? 2 : 1;
            float ga_scaled = s[GA] * p.alpha;
            float g_term = g * p.one_minus_alpha;
            float ga = ga_scaled + g_term;
            float ga_sq = ga * ga;
            float var = sq - ga_sq;
            float var_eps = var + p.eps;
            den = sqrtf(var_eps);
            s[GA] = ga;
        } else {
            float s_eps = sq + p.eps;
            den = sqrtf(s_eps);
        }
        float upd = g / den;
        if (MOMENTUM) {
            float b_scaled = s[1] * p.momentum;
            float b = b_scaled + upd;
            s[1] = b;
            upd = b;
        }
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            upd = upd + decay;
        }
        float scaled = upd * p.lr;
        w = w - scaled;
        s[0] = sq;
    }
};

// bridge_optimizer.m:1480-1517
struct AdaGradRule {
    static constexpr int NSTATE = 1;
    __device__ static inline void apply(float &w, float g, float *s, const StepParams &p)
    {
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            g = g + decay;
        }
        float g_sq = g * g;
        float acc = s[0] + g_sq;
        float root = sqrtf(acc);
        float den = root + p.eps;
        float alr = p.lr / den;
        float upd = alr * g;
        w = w - upd;
        s[0] = acc;
    }
};

// bridge_optimizer.m:1773-1843
struct AdaDeltaRule {
    static constexpr int NSTATE = 2;
    __device__ static inline void apply(float &w, float g, float *s, const StepParams &p)
    {
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            g = g + decay;
        }
        float a = s[1];
        float g_sq = g * g;
        float s_scaled = s[0] * p.rho;
        float g_sq_scaled = g_sq * p.one_minus_rho;
        float sq = s_scaled + g_sq_scaled;
        float s_eps = sq + p.eps;
        float rms_g = sqrtf(s_eps);
        float a_eps = a + p.eps;
        float rms_u = sqrtf(a_eps);
        float alr = rms_u / rms_g;
        float d = alr * g;
        float neg_d = -d;
        w = w + neg_d;
        float d_sq = neg_d * neg_d;
        float a_scaled = a * p.rho;
        float d_sq_scaled = d_sq * p.one_minus_rho;
        s[1] = a_scaled + d_sq_scaled;
        s[0] = sq;
    }
};

// bridge_optimizer.m:2114-2200
struct NAdamRule {
    static constexpr int NSTATE = 2;
    __device__ static inline void apply(float &w, float g, float *s, const StepParams &p)
    {
        float m_scaled = s[0] * p.beta1;
        float g_scaled = g * p.one_minus_beta1;
        float m = m_scaled + g_scaled;
        float g_sq = g * g;
        float v_scaled = s[1] * p.beta2;
        float g_sq_scaled = g_sq * p.one_minus_beta2;
        float v = v_scaled + g_sq_scaled;
        float v_hat = v / p.bc2;
        float m_hat = m / p.bc1;
        float g_hat = g / p.bc1;
        float m_term = m_hat * p.mu;
        float g_term = g_hat * p.one_minus_mu;
        float m_bar = m_term + g_term;
        float root = sqrtf(v_hat);
        float den = root + p.eps;
        float upd = m_bar / den;
        if (p.weight_decay > 0.0f) {
            float decay = w * p.weight_decay;
            upd = upd + decay;
        }
        float scaled = upd * p.lr;
        w = w - scaled;
        s[0] = m;
        s[1] = v;
    }
};

}  // namespace gm
