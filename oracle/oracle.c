/*
 * CPU oracle for the go-metal optimizer step (see oracle.h).  TEST
 * INFRASTRUCTURE ONLY: nothing in the shipped library links this file.
 *
 * Every statement below is one node of the reference's MPSGraph op chain and
 * performs exactly one binary32 rounding.  Build flags that this relies on:
 * -ffp-contract=off (no FMA fusion), no -ffast-math, SSE scalar/vector math
 * (IEEE division and square root), denormals left enabled.
 */
#include "oracle.h"

#include <float.h>
#include <math.h>
#include <string.h>

#define GM_PARALLEL_FOR _Pragma("omp parallel for schedule(static) num_threads(nt) if(nt > 1)")

static int clamp_threads(int nthreads) { return nthreads < 1 ? 1 : nthreads; }

/* bridge_optimizer.m:398-399 */
void gm_oracle_bias_corrections(float beta1, float beta2, int step, float *bc1, float *bc2)
{
    *bc1 = 1.0f - powf(beta1, (float)step);
    *bc2 = 1.0f - powf(beta2, (float)step);
}

/* bridge_optimizer.m:2066 (momentum_schedule_next; the :2065 value is unused there) */
float gm_oracle_nadam_mu_next(float beta1, int step)
{
    float exponent = (float)(step + 1) * 0.004f;
    float decay = powf(0.96f, exponent);
    float half_decay = 0.5f * decay;
    float one_minus = 1.0f - half_decay;
    return beta1 * one_minus;
}

/* bridge_optimizer.m:160-357 */
void gm_oracle_sgd_step(float *w, const float *g, float *m, size_t n,
                        float lr, float momentum, float weight_decay, int nesterov,
                        int nthreads)
{
    const int nt = clamp_threads(nthreads);
    const int use_momentum = (momentum > 0.0f) && (m != NULL);   /* :233 */
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) {
        float wi = w[i];
        float gi = g[i];
        if (weight_decay > 0.0f) {          /* :219-228 */
            float decay = wi * weight_decay;
            gi = gi + decay;
        }
        if (use_momentum) {
            float scaled = m[i] * momentum;  /* :245 */
            float mi = scaled + gi;          /* :248 */
            float upd;
            if (nesterov != 0) {             /* :257-267 */
                float t1 = momentum * mi;
                float t2 = t1 + gi;
                upd = lr * t2;
            } else {                         /* :270-272 */
                upd = lr * mi;
            }
            w[i] = wi - upd;                 /* :276 */
            m[i] = mi;
        } else {                             /* :315-322 */
            float upd = lr * gi;
            w[i] = wi - upd;
        }
    }
}

/* One element of bridge_optimizer.m:484-550; shared with the AMP step. */
static inline void adam_element(float *w, float g, float *m, float *v,
                                float lr, float beta1, float beta2,
                                float one_minus_beta1, float one_minus_beta2,
                                float eps, float weight_decay, float bc1, float bc2)
{
    float wi = *w;
    float m_scaled = *m * beta1;               /* :484 */
    float g_scaled = g * one_minus_beta1;      /* :487 */
    float mi = m_scaled + g_scaled;            /* :490 */
    float g_sq = g * g;                        /* :495 */
    float v_scaled = *v * beta2;               /* :498 */
    float g_sq_scaled = g_sq * one_minus_beta2;/* :501 */
    float vi = v_scaled + g_sq_scaled;         /* :504 */
    float m_hat = mi / bc1;                    /* :509 */
    float v_hat = vi / bc2;                    /* :514 */
    float root = sqrtf(v_hat);                 /* :519 */
    float den = root + eps;                    /* :521 */
    float upd = m_hat / den;                   /* :526 */
    if (weight_decay > 0.0f) {                 /* :531-540 */
        float decay = wi * weight_decay;
        upd = upd + decay;
    }
    float scaled = upd * lr;                   /* :543 */
    *w = wi - scaled;                          /* :548 */
    *m = mi;
    *v = vi;
}

/* bridge_optimizer.m:360-641 */
void gm_oracle_adam_step(float *w, const float *g, float *m, float *v, size_t n,
                         float lr, float beta1, float beta2, float eps, float weight_decay,
                         int step, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    float bc1, bc2;
    gm_oracle_bias_corrections(beta1, beta2, step, &bc1, &bc2);
    const float omb1 = 1.0f - beta1;           /* :469 */
    const float omb2 = 1.0f - beta2;           /* :471 */
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++)
        adam_element(&w[i], g[i], &m[i], &v[i], lr, beta1, beta2, omb1, omb2,
                     eps, weight_decay, bc1, bc2);
}

/* bridge_optimizer.m:691-951 */
void gm_oracle_rmsprop_step(float *w, const float *g, float *s, float *mom, float *gavg, size_t n,
                            float lr, float alpha, float eps, float weight_decay,
                            float momentum, int centered, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    const float oma = 1.0f - alpha;            /* :773 */
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) {
        float wi = w[i];
        float gi = g[i];
        float g_sq = gi * gi;                  /* :782 */
        float s_scaled = s[i] * alpha;         /* :785 */
        float g_sq_scaled = g_sq * oma;        /* :788 */
        float si = s_scaled + g_sq_scaled;     /* :791 */
        float den;
        if (centered) {                        /* :797-824 */
            float ga_scaled = gavg[i] * alpha;
            float g_term = gi * oma;
            float ga = ga_scaled + g_term;
            float ga_sq = ga * ga;
            float var = si - ga_sq;
            float var_eps = var + eps;
            den = sqrtf(var_eps);
            gavg[i] = ga;
        } else {                               /* :827-830 */
            float s_eps = si + eps;
            den = sqrtf(s_eps);
        }
        float upd = gi / den;                  /* :834 */
        if (momentum > 0.0f) {                 /* :839-854 */
            float b_scaled = mom[i] * momentum;
            float bi = b_scaled + upd;
            mom[i] = bi;
            upd = bi;
        }
        if (weight_decay > 0.0f) {             /* :857-866 */
            float decay = wi * weight_decay;
            upd = upd + decay;
        }
        float scaled = upd * lr;               /* :869 */
        w[i] = wi - scaled;                    /* :874 */
        s[i] = si;
    }
}

/* bridge_optimizer.m:1421-1588 */
void gm_oracle_adagrad_step(float *w, const float *g, float *s, size_t n,
                            float lr, float eps, float weight_decay, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) {
        float wi = w[i];
        float gi = g[i];
        if (weight_decay > 0.0f) {             /* :1480-1488 */
            float decay = wi * weight_decay;
            gi = gi + decay;
        }
        float g_sq = gi * gi;                  /* :1492 */
        float si = s[i] + g_sq;                /* :1495 */
        float root = sqrtf(si);                /* :1501 */
        float den = root + eps;                /* :1503 */
        float alr = lr / den;                  /* :1506 */
        float upd = alr * gi;                  /* :1512 */
        w[i] = wi - upd;                       /* :1515 */
        s[i] = si;
    }
}

/* bridge_optimizer.m:1708-1925 */
void gm_oracle_adadelta_step(float *w, const float *g, float *s, float *a, size_t n,
                             float rho, float eps, float weight_decay, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    const float omr = 1.0f - rho;
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) {
        float wi = w[i];
        float gi = g[i];
        float ai = a[i];
        if (weight_decay > 0.0f) {             /* :1773-1781 */
            float decay = wi * weight_decay;
            gi = gi + decay;
        }
        float g_sq = gi * gi;                  /* :1785 */
        float s_scaled = s[i] * rho;           /* :1788 */
        float g_sq_scaled = g_sq * omr;        /* :1791 */
        float si = s_scaled + g_sq_scaled;     /* :1794 */
        float s_eps = si + eps;                /* :1800 */
        float rms_g = sqrtf(s_eps);            /* :1803 */
        float a_eps = ai + eps;                /* :1807 */
        float rms_u = sqrtf(a_eps);            /* :1810 */
        float alr = rms_u / rms_g;             /* :1815 */
        float d = alr * gi;                    /* :1818 */
        float neg_d = -d;                      /* :1821 */
        w[i] = wi + neg_d;                     /* :1826 */
        float d_sq = neg_d * neg_d;            /* :1832 */
        float a_scaled = ai * rho;             /* :1835 */
        float d_sq_scaled = d_sq * omr;        /* :1838 */
        a[i] = a_scaled + d_sq_scaled;         /* :1841 */
        s[i] = si;
    }
}

/* bridge_optimizer.m:2023-2280 */
void gm_oracle_nadam_step(float *w, const float *g, float *m, float *v, size_t n,
                          float lr, float beta1, float beta2, float eps, float weight_decay,
                          int step, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    float bc1, bc2;
    gm_oracle_bias_corrections(beta1, beta2, step, &bc1, &bc2);   /* :2061-2062 */
    const float mu = gm_oracle_nadam_mu_next(beta1, step);        /* :2066 */
    const float one_minus_mu = 1.0f - mu;                         /* :2153 */
    const float omb1 = 1.0f - beta1;
    const float omb2 = 1.0f - beta2;
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) {
        float wi = w[i];
        float gi = g[i];
        float m_scaled = m[i] * beta1;          /* :2114 */
        float g_scaled = gi * omb1;             /* :2117 */
        float mi = m_scaled + g_scaled;         /* :2120 */
        float g_sq = gi * gi;                   /* :2125 */
        float v_scaled = v[i] * beta2;          /* :2128 */
        float g_sq_scaled = g_sq * omb2;        /* :2131 */
        float vi = v_scaled + g_sq_scaled;      /* :2134 */
        float v_hat = vi / bc2;                 /* :2139 */
        float m_hat = mi / bc1;                 /* :2145 */
        float g_hat = gi / bc1;                 /* :2148 */
        float m_term = m_hat * mu;              /* :2158 */
        float g_term = g_hat * one_minus_mu;    /* :2161 */
        float m_bar = m_term + g_term;          /* :2164 */
        float root = sqrtf(v_hat);              /* :2170 */
        float den = root + eps;                 /* :2171 */
        float upd = m_bar / den;                /* :2176 */
        if (weight_decay > 0.0f) {              /* :2181-2190 */
            float decay = wi * weight_decay;
            upd = upd + decay;
        }
        float scaled = upd * lr;                /* :2193 */
        w[i] = wi - scaled;                     /* :2198 */
        m[i] = mi;
        v[i] = vi;
    }
}

/* ---- fp16 casts, bridge_memory.m:361-377 ---- */

uint16_t gm_oracle_f32_to_f16(float x)
{
    uint32_t u;
    memcpy(&u, &x, sizeof u);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t exp = (u >> 23) & 0xFFu;
    uint32_t man = u & 0x7FFFFFu;
    if (exp == 0xFFu) {                         /* inf / NaN */
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        /* quiet NaN, keep the top payload bits */
        return (uint16_t)(sign | 0x7E00u | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;        /* biased half exponent */
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);   /* overflow before rounding */
    if (e <= 0) {
        /* subnormal half or zero: value = 1.man * 2^(exp-127), ulp = 2^-24 */
        if (e < -10) return (uint16_t)sign;     /* below half of the smallest subnormal */
        uint32_t full = man | 0x800000u;        /* 24-bit significand */
        uint32_t shift = (uint32_t)(14 - e);    /* 14..24 */
        uint32_t q = full >> shift;
        uint32_t rem = full & ((1u << shift) - 1u);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (q & 1u))) q++;
        return (uint16_t)(sign | q);            /* q may carry into the normal range */
    }
    uint32_t q = ((uint32_t)e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (q & 1u))) q++;   /* may carry up to inf */
    return (uint16_t)(sign | q);
}

float gm_oracle_f16_to_f32(uint16_t h)
{
    uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    uint32_t u;
    if (exp == 0x1Fu) {
        u = sign | 0x7F800000u | (man << 13);
    } else if (exp != 0) {
        u = sign | ((exp - 15 + 127) << 23) | (man << 13);
    } else if (man == 0) {
        u = sign;
    } else {
        /* subnormal half: normalise */
        int e = -1;
        do { e++; man <<= 1; } while ((man & 0x400u) == 0);
        u = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
    float f;
    memcpy(&f, &u, sizeof f);
    return f;
}

/* The two conversions above are the reference: one branch per class of value.  The loops
 * below run them over hundreds of millions of elements per step, so the common class (a result
 * in the normal half range) is handled inline by integer arithmetic and everything else falls
 * through to the reference.  gm_oracle_f16_fast_mismatches compares the two forms over any
 * range of bit patterns; the tests run it over all 2^32 floats and all 2^16 halves. */
static inline float f16_to_f32_fast(uint16_t h)
{
    const uint32_t em = (uint32_t)h & 0x7FFFu;
    if (em - 0x0400u < 0x7800u) {               /* exponent field 1..30: a normal half */
        const uint32_t u = (((uint32_t)h & 0x8000u) << 16) | ((em << 13) + 0x38000000u);
        float f;
        memcpy(&f, &u, sizeof f);
        return f;
    }
    return gm_oracle_f16_to_f32(h);
}

static inline uint16_t f32_to_f16_fast(float x)
{
    uint32_t u;
    memcpy(&u, &x, sizeof u);
    const uint32_t a = u & 0x7FFFFFFFu;
    /* 2^-14 <= |x| < 65504: the result is a normal half and rounding cannot reach infinity */
    if (a - 0x38800000u < 0x477FE000u - 0x38800000u) {
        const uint32_t r = a + 0xFFFu + ((a >> 13) & 1u);     /* nearest, ties to even, at bit 13 */
        return (uint16_t)(((u >> 16) & 0x8000u) | ((r - 0x38000000u) >> 13));
    }
    return gm_oracle_f32_to_f16(x);
}

uint64_t gm_oracle_f16_fast_mismatches(uint64_t first_bits, uint64_t count, int halves, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    uint64_t bad = 0;
    #pragma omp parallel for schedule(static) num_threads(nt) if(nt > 1) reduction(+:bad)
    for (uint64_t k = 0; k < count; k++) {
        if (halves) {
            const uint16_t h = (uint16_t)(first_bits + k);
            const float a = f16_to_f32_fast(h), b = gm_oracle_f16_to_f32(h);
            bad += memcmp(&a, &b, sizeof a) != 0;
        } else {
            const uint32_t u = (uint32_t)(first_bits + k);
            float x;
            memcpy(&x, &u, sizeof x);
            bad += f32_to_f16_fast(x) != gm_oracle_f32_to_f16(x);
        }
    }
    return bad;
}

void gm_oracle_convert_f32_to_f16(const float *src, uint16_t *dst, size_t n, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) dst[i] = f32_to_f16_fast(src[i]);
}

void gm_oracle_convert_f16_to_f32(const uint16_t *src, float *dst, size_t n, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    GM_PARALLEL_FOR
    for (size_t i = 0; i < n; i++) dst[i] = f16_to_f32_fast(src[i]);
}

/* ---- mixed-precision Adam ---- */

int gm_oracle_amp_found_inf(const uint16_t *const *g16, const size_t *n, int num_tensors, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    int found = 0;
    for (int t = 0; t < num_tensors; t++) {
        const uint16_t *g = g16[t];
        const size_t cnt = n[t];
        int local = 0;
        #pragma omp parallel for schedule(static) num_threads(nt) if(nt > 1) reduction(|:local)
        for (size_t i = 0; i < cnt; i++)
            local |= ((g[i] & 0x7C00u) == 0x7C00u);
        found |= local;
    }
    return found;
}

/* Eight elements of the mixed-precision Adam step at once, for hosts with AVX2 and F16C: the
 * same operations in the same order as the scalar loop below, each one a single IEEE
 * binary32 operation per lane (explicit intrinsics, no FMA in the target set), the two
 * conversions by the hardware (vcvtph2ps is exact, vcvtps2ph rounds to nearest even and
 * quiets NaNs exactly like gm_oracle_f32_to_f16).  gm_oracle_amp_vector_mismatches runs both
 * forms over the same data; the tests hold them to identical bits. */
#if defined(__x86_64__)
#include <immintrin.h>
#define GM_HAVE_AMP_VECTOR 1
__attribute__((target("avx2,f16c")))
static void adam_amp_span_avx2(float *w, const uint16_t *g16, float *m, float *v, uint16_t *w16, size_t n,
                               float lr, float beta1, float beta2, float omb1, float omb2, float eps,
                               float weight_decay, float bc1, float bc2, float inv_scale)
{
    const __m256 vlr = _mm256_set1_ps(lr), vb1 = _mm256_set1_ps(beta1), vb2 = _mm256_set1_ps(beta2);
    const __m256 vomb1 = _mm256_set1_ps(omb1), vomb2 = _mm256_set1_ps(omb2), veps = _mm256_set1_ps(eps);
    const __m256 vwd = _mm256_set1_ps(weight_decay), vbc1 = _mm256_set1_ps(bc1), vbc2 = _mm256_set1_ps(bc2);
    const __m256 vinv = _mm256_set1_ps(inv_scale);
    const int decay_on = weight_decay > 0.0f;
    for (size_t i = 0; i + 8 <= n; i += 8) {
        const __m256 g = _mm256_mul_ps(_mm256_cvtph_ps(_mm_loadu_si128((const __m128i *)(g16 + i))), vinv);
        const __m256 wi = _mm256_loadu_ps(w + i);
        const __m256 mi = _mm256_add_ps(_mm256_mul_ps(_mm256_loadu_ps(m + i), vb1), _mm256_mul_ps(g, vomb1));
        const __m256 vi = _mm256_add_ps(_mm256_mul_ps(_mm256_loadu_ps(v + i), vb2),
                                        _mm256_mul_ps(_mm256_mul_ps(g, g), vomb2));
        const __m256 m_hat = _mm256_div_ps(mi, vbc1);
        const __m256 v_hat = _mm256_div_ps(vi, vbc2);
        const __m256 den = _mm256_add_ps(_mm256_sqrt_ps(v_hat), veps);
        __m256 upd = _mm256_div_ps(m_hat, den);
        if (decay_on) upd = _mm256_add_ps(upd, _mm256_mul_ps(wi, vwd));
        const __m256 wn = _mm256_sub_ps(wi, _mm256_mul_ps(upd, vlr));
        _mm256_storeu_ps(w + i, wn);
        _mm256_storeu_ps(m + i, mi);
        _mm256_storeu_ps(v + i, vi);
        _mm_storeu_si128((__m128i *)(w16 + i), _mm256_cvtps_ph(wn, _MM_FROUND_TO_NEAREST_INT | _MM_FROUND_NO_EXC));
    }
}
static int amp_vector_usable(void)
{
    return __builtin_cpu_supports("avx2") && __builtin_cpu_supports("f16c");
}
#else
#define GM_HAVE_AMP_VECTOR 0
#endif

/* One tensor of the applied step: elements [0, n).  use_vector = 0 forces the scalar form. */
static void adam_amp_tensor(float *wt, const uint16_t *gt, float *mt, float *vt, uint16_t *ht, size_t cnt,
                            float lr, float beta1, float beta2, float omb1, float omb2, float eps,
                            float weight_decay, float bc1, float bc2, float inv_scale, int nt, int use_vector)
{
#if GM_HAVE_AMP_VECTOR
    if (use_vector && amp_vector_usable()) {
        /* spans of a multiple of eight elements per thread; the tail below is scalar */
        const size_t span = 1u << 16;
        const size_t spans = cnt / span;
        #pragma omp parallel for schedule(static) num_threads(nt) if(nt > 1)
        for (size_t s = 0; s < spans; s++)
            adam_amp_span_avx2(wt + s * span, gt + s * span, mt + s * span, vt + s * span, ht + s * span, span, lr,
                               beta1, beta2, omb1, omb2, eps, weight_decay, bc1, bc2, inv_scale);
        const size_t done = spans * span;
        const size_t rest8 = (cnt - done) / 8 * 8;
        adam_amp_span_avx2(wt + done, gt + done, mt + done, vt + done, ht + done, rest8, lr, beta1, beta2, omb1,
                           omb2, eps, weight_decay, bc1, bc2, inv_scale);
        wt += done + rest8, gt += done + rest8, mt += done + rest8, vt += done + rest8, ht += done + rest8;
        cnt -= done + rest8;
    }
#else
    (void)use_vector;
#endif
    GM_PARALLEL_FOR
    for (size_t i = 0; i < cnt; i++) {
        float gi = f16_to_f32_fast(gt[i]) * inv_scale;
        adam_element(&wt[i], gi, &mt[i], &vt[i], lr, beta1, beta2, omb1, omb2,
                     eps, weight_decay, bc1, bc2);
        ht[i] = f32_to_f16_fast(wt[i]);
    }
}

uint64_t gm_oracle_amp_vector_mismatches(const float *w, const uint16_t *g16, const float *m, const float *v,
                                         size_t n, float lr, float beta1, float beta2, float eps,
                                         float weight_decay, float bc1, float bc2, float inv_scale)
{
#if GM_HAVE_AMP_VECTOR
    if (!amp_vector_usable()) return UINT64_MAX;
    uint64_t bad = 0;
    const float omb1 = 1.0f - beta1, omb2 = 1.0f - beta2;
    float a[4][64], b[4][64];             /* w, m, v and (as floats) nothing: blocks of 64 elements */
    uint16_t ha[64], hb[64];
    for (size_t i = 0; i < n; i += 64) {
        const size_t k = n - i < 64 ? n - i : 64;
        memcpy(a[0], w + i, k * 4), memcpy(a[1], m + i, k * 4), memcpy(a[2], v + i, k * 4);
        memcpy(b[0], w + i, k * 4), memcpy(b[1], m + i, k * 4), memcpy(b[2], v + i, k * 4);
        memset(ha, 0, sizeof ha), memset(hb, 0, sizeof hb);
        adam_amp_tensor(a[0], g16 + i, a[1], a[2], ha, k, lr, beta1, beta2, omb1, omb2, eps, weight_decay, bc1, bc2,
                        inv_scale, 1, 1);
        adam_amp_tensor(b[0], g16 + i, b[1], b[2], hb, k, lr, beta1, beta2, omb1, omb2, eps, weight_decay, bc1, bc2,
                        inv_scale, 1, 0);
        /* identical bits, except that any NaN equals any NaN: which operand's payload survives an
         * operation on two NaNs depends on operand order, which the compiler is free to choose */
        int differs = 0;
        for (int q = 0; q < 3; q++)
            for (size_t e = 0; e < k; e++)
                differs |= memcmp(&a[q][e], &b[q][e], 4) != 0 && !(isnan(a[q][e]) && isnan(b[q][e]));
        for (size_t e = 0; e < k; e++)
            differs |= ha[e] != hb[e] && !((ha[e] & 0x7FFFu) > 0x7C00u && (hb[e] & 0x7FFFu) > 0x7C00u);
        bad += differs;
    }
    return bad;
#else
    (void)w, (void)g16, (void)m, (void)v, (void)n, (void)lr, (void)beta1, (void)beta2, (void)eps;
    (void)weight_decay, (void)bc1, (void)bc2, (void)inv_scale;
    return UINT64_MAX;
#endif
}

int gm_oracle_adam_amp_step(float *const *w, const uint16_t *const *g16, float *const *m,
                            float *const *v, uint16_t *const *w16, const size_t *n, int num_tensors,
                            float lr, float beta1, float beta2, float eps, float weight_decay,
                            gm_oracle_amp_state *st, int nthreads)
{
    const int nt = clamp_threads(nthreads);
    if (gm_oracle_amp_found_inf(g16, n, num_tensors, nthreads)) {
        const float next = st->scale * st->backoff_factor;
        if (next >= FLT_MIN) st->scale = next;        /* the scale stays a normal number */
        st->growth_tracker = 0;
        return 1;
    }
    st->step_count += 1;
    float bc1, bc2;
    gm_oracle_bias_corrections(beta1, beta2, (int)st->step_count, &bc1, &bc2);
    const float omb1 = 1.0f - beta1;
    const float omb2 = 1.0f - beta2;
    const float inv_scale = 1.0f / st->scale;
    for (int t = 0; t < num_tensors; t++)
        adam_amp_tensor(w[t], g16[t], m[t], v[t], w16[t], n[t], lr, beta1, beta2, omb1, omb2, eps, weight_decay,
                        bc1, bc2, inv_scale, nt, 1);
    st->growth_tracker += 1;
    if (st->growth_tracker == st->growth_interval) {
        const float next = st->scale * st->growth_factor;
        if (next <= FLT_MAX) st->scale = next;        /* "up to maximum": never +inf */
        st->growth_tracker = 0;
    }
    return 0;
}
