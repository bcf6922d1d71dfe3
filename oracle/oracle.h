/*
 * CPU oracle for the go-metal optimizer step.  TEST INFRASTRUCTURE ONLY.
 *
 * This is a plain-C restatement of the update equations that the reference
 * evaluates as MPSGraph op chains in cgo_bridge/bridge_optimizer.m, with every
 * arithmetic node of the graph written as exactly one IEEE-754 binary32
 * operation (build with -ffp-contract=off, no fast-math).  Only tests/, the
 * smoke check and the bench's cpu_baseline leg may link or call it; the
 * shipped library never does.
 *
 * Pinning status (what holds each function to the reference's equations):
 *   - gm_oracle_{sgd,adam,rmsprop,adagrad,adadelta,nadam}_step: pinned by
 *     tests/golden/optimizer_kat.json, which is produced by two evaluators
 *     that share no code with this file (an exact-rational evaluator that
 *     rounds every node to binary32 by integer arithmetic, and a numpy
 *     float32 ufunc chain), on the inputs the reference's own bridge tests
 *     use (cgo_bridge/optimizer_test.go:54-59) plus edge values, and by
 *     closed forms / invariants in tests/test_oracle_properties.py, among
 *     them checks that separate neighbouring formulas (epsilon inside or
 *     outside the root, mu at t or t + 1, the old or the new E[dx^2], decay
 *     into the update or into the gradient), each one shown to fail against
 *     this file with the corresponding line changed.
 *     The reference's tests assert no numerical output for these functions
 *     (they only log), so the equations are pinned, not Apple's MPSGraph bits.
 *   - gm_oracle_f32_to_f16 / gm_oracle_f16_to_f32: pinned exhaustively
 *     against numpy's float16 casts (all 65536 half patterns, boundary set).
 *     The bulk loops use inlined fast paths of both, equal to these functions
 *     on every bit pattern (gm_oracle_f16_fast_mismatches over all 2^32 / 2^16).
 *   - gm_oracle_adam_amp_step: PARITY UNPINNED against the reference: the
 *     reference holds no implementation of loss scaling, only constants
 *     (training/model_trainer.go:258-270) and prose
 *     (docs/tutorials/mixed-precision.md:610-629).  The semantics are defined
 *     here and pinned by a pure-Python brute-force state machine.  Its
 *     applied-step loop has an eight-lane form for hosts with AVX2 + F16C,
 *     held to the scalar loop bit for bit (gm_oracle_amp_vector_mismatches).
 */
#ifndef GM_ORACLE_H
#define GM_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Host scalars.  bridge_optimizer.m:398-399 (Adam), :2061-2066 (NAdam). */
void  gm_oracle_bias_corrections(float beta1, float beta2, int step, float *bc1, float *bc2);
float gm_oracle_nadam_mu_next(float beta1, int step);

/* One optimizer step over one flat fp32 tensor, in place.
 * nthreads <= 1: scalar loop on the calling thread; > 1: OpenMP static split
 * (elements are independent, so the result does not depend on nthreads). */

/* bridge_optimizer.m:160-357.  m may be NULL (vanilla path, :313-347). */
void gm_oracle_sgd_step(float *w, const float *g, float *m, size_t n,
                        float lr, float momentum, float weight_decay, int nesterov,
                        int nthreads);

/* bridge_optimizer.m:360-641.  step is the value optimizer/adam.go:183,225 passes
 * (StepCount after the pre-increment; first call uses 1). */
void gm_oracle_adam_step(float *w, const float *g, float *m, float *v, size_t n,
                         float lr, float beta1, float beta2, float eps, float weight_decay,
                         int step, int nthreads);

/* bridge_optimizer.m:691-951.  mom / gavg may be NULL when momentum == 0 /
 * centered == 0.  Unlike the reference (which never writes them back, :909-915)
 * the momentum and gradient-average states are persisted. */
void gm_oracle_rmsprop_step(float *w, const float *g, float *s, float *mom, float *gavg, size_t n,
                            float lr, float alpha, float eps, float weight_decay,
                            float momentum, int centered, int nthreads);

/* bridge_optimizer.m:1421-1588. */
void gm_oracle_adagrad_step(float *w, const float *g, float *s, size_t n,
                            float lr, float eps, float weight_decay, int nthreads);

/* bridge_optimizer.m:1708-1925. */
void gm_oracle_adadelta_step(float *w, const float *g, float *s, float *a, size_t n,
                             float rho, float eps, float weight_decay, int nthreads);

/* bridge_optimizer.m:2023-2280. */
void gm_oracle_nadam_step(float *w, const float *g, float *m, float *v, size_t n,
                          float lr, float beta1, float beta2, float eps, float weight_decay,
                          int step, int nthreads);

/* fp32 <-> fp16 casts, bridge_memory.m:361-377 (half(x): round to nearest
 * even, overflow to +-inf; float(h): exact).  Software bit manipulation, no
 * hardware conversion instruction. */
uint16_t gm_oracle_f32_to_f16(float x);
float    gm_oracle_f16_to_f32(uint16_t h);
/* Number of bit patterns in [first_bits, first_bits + count) on which the inlined fast forms of
 * the two conversions (used by the bulk loops) differ from the functions above: fp32 patterns
 * through f32 -> f16, or (halves != 0) fp16 patterns through f16 -> f32.  Must be 0. */
uint64_t gm_oracle_f16_fast_mismatches(uint64_t first_bits, uint64_t count, int halves, int nthreads);
void gm_oracle_convert_f32_to_f16(const float *src, uint16_t *dst, size_t n, int nthreads);
void gm_oracle_convert_f16_to_f32(const uint16_t *src, float *dst, size_t n, int nthreads);

/* Dynamic loss-scaling state.  Constants: training/model_trainer.go:258-270
 * (65536, x2, x0.5, 2000). */
typedef struct {
    float    scale;
    int32_t  growth_tracker;
    float    growth_factor;
    float    backoff_factor;
    int32_t  growth_interval;
    uint64_t step_count;      /* optimizer StepCount: advanced only by clean steps */
} gm_oracle_amp_state;

/* 1 if any fp16 element of any tensor is +-inf or NaN. */
int gm_oracle_amp_found_inf(const uint16_t *const *g16, const size_t *n, int num_tensors, int nthreads);

/* Mixed-precision Adam step over a tensor list.  Returns 1 when the step was
 * skipped (w, m, v, w16 and step_count untouched; scale *= backoff; tracker = 0),
 * else 0 (step_count++, g = float(g16) * (1.0f / scale), the Adam rule above,
 * w16 = half(w'), tracker++, and scale *= growth when tracker reaches the
 * interval).  The scale stays a normal finite number: a growth whose product exceeds
 * FLT_MAX and a backoff whose product falls below FLT_MIN are not applied (the
 * reference's tutorial: "scale = scale * 2 (up to maximum)",
 * docs/tutorials/mixed-precision.md:624; it names no value). */
int gm_oracle_adam_amp_step(float *const *w, const uint16_t *const *g16, float *const *m,
                            float *const *v, uint16_t *const *w16, const size_t *n, int num_tensors,
                            float lr, float beta1, float beta2, float eps, float weight_decay,
                            gm_oracle_amp_state *st, int nthreads);

/* The applied mixed-precision step has an eight-lane form for hosts with AVX2 and F16C (same
 * operations, one IEEE operation per lane each).  This runs both forms over n elements in
 * blocks of 64 and returns the number of blocks whose w / m / v / w16 differ in any bit, any
 * NaN counting as equal to any NaN (must be 0); UINT64_MAX when the host cannot run the vector form. */
uint64_t gm_oracle_amp_vector_mismatches(const float *w, const uint16_t *g16, const float *m, const float *v,
                                         size_t n, float lr, float beta1, float beta2, float eps,
                                         float weight_decay, float bc1, float bc2, float inv_scale);

/* L-BFGS step, cgo_bridge/bridge_optimizer.m:980-1321 (oracle_lbfgs.c states what is
 * reproduced).  s and y hold history_size * num_tensors tensors, entry [h * num_tensors + i];
 * rho and alpha are host arrays of history_size floats (the reference keeps each rho in a
 * 4-byte buffer of its own).  Returns 0, or -5 for history arguments out of range.
 *
 * Pinning status: the reference's tests assert no numerical output of this function
 * (optimizer/lbfgs_test.go checks construction, counters and error strings only).  The
 * statement order is pinned by tests/golden/lbfgs_kat.json, written by two independent
 * evaluators that must agree bit for bit (numpy float32 element ops with Python floats for
 * the fp64 tree; exact rational arithmetic rounded by integer arithmetic), by the
 * closed form w' = w + initial_step * g for an empty history, and, for GM_ORACLE_DOT_TREE,
 * by agreement with the exactly rounded dot product (math.fsum) to 1 ulp. */
enum { GM_ORACLE_DOT_REFERENCE = 0, GM_ORACLE_DOT_TREE = 1 };
float gm_oracle_lbfgs_dot(const float *const *a, const float *const *b, const size_t *n, int num_tensors,
                          int dot_mode, int per_tensor);
int gm_oracle_lbfgs_step(float *const *w, const float *const *g, float *const *old_g, float *const *dir,
                         float *const *s, float *const *y, float *rho, float *alpha,
                         const size_t *n, int num_tensors, int history_size, int history_count,
                         int history_index, float initial_step, int dot_mode, float *step_size);

#ifdef __cplusplus
}
#endif
#endif
