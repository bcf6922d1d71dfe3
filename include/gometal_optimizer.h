/*
 * Flat C view of the host-side mirror of go-metal's Go packages `optimizer` and `memory`
 * (C++ classes in go-metal_amd/host/, built into libgometal_hip.so).  The reference's host
 * layer is Go; no Go toolchain exists on the build machines, so the same objects are written
 * in C++ with the Go names, and this header lets C, ctypes or cgo callers drive them.
 *
 * Conventions: handles are opaque uintptr_t (0 = nil).  Functions that can fail return 0 on
 * success and -1 on error (constructors return 0); the error text, identical to the string
 * the Go method would return, is read with gmo_last_error() on the same thread.
 */
#ifndef GOMETAL_OPTIMIZER_H
#define GOMETAL_OPTIMIZER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

const char *gmo_last_error(void);
void gmo_free_string(char *s);

/* ---- package memory (memory/manager.go) ---- */
uintptr_t gmo_memory_manager_new(uintptr_t device);                 /* NewMemoryManager, manager.go:114 */
void      gmo_memory_manager_free(uintptr_t mm);
void      gmo_initialize_global_memory_manager(uintptr_t device);   /* manager.go:246 */
uintptr_t gmo_get_global_memory_manager(void);                      /* manager.go:253; 0 before initialisation */
uintptr_t gmo_allocate_buffer(uintptr_t mm, int size);              /* AllocateBuffer, manager.go:289 */
void      gmo_release_buffer(uintptr_t mm, uintptr_t buffer);       /* ReleaseBuffer, manager.go:299 */
int       gmo_find_pool_size(uintptr_t mm, int size);               /* findPoolSize, manager.go:172 */
int       gmo_calculate_max_pool_size(int buffer_size);             /* manager.go:210, byte-budget extension */
int       gmo_reference_max_pool_size(int buffer_size);             /* manager.go:210 cap table verbatim */
void      gmo_set_pool_byte_budget(size_t bytes);
/* BufferPool.Stats of the pools holding buffers of pool_size (buffers placed at a phase are pooled apart: available
 * and allocated are summed over those pools, max_size is one pool's cap); -1 if no such pool exists. */
int       gmo_pool_stats(uintptr_t mm, int pool_size, int *available, int *allocated, int *max_size);

/* ---- package optimizer ---- */
enum { GMO_SGD = 0, GMO_ADAM = 1, GMO_RMSPROP = 2, GMO_ADAGRAD = 3, GMO_ADADELTA = 4, GMO_NADAM = 5 };

/* Config values in declaration order of the Go config struct (bools as 0 / 1):
 *   SGD      LearningRate, Momentum, WeightDecay, Nesterov            (sgd.go:39-45)
 *   Adam     LearningRate, Beta1, Beta2, Epsilon, WeightDecay         (adam.go:42-48)
 *   RMSProp  LearningRate, Alpha, Epsilon, WeightDecay, Momentum, Centered (rmsprop.go:44-51)
 *   AdaGrad  LearningRate, Epsilon, WeightDecay                       (adagrad.go:35-39)
 *   AdaDelta Rho, Epsilon, WeightDecay                                (adadelta.go:36-40)
 *   Nadam    LearningRate, Beta1, Beta2, Epsilon, WeightDecay         (nadam.go:38-44) */
int gmo_default_config(int kind, float config[6]);                   /* Default<Kind>Config(); returns the field count */

/* New<Kind>Optimizer(config, weightShapes, memoryManager, device).  shape_dims holds the
 * dimensions of all tensors back to back, shape_ndims[i] the rank of tensor i. */
uintptr_t gmo_optimizer_new(int kind, const float *config, const int *shape_dims, const int *shape_ndims,
                            int num_weights, uintptr_t memory_manager, uintptr_t device);
void gmo_optimizer_free(uintptr_t opt);                              /* destroys the object (after Cleanup) */

/* optimizer.Optimizer (interface.go:13-43) */
int      gmo_set_weight_buffers(uintptr_t opt, const uintptr_t *weight_buffers, int n);
int      gmo_step(uintptr_t opt, const uintptr_t *gradient_buffers, int n);
uint64_t gmo_get_step_count(uintptr_t opt);
void     gmo_update_learning_rate(uintptr_t opt, float lr);
void     gmo_set_command_pool(uintptr_t opt, uintptr_t command_pool);
void     gmo_cleanup(uintptr_t opt);
/* GetState() as the JSON encoding/json would write (caller frees with gmo_free_string); NULL on error. */
char    *gmo_get_state_json(uintptr_t opt);
/* LoadState(state) with state decoded from JSON (every number becomes a float64, as in Go). */
int      gmo_load_state_json(uintptr_t opt, const char *json);
/* Decodes an OptimizerState document and encodes it again (caller frees with gmo_free_string);
 * NULL with gmo_last_error() set when the document does not decode.  No optimizer object and no
 * GPU are involved: the serializer on its own, for tools and tests. */
char    *gmo_state_json_normalize(const char *json);
/* The same through the reference's JSON checkpoint document (checkpoints/checkpoint.go:38-52):
 * GetState() wrapped as {"model_spec", "weights", "training_state", "optimizer_state", "metadata"},
 * and LoadState() from the "optimizer_state" member of such a document. */
char    *gmo_get_checkpoint_json(uintptr_t opt);
int      gmo_load_checkpoint_json(uintptr_t opt, const char *json);

/* Field access for tests: hyper-parameter by Go field name ("LearningRate", "Beta1", ...; bools
 * as 0 / 1); NaN if the optimizer has no such field. */
float     gmo_get_field(uintptr_t opt, const char *name);
/* Handle of state buffer `index` of one kind: "momentum", "variance", "squared_grad_avg",
 * "gradient_avg", "squared_update_avg"; 0 if absent.  Adam also answers "weight" (the buffer that
 * holds the current fp32 weights: the caller's own unless the ping-pong step has made the shadow set current). */
uintptr_t gmo_state_buffer(uintptr_t opt, const char *state_type, int index);
int       gmo_uses_pooling(uintptr_t opt);
void      gmo_set_log_progress(uintptr_t opt, int on);               /* AdaGrad / AdaDelta print every 10 steps */

/* Adam mixed precision (no counterpart in the reference's optimizer package) */
int   gmo_enable_mixed_precision(uintptr_t adam, float initial_scale, float growth_factor, float backoff_factor,
                                 int growth_interval);
/* EnablePingPong: StepAMP / StepAMPAsync become the one-pass step over two sets of weights and moments
 * (execute_adam_amp_step_fused); call after SetWeightBuffers and EnableMixedPrecision.  The current fp32
 * weights are then gmo_state_buffer(adam, "weight", i); gmo_current_set tells which set that is (0: the
 * caller's buffers, 1: the shadow set; -1 on error). */
int   gmo_enable_ping_pong(uintptr_t adam);
int   gmo_current_set(uintptr_t adam);
int   gmo_step_amp(uintptr_t adam, const uintptr_t *gradient16_buffers, const uintptr_t *weight16_buffers, int n,
                   int *skipped);
int   gmo_step_amp_async(uintptr_t adam, const uintptr_t *gradient16_buffers, const uintptr_t *weight16_buffers,
                         int n);                     /* StepAMPAsync: no wait, no result */
int   gmo_sync_amp(uintptr_t adam, uint64_t *skipped_steps);   /* SyncAMP: waits, refreshes StepCount / scale */
float gmo_loss_scale(uintptr_t adam);
int   gmo_growth_tracker(uintptr_t adam);

/* ---- optimizer/lbfgs.go: LBFGSOptimizerState (not an optimizer.Optimizer in the reference
 * either: Step also takes the current loss).  Errors as above: -1 / 0 and gmo_last_error(). ---- */
void      gmo_lbfgs_default_config(int *history_size, float *line_search_tol, int *max_line_search, float *c1,
                                   float *c2, float *initial_step);            /* DefaultLBFGSConfig, lbfgs.go:55 */
uintptr_t gmo_lbfgs_new(int history_size, float line_search_tol, int max_line_search, float c1, float c2,
                        float initial_step, const int *dims, const int *ndims, int num_weights,
                        uintptr_t memory_manager, uintptr_t device);           /* NewLBFGSOptimizer, lbfgs.go:67 */
void      gmo_lbfgs_free(uintptr_t lbfgs);
int       gmo_lbfgs_set_weight_buffers(uintptr_t lbfgs, const uintptr_t *buffers, int n);   /* lbfgs.go:235 */
int       gmo_lbfgs_step(uintptr_t lbfgs, const uintptr_t *gradient_buffers, int n, float current_loss); /* :245 */
void      gmo_lbfgs_set_command_pool(uintptr_t lbfgs, uintptr_t pool);         /* lbfgs.go:304 */
int       gmo_lbfgs_uses_pooling(uintptr_t lbfgs);
uint64_t  gmo_lbfgs_get_step(uintptr_t lbfgs);                                 /* lbfgs.go:310 */
void      gmo_lbfgs_get_stats(uintptr_t lbfgs, uint64_t *step, int *history_size, int *history_used,
                              float *prev_loss);                               /* GetStats, lbfgs.go:315 */
void      gmo_lbfgs_history(uintptr_t lbfgs, int *count, int *index, float *last_step_size);
void      gmo_lbfgs_cleanup(uintptr_t lbfgs);                                  /* lbfgs.go:325 */
int       gmo_lbfgs_update_learning_rate(uintptr_t lbfgs, float lr);           /* always an error, lbfgs.go:330 */
void      gmo_lbfgs_set_log_progress(uintptr_t lbfgs, int on);
int       gmo_lbfgs_buffer_size(uintptr_t lbfgs, int index);                   /* bytes; -1 if out of range */
/* which: "s", "y" (history, index), "rho" (history), "alpha", "old_gradient", "search_dir", "weight" (index) */
uintptr_t gmo_lbfgs_buffer(uintptr_t lbfgs, const char *which, int history, int index);

/* ---- memory.Tensor (memory/tensor.go): reference-counted tensor over a pooled buffer.
 * dtype codes: Float32 = 0, Int32 = 1, Float16 = 2, Int8 = 3 (tensor.go:10-17). ---- */
uintptr_t gmo_tensor_new(const int *shape, int ndims, int dtype, int device_type);   /* NewTensor, tensor.go:41 */
uintptr_t gmo_tensor_retain(uintptr_t tensor);                 /* Retain; 0 if already released */
void      gmo_tensor_release(uintptr_t tensor);                /* Release, tensor.go:78 */
void      gmo_tensor_free(uintptr_t tensor);                   /* destroys the released object */
uintptr_t gmo_tensor_buffer(uintptr_t tensor);                 /* MetalBuffer */
int       gmo_tensor_size(uintptr_t tensor);                   /* Size, bytes */
int       gmo_tensor_ref_count(uintptr_t tensor);              /* RefCount */
int       gmo_tensor_dtype(uintptr_t tensor);
uintptr_t gmo_tensor_convert_to(uintptr_t tensor, int dtype);  /* ConvertTo, tensor.go:166; same handle retained if the type matches */
int       gmo_tensor_copy_float32_data(uintptr_t tensor, const float *data, int n);   /* tensor.go:189 */
int       gmo_tensor_to_float32_slice(uintptr_t tensor, float *out, int capacity);    /* tensor.go:341; returns the element count */
int       gmo_tensor_copy_from(uintptr_t dst, uintptr_t src);  /* CopyFrom, tensor.go:248 */
char     *gmo_tensor_string(uintptr_t tensor);                 /* String, tensor.go:363-366; caller frees with gmo_free_string */
int       gmo_calculate_size(const int *shape, int ndims, int dtype);                 /* tensor.go:137 */

/* engine.ExecuteStepWithPrecomputedGradients (engine/training_engine.go:100-147) for any optimizer:
 * tensors -> buffer handles -> SetWeightBuffers -> Step.  A 0 entry is a nil tensor. */
int gmo_execute_step_with_precomputed_gradients(uintptr_t opt, const uintptr_t *weight_tensors, int num_weights,
                                                const uintptr_t *gradient_tensors, int num_gradients);

/* ---- learning-rate schedules (training/scheduler.go).  kind: 0 StepLR(a = stepSize, b = gamma),
 * 1 ExponentialLR(b = gamma), 2 CosineAnnealingLR(a = tMax, b = etaMin),
 * 3 ReduceLROnPlateau(a = patience, b = factor, c = threshold, mode "min" / "max"), 4 constant. ---- */
uintptr_t   gmo_scheduler_new(int kind, int a, double b, double c, const char *mode);
void        gmo_scheduler_free(uintptr_t scheduler);
double      gmo_scheduler_get_lr(uintptr_t scheduler, int epoch, int step, double base_lr);   /* GetLR */
double      gmo_scheduler_plateau_step(uintptr_t scheduler, double metric, double current_lr);/* Step (kind 3 only; else NaN) */
const char *gmo_scheduler_name(uintptr_t scheduler);                                          /* GetName */
/* GetLR followed by the optimizer's UpdateLearningRate(float32(lr)), the fan-out of
 * engine/model_engine.go:2332-2390.  Returns the rate that was set. */
double      gmo_scheduler_apply(uintptr_t scheduler, uintptr_t opt, int epoch, int step, double base_lr);

/* helpers (interface.go:56-76, adam.go:142-148) */
float gmo_pow(float x, float y);                           /* pow, optimizer/adam.go:236-251 */
int gmo_extract_buffer_index(const char *name);
int gmo_calculate_tensor_size(const int *dims, int ndims);
/* state_helpers.go:53-74 on a JSON object of parameters (numbers decode to float64, as through
 * encoding/json): the value under key when it has the type the helper accepts, else the default. */
float    gmo_extract_float32_param(const char *parameters_json, const char *key, float default_value);
int      gmo_extract_bool_param(const char *parameters_json, const char *key, int default_value);
uint64_t gmo_extract_uint64_param(const char *parameters_json, const char *key, uint64_t default_value);
/* validateStateType, interface.go:79-84.  0, or -1 with the message in gmo_last_error(). */
int gmo_validate_state_type(const char *optimizer_type, const char *state_type);
/* restoreBufferState, state_helpers.go:34-50: 0, or -1 with the Go error string. */
int gmo_restore_buffer_state(uintptr_t buffer, const float *data, int num_elements, int buffer_size,
                             const char *name);
/* extractBufferState, state_helpers.go:14-32: 1 when a tensor came back (its num_elements floats
 * in data), 0 for a nil buffer (no tensor and no error), -1 with the Go error string. */
int gmo_extract_buffer_state(uintptr_t buffer, int buffer_size, const char *name, const char *state_type,
                             float *data, int num_elements);

#ifdef __cplusplus
}
#endif
#endif
