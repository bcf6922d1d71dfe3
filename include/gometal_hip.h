/*
 * C ABI of libgometal_hip.so: the MI355X (gfx950) replacement for the part of
 * go-metal's Objective-C bridge that the `optimizer` package reaches:
 * cgo_bridge/bridge_optimizer.m (update rules), cgo_bridge/bridge_memory.m
 * (buffers) and the device / queue subset of cgo_bridge/bridge_device.m.
 *
 * Every function in the first part keeps the name, argument order, argument
 * meaning and return-code convention of the C prototype that
 * cgo_bridge/bridge.go declares in its cgo preamble, so the Go wrappers in
 * bridge.go bind to this library unchanged.  Handles are opaque uintptr_t:
 * a buffer handle IS the device address of the allocation (kernels take it
 * without indirection); a device handle is a pointer to a process-lifetime
 * context; 0 is the nil handle everywhere.  Return 0 = success, negative =
 * error (per-function tables below).  No function throws or aborts.
 *
 * Ordering: all work is enqueued on one HIP stream per device context.  The
 * update entry points return after enqueueing; every entry point that hands
 * data to the host (copy_metal_buffer_to_*), and copy_buffer_to_buffer_sync,
 * synchronise that stream before returning, so the host observes the same
 * values it would after the reference's blocking calls.
 *
 * Sizes: buffer_sizes[] are BYTES of the fp32 weight tensor, as in the
 * reference (numel = size / 4).  They cross this ABI as C int, so one tensor
 * is limited to 2 GiB - 1 (cgo_bridge/bridge.go:920, 1003).
 */
#ifndef GOMETAL_HIP_H
#define GOMETAL_HIP_H

#include <stdbool.h>
#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------ */
/* Device and queue.  cgo_bridge/bridge_device.m:87-107, 901-925;            */
/* prototypes cgo_bridge/bridge.go:57-60, 247-248.                           */
/* ------------------------------------------------------------------------ */

/* Returns a handle to the context of HIP device 0 (created on first use, kept
 * until the process ends, reference counted), or 0 when no GPU is usable.
 * All handles alias the same GPU, as MTLCreateSystemDefaultDevice does. */
uintptr_t create_metal_device(void);
/* Drops one reference.  Buffers, streams and pooled memory reachable through
 * other handles stay valid (memory/manager.go:246-250 keeps the first handle). */
void destroy_metal_device(uintptr_t device);
/* 0 when device is 0 (bridge_device.m:903-906); else an ordering token for the
 * context's stream. */
uintptr_t create_command_queue(uintptr_t device);
void release_command_queue(uintptr_t command_queue);

/* ------------------------------------------------------------------------ */
/* Buffers.  cgo_bridge/bridge_memory.m; prototypes bridge.go:75-77, 110-137. */
/* ------------------------------------------------------------------------ */

/* bridge_memory.m:4-42.  size <= 0 or device 0 -> 0.  The length is rounded up
 * to 16 bytes (:28); the address is 256-byte aligned.  device_type 0=CPU
 * 1=GPU 2=PersistentGPU (bridge.go:623-629) all map to HBM. */
uintptr_t allocate_metal_buffer(uintptr_t device, int size, int device_type);
/* bridge_memory.m:45-55.  0 is ignored. */
void deallocate_metal_buffer(uintptr_t buffer);
/* bridge_memory.m:163-188.  -1: nil device or buffer; -5: HIP error. */
int zero_metal_buffer(uintptr_t device, uintptr_t buffer, int size);
/* bridge_memory.m:58-160; same effect as zero_metal_buffer here. */
int zero_metal_buffer_mpsgraph(uintptr_t device, uintptr_t buffer, int size);
/* bridge_memory.m:191-218.  -1: nil buffer / NULL data / size <= 0; -3: the range exceeds
 * the allocation (buffers of this library only; the reference does not check); -4: HIP error.
 * The host array is ordinary (pageable) memory.  Both directions return once the data has
 * arrived; copies of 8 MiB and more are staged through pinned slots on two lanes, one of them
 * driven by a helper thread that lives for the call (about 49 GB/s each way on MI355X hosts). */
int copy_data_to_metal_buffer(uintptr_t buffer, void *data, int size);
/* bridge_memory.m:221-258.  -1: nil / NULL / n <= 0. */
int copy_float32_array_to_metal_buffer(uintptr_t buffer, float *data, int num_elements);
int copy_int32_array_to_metal_buffer(uintptr_t buffer, int *data, int num_elements);
/* bridge_memory.m:261-320.  Synchronises the stream first.  -1 / -3 / -4 as above. */
int copy_metal_buffer_to_float32_array(uintptr_t buffer, float *data, int num_elements);
int copy_metal_buffer_to_int32_array(uintptr_t buffer, int *data, int num_elements);
/* bridge_memory.m:323-423.  Element count = product of shape[0..num_dims).
 * Type codes from memory/tensor.go:12-17: Float32 = 0, Float16 = 2.
 * fp32->fp16 rounds to nearest even and overflows to +-inf; fp16->fp32 is
 * exact.  -1: nil buffers / NULL shape / num_dims <= 0; -2: nil device;
 * -3: any pair other than 0->2 or 2->0; -4: HIP error; -5: the element count exceeds
 * one of the allocations (buffers of this library only). */
int convert_tensor_type(uintptr_t src_buffer, uintptr_t dst_buffer, int *shape, int num_dims,
                        int src_type, int dst_type, uintptr_t device);
/* bridge_memory.m:504-592.  -1: nil handle; -2: size <= 0 or negative offset;
 * -4 / -5: source / destination range exceeds the allocation; -10: HIP error. */
int copy_buffer_to_buffer_sync(uintptr_t src_buffer, uintptr_t dst_buffer, int src_offset,
                               int dst_offset, int size);

/* ------------------------------------------------------------------------ */
/* Optimizer steps.  cgo_bridge/bridge_optimizer.h; prototypes                */
/* bridge.go:79-123, 277-413.  Arrays have num_weights entries of buffer      */
/* handles; they are read during the call and not retained.  Weights and      */
/* states are updated in place; gradients are read only.                      */
/* Common codes: -1 device 0 (checked first, nothing else touched);           */
/* -3 no usable GPU stream; others per function.  A tensor whose allocation   */
/* (when the handle is one of this library's) is shorter than buffer_sizes[i] */
/* is skipped, as the reference does (bridge_optimizer.m:427-436).            */
/* No C++ exception crosses this boundary: one caught inside an entry point   */
/* (a failed host allocation, say) returns the code the reference returns     */
/* from its own @catch block: the "HIP error" code of each function below     */
/* (-13 for execute_adam_step_mpsgraph_pooled, .m:683-686), with the reason   */
/* in gm_last_error().                                                        */
/* ------------------------------------------------------------------------ */

/* bridge_optimizer.h:11-23 / .m:160-357.  momentum_buffers may be NULL or hold
 * 0 entries: those tensors take the vanilla path.  A tensor whose weight or
 * gradient handle is 0 is skipped (.m:199-202).  -10: HIP error. */
int execute_sgd_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                              uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                              int num_weights, int *buffer_sizes, float learning_rate,
                              float momentum, float weight_decay, int nesterov, int step_count);

/* bridge_optimizer.h:26-40 / .m:360-641.  -4: a weight / gradient / momentum /
 * variance handle is 0 (nothing is updated); -6: HIP error. */
int execute_adam_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                               uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                               uintptr_t *variance_buffers, int num_weights, int *buffer_sizes,
                               float learning_rate, float beta1, float beta2, float epsilon,
                               float weight_decay, int step_count);

/* bridge_optimizer.h:58-73 / .m:645-688.  The reference's body is a stub that
 * validates its handles and updates nothing (and optimizer/adam.go:191-227
 * never calls it).  Here: -1 device 0, -15 command_pool 0, otherwise the same
 * step as execute_adam_step_mpsgraph. */
int execute_adam_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                      uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                                      uintptr_t *variance_buffers, int num_weights,
                                      int *buffer_sizes, float learning_rate, float beta1,
                                      float beta2, float epsilon, float weight_decay,
                                      int step_count, uintptr_t command_pool);

/* bridge_optimizer.h:76-92 / .m:691-951.  -4: weight / gradient / squared-avg
 * handle 0; -5: momentum > 0 with a 0 momentum handle; -6: centered with a 0
 * gradient-average handle; -8: HIP error.  The momentum and gradient-average
 * states ARE written back (the reference omits them from its feeds and
 * targets, .m:909-915, so its momentum / centered variants cannot run). */
int execute_rmsprop_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                  uintptr_t *gradient_buffers,
                                  uintptr_t *squared_grad_avg_buffers,
                                  uintptr_t *momentum_buffers, uintptr_t *gradient_avg_buffers,
                                  int num_weights, int *buffer_sizes, float learning_rate,
                                  float alpha, float epsilon, float weight_decay, float momentum,
                                  bool centered, int step_count);

/* bridge_optimizer.h:97-120 / .m:1421-1674.  A tensor with a 0 handle is
 * skipped.  -8: HIP error.  _pooled ignores command_pool (0 or not). */
int execute_adagrad_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                  uintptr_t *gradient_buffers,
                                  uintptr_t *squared_grad_avg_buffers, int num_weights,
                                  int *buffer_sizes, float learning_rate, float epsilon,
                                  float weight_decay);
int execute_adagrad_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                         uintptr_t *gradient_buffers,
                                         uintptr_t *squared_grad_avg_buffers, int num_weights,
                                         int *buffer_sizes, float learning_rate, float epsilon,
                                         float weight_decay, uintptr_t command_pool);

/* bridge_optimizer.h:125-150 / .m:1708-2019.  As AdaGrad. */
int execute_adadelta_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                   uintptr_t *gradient_buffers,
                                   uintptr_t *squared_grad_avg_buffers,
                                   uintptr_t *squared_update_avg_buffers, int num_weights,
                                   int *buffer_sizes, float rho, float epsilon,
                                   float weight_decay);
int execute_adadelta_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                          uintptr_t *gradient_buffers,
                                          uintptr_t *squared_grad_avg_buffers,
                                          uintptr_t *squared_update_avg_buffers,
                                          int num_weights, int *buffer_sizes, float rho,
                                          float epsilon, float weight_decay,
                                          uintptr_t command_pool);

/* bridge_optimizer.h:207-221 / .m:2023-2280.  -4: a handle is 0; -6: HIP error. */
int execute_nadam_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                uintptr_t *gradient_buffers, uintptr_t *momentum_buffers,
                                uintptr_t *variance_buffers, int num_weights, int *buffer_sizes,
                                float learning_rate, float beta1, float beta2, float epsilon,
                                float weight_decay, int step_count);

/* bridge_optimizer.h:155-203 / .m:980-1393; prototypes bridge.go:296-343.  One L-BFGS step
 * with the statement order of the reference's loop nest: q = -g; two-loop recursion over
 * the history pairs whose |rho| >= 1e-10 (H0 = I); p = -r; x += initial_step * p (no line
 * search: c1, c2, max_line_search and the losses are ignored, as in the reference);
 * old_g = g; s[history_index] = initial_step * p; and, when history_count > 0,
 * y[prev] = g - old_g and rho[prev] = 1 / (s[prev] . y[prev]) (0 when |s.y| <= 1e-10) for
 * prev = history_index - 1.  In that order old_g already equals g, so y[prev] is g - g
 * (+0, NaN for a non-finite g) and rho[prev] is 0: that is what the reference's code yields
 * and what this call writes, without summing s[prev] . y[prev].  s_vectors_flat / y_vectors_flat hold history_size * num_weights
 * handles, entry [h * num_weights + i]; rho_buffers holds history_size handles of 4-byte
 * buffers; alpha_buffer holds history_size floats.  *step_size = initial_step.
 * Dot products are exact fp64 products summed by a fixed tree and rounded once to fp32
 * (the reference keeps a running fp32 sum in element order).
 * The call reads back which pairs are valid (it synchronises when history_count > 0); the
 * passes themselves are asynchronous on the device's stream.
 * -1 device 0; -3 no GPU; -5 history arguments out of range; -8 a handle or array is nil,
 * a buffer of this library is shorter than its tensor, or a HIP error (the reference's
 * exception code). */
int execute_lbfgs_step_mpsgraph(uintptr_t device, uintptr_t *weight_buffers,
                                uintptr_t *gradient_buffers, uintptr_t *old_gradient_buffers,
                                uintptr_t *search_dir_buffers, uintptr_t *s_vectors_flat,
                                uintptr_t *y_vectors_flat, uintptr_t *rho_buffers,
                                uintptr_t alpha_buffer, int num_weights, int *buffer_sizes,
                                int history_size, int history_count, int history_index,
                                float initial_step, float c1, float c2, int max_line_search,
                                float current_loss, float prev_loss, float *step_size);
/* bridge_optimizer.h:179-203 / .m:1324-1393: the same step (the pool is not used). */
int execute_lbfgs_step_mpsgraph_pooled(uintptr_t device, uintptr_t *weight_buffers,
                                       uintptr_t *gradient_buffers,
                                       uintptr_t *old_gradient_buffers,
                                       uintptr_t *search_dir_buffers, uintptr_t *s_vectors_flat,
                                       uintptr_t *y_vectors_flat, uintptr_t *rho_buffers,
                                       uintptr_t alpha_buffer, int num_weights, int *buffer_sizes,
                                       int history_size, int history_count, int history_index,
                                       float initial_step, float c1, float c2,
                                       int max_line_search, float current_loss, float prev_loss,
                                       uintptr_t command_pool, float *step_size);

/* ------------------------------------------------------------------------ */
/* Additions (no counterpart in the reference's C ABI).                       */
/* ------------------------------------------------------------------------ */

/* Blocks until everything enqueued on the device's stream has finished.
 * -1: device 0; -3: no GPU; -10: HIP error (a kernel fault surfaces here). */
int gm_synchronize(uintptr_t device);

/* Ordering against a caller's own HIP stream without a host wait (hip_stream is a hipStream_t;
 * NULL is the legacy default stream).  gm_wait_for_stream: work the library enqueues after the
 * call starts only when everything enqueued on hip_stream before the call has finished (use it
 * after producing gradients on that stream).  gm_signal_stream: work enqueued on hip_stream after
 * the call starts only when everything the library has enqueued so far has finished (use it
 * before consuming updated weights on that stream).  Codes as gm_synchronize. */
int gm_wait_for_stream(uintptr_t device, void *hip_stream);
int gm_signal_stream(uintptr_t device, void *hip_stream);

/* Message of the most recent failure on the calling thread ("" if none). */
const char *gm_last_error(void);

/* Allocation length in bytes of one of this library's buffers; 0 if unknown. */
size_t gm_buffer_length(uintptr_t buffer);

/* Host-side step scalars, exactly as the update entry points compute them
 * (bridge_optimizer.m:398-399, :2066). */
void  gm_bias_corrections(float beta1, float beta2, int step_count, float *bc1, float *bc2);
float gm_nadam_mu_next(float beta1, int step_count);

/* Dynamic loss-scale state for the mixed-precision Adam step, resident on the
 * device.  Defaults in the reference's trainer config: 65536, 2.0, 0.5, 2000
 * (training/model_trainer.go:258-270).  The reference itself never unscales,
 * checks or rescales (it only stores those constants); this step is the
 * algorithm its tutorial describes (docs/tutorials/mixed-precision.md:610-629). */
uintptr_t gm_amp_state_create(uintptr_t device, float init_scale, float growth_factor,
                              float backoff_factor, int growth_interval);
void gm_amp_state_destroy(uintptr_t amp_state);
/* Reads / overwrites scale and the clean-step counter (checkpointing). */
int gm_amp_state_get(uintptr_t amp_state, float *scale, int *growth_tracker);
int gm_amp_state_set(uintptr_t amp_state, float scale, int growth_tracker);
/* As gm_amp_state_get, plus the number of steps applied (the optimizer's StepCount as the
 * device counts it: +1 per clean step) and dropped since creation / the last
 * gm_amp_state_set_step_count.  Waits for every step in flight.  Pointers may be NULL. */
int gm_amp_state_query(uintptr_t amp_state, float *scale, int *growth_tracker, int *applied_steps,
                       int *skipped_steps);
/* The largest number of asynchronous steps that were still unconfirmed when another one was
 * issued (0 to 6): tells whether a caller actually ran ahead of the device.  -16: nil state. */
int gm_amp_state_max_in_flight(uintptr_t amp_state);
/* Sets the device's applied-step count (call when the optimizer's StepCount is set by other
 * means: construction, LoadState).  -5: negative count. */
int gm_amp_state_set_step_count(uintptr_t amp_state, int applied_steps);

/* One mixed-precision Adam step over the whole tensor list.
 *   gradient16_buffers: fp16 gradients of the SCALED loss (read only)
 *   weight/momentum/variance_buffers: fp32 master state, updated in place
 *   weight16_buffers: fp16 copy of the updated weights (entries may be 0 or
 *                     the array NULL: no copy is emitted for those tensors)
 *   buffer_sizes: bytes of the fp32 weight tensor (numel = size / 4)
 *   step_count: the bias-correction step to use IF the step is applied
 * If any gradient element of any tensor is +-inf or NaN the step is skipped:
 * no buffer is written, scale *= backoff, clean-step counter = 0, *skipped = 1.
 * Otherwise g = float(g16) * (1.0f / scale), the Adam rule of
 * execute_adam_step_mpsgraph, w16 = half(w'), counter++, and scale *= growth
 * when the counter reaches growth_interval; *skipped = 0.
 * The call returns once the step's outcome is known (it reports *skipped): the check has
 * finished and the update, if any, is launched; like the fp32 steps the update itself completes
 * on the library's stream, ahead of whatever is enqueued there next, and every call that hands
 * data to the host waits for it (gm_synchronize waits explicitly).  scale_out /
 * growth_tracker_out (may be NULL) receive the state after the step.
 * -1 device 0; -3 no GPU; -4 a required handle is 0; -6 HIP error; -16 amp_state 0. */
int execute_adam_amp_step(uintptr_t device, uintptr_t *weight_buffers,
                          uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                          uintptr_t *variance_buffers, uintptr_t *weight16_buffers,
                          int num_weights, int *buffer_sizes, float learning_rate, float beta1,
                          float beta2, float epsilon, float weight_decay, int step_count,
                          uintptr_t amp_state, int *skipped, float *scale_out,
                          int *growth_tracker_out);

/* execute_adam_amp_step without the read-back: enqueues the step and returns.  The bias-correction
 * step is taken from the device's own applied-step count (gm_amp_state_set_step_count, +1 per
 * clean step), so a dropped step needs no host decision: the host sends the corrections for
 * every count that the steps still in flight leave possible (at most 8) and the kernel picks.
 * Up to 7 steps run ahead of the host; the call waits for the oldest one beyond that.
 * Results and counters are read with gm_amp_state_query (which waits).  Buffers, arithmetic
 * and results are exactly those of the synchronous step.  Codes as execute_adam_amp_step. */
int execute_adam_amp_step_async(uintptr_t device, uintptr_t *weight_buffers,
                                uintptr_t *gradient16_buffers, uintptr_t *momentum_buffers,
                                uintptr_t *variance_buffers, uintptr_t *weight16_buffers,
                                int num_weights, int *buffer_sizes, float learning_rate,
                                float beta1, float beta2, float epsilon, float weight_decay,
                                uintptr_t amp_state);

/* The mixed-precision Adam step in ONE pass over ping-pong state.  Weights, momentum and variance
 * exist twice, as sets A and B of equal shape; one set is current (set A after
 * gm_amp_state_create).  The step reads the current set and the fp16 gradients, checks the
 * gradients as it reads them, and writes the OTHER set plus the fp16 weight copy; only if no
 * gradient was +-inf or NaN does the written set become the current one.  A dropped step
 * therefore leaves the current set untouched without any buffer having been read twice: 28 bytes
 * move per parameter, against 30 for execute_adam_amp_step, which updates in place and must check
 * every gradient before it may write anything.  Arithmetic, skip decision, loss-scale sequence and
 * step counting are those of execute_adam_amp_step; the current set after any sequence of steps
 * equals, bit for bit, what the in-place step leaves in its buffers.
 *   - Which set is current: *current_set_out (0 = A, 1 = B) after the synchronous step,
 *     gm_amp_state_current_set (which waits) at any time.  The other set holds scratch.
 *   - weight16_buffers (may be NULL, entries may be 0) receives half(w') speculatively; after a
 *     dropped step a repair pass rewrites it as half(current weights).  Callers keep the invariant
 *     "the fp16 copy is half of the current weights" from the start (convert_tensor_type once
 *     before the first step); with it a dropped step leaves the copy bit-identical as well.
 *   - Both sets must hold every tensor (a buffer shorter than its tensor in one set only: -4).
 * The _async form enqueues and returns, exactly as execute_adam_amp_step_async does.
 * Codes as execute_adam_amp_step. */
int execute_adam_amp_step_fused(uintptr_t device, uintptr_t *weight_a, uintptr_t *momentum_a, uintptr_t *variance_a,
                                uintptr_t *weight_b, uintptr_t *momentum_b, uintptr_t *variance_b,
                                uintptr_t *gradient16_buffers, uintptr_t *weight16_buffers, int num_weights,
                                int *buffer_sizes, float learning_rate, float beta1, float beta2, float epsilon,
                                float weight_decay, int step_count, uintptr_t amp_state, int *skipped,
                                float *scale_out, int *growth_tracker_out, int *current_set_out);
int execute_adam_amp_step_fused_async(uintptr_t device, uintptr_t *weight_a, uintptr_t *momentum_a,
                                      uintptr_t *variance_a, uintptr_t *weight_b, uintptr_t *momentum_b,
                                      uintptr_t *variance_b, uintptr_t *gradient16_buffers,
                                      uintptr_t *weight16_buffers, int num_weights, int *buffer_sizes,
                                      float learning_rate, float beta1, float beta2, float epsilon,
                                      float weight_decay, uintptr_t amp_state);
/* 0 when set A holds the current weights and moments of the ping-pong step, 1 when set B does.
 * Waits for every step in flight.  -16: nil state; -6: HIP error. */
int gm_amp_state_current_set(uintptr_t amp_state);
/* Tells a loss-scale state which set holds the current weights and moments (0: A, 1: B): for a state
 * created anew over ping-pong buffers that are already in use.  Waits for every step in flight.
 * -16: nil state; -5: not 0 or 1; -6: HIP error.  No counterpart in the reference. */
int gm_amp_state_set_current_set(uintptr_t amp_state, int current_set);

/* allocate_metal_buffer with a say in where the buffer starts: the handle's address is congruent to
 * phase_bytes modulo 2 MiB (phase_bytes: a multiple of 256 below 2 MiB).  No counterpart in the
 * reference.  Buffers that start at the same phase put element i of each of them on the same HBM
 * channel; the optimizers place their state buffers at phases of their own (512 KiB, 1.5 MiB, 1 MiB
 * for the first, second and third state of a tensor), which is worth a point of bandwidth for
 * Adam over the 1.012B-parameter list.  Requests under 1 MiB ignore the phase; larger ones cost
 * 2 MiB more than their size.  The handle is freed with deallocate_metal_buffer and has the
 * length `size` for every range check.  0 on failure, like allocate_metal_buffer. */
uintptr_t gm_allocate_buffer_phased(uintptr_t device, int size, int device_type, int phase_bytes);

/* execute_adam_step_mpsgraph for callers that cannot allocate.  No counterpart in the reference:
 * it exists for code under HIP graph capture, tight serving loops and harnesses that forbid
 * hipMalloc.  Same arguments, arithmetic, update kernel and results as execute_adam_step_mpsgraph;
 * the chunk table lives in a __device__ array of the library (2 MiB per GPU, held until the
 * process ends) and is written by a kernel from tensor records passed as kernel arguments, so the
 * call performs no hipMalloc, hipFree, copy or other allocating routine and never waits for the
 * device.  Limits: 4096 tensors and 32768 chunk descriptors (about 2.1e9 parameters in chunks of
 * 65536 elements); beyond them -17 and a message in gm_last_error, nothing launched.  Every call on
 * a GPU rewrites that GPU's one table: calls are ordered on the library's stream, and calls that
 * overlap on one GPU by any other means race.  Under graph capture the call's scalars (learning rate, the
 * bias corrections of step_count) and the handle records travel as kernel arguments and are frozen
 * into the captured nodes: a replay repeats THAT step's corrections, so capture per step count or set
 * the nodes' kernel parameters before each replay (no test here exercises capture).
 * -1 device 0; -3 no GPU; -4 a required handle is 0 (nothing updated); -6 HIP error; -17 over the limits. */
int execute_adam_step_noalloc(uintptr_t device, uintptr_t *weight_buffers, uintptr_t *gradient_buffers,
                              uintptr_t *momentum_buffers, uintptr_t *variance_buffers, int num_weights,
                              int *buffer_sizes, float learning_rate, float beta1, float beta2,
                              float epsilon, float weight_decay, int step_count);

/* The dot product of two tensor lists exactly as the L-BFGS step forms it (fp64 tree,
 * one rounding to fp32).  Synchronises.  Codes as execute_lbfgs_step_mpsgraph. */
int gm_lbfgs_dot(uintptr_t device, uintptr_t *a_buffers, uintptr_t *b_buffers, int num_tensors,
                 int *buffer_sizes, float *result);

/* Diagnostics of the plan cache behind the multi-tensor steps: chunk tables laid out so far
 * (a step whose list and handles were seen before builds none), table slots allocated so far
 * (device table + pinned host twin; dropped plans hand theirs on, so the count stops growing once
 * the working set of lists has been seen) and plans currently cached.  Pointers may be NULL. */
int gm_plan_cache_stats(uintptr_t device, uint64_t *plan_builds, uint64_t *table_allocations,
                        int *cached_plans);

/* Measurement helpers used by the benchmark and the profiles. */

/* Records a start / stop event pair on the device's stream; gm_timer_stop
 * synchronises and returns the elapsed milliseconds between them (< 0 on error). */
int   gm_timer_start(uintptr_t device);
float gm_timer_stop(uintptr_t device);
/* Fills a buffer with counter-based pseudo-random normals N(mean, std) (fp32)
 * or half(N(mean, std) * scale) (fp16), reproducible from (seed, element index). */
int gm_fill_normal_f32(uintptr_t device, uintptr_t buffer, size_t num_elements, uint64_t seed,
                       float mean, float std);
int gm_fill_normal_f16(uintptr_t device, uintptr_t buffer, size_t num_elements, uint64_t seed,
                       float mean, float std, float scale);
/* Plain 16-byte-per-lane copy kernel: the measured HBM ceiling the update
 * kernels are compared with, and the known-size launch that calibrates the
 * profiler's FETCH_SIZE / WRITE_SIZE counters. */
int gm_copy_probe(uintptr_t device, uintptr_t dst_buffer, uintptr_t src_buffer, size_t bytes);
/* Launch-shape overrides for sweeps.  They belong to the device's context: every step issued on that
 * device handle uses them from the next call on, steps on another context do not.  Elements per chunk (a power-of-two multiple of
 * 256 * vec, of 1024 when vec is automatic; 0 = default: 65536, 16384, 4096, 1024 or 256, the largest
 * that keeps idle workgroups under 5 % for the tensor list, plus a smaller size for the list's
 * small tensors when they would idle 16384 workgroups or more; a size given here applies to
 * the whole list), non-temporal memory hints
 * on/off (-1 = default on) and fp32 elements per lane (1, 2 or 4; 0 = default: 2 for rules
 * with up to five streams, else 1).
 * -1 if the combination is not valid or device is 0 (nothing changes), -2 without a usable GPU. */
int gm_set_tuning(uintptr_t device, int chunk_elements, int nontemporal, int vec);
/* Lanes per workgroup of the update kernels: 128 or 256; 0 = default (128 for rules with up to
 * five streams, else 256).  Per context, like gm_set_tuning.  -1 on any other value or device 0
 * (nothing changes), -2 without a usable GPU. */
int gm_set_workgroup_lanes(uintptr_t device, int lanes);

/* The overflow check of the mixed-precision step, for re-measurement: whether its loads carry the
 * non-temporal hint (default 1; -1 = default) and whether it walks the chunk table backwards, ending
 * on the gradients the update pass reads first (default 0; -1 = default).  Results do not depend on
 * either.  Per context, like gm_set_tuning.  0, -1 for device 0, -2 without a usable GPU. */
int gm_set_amp_check_order(uintptr_t device, int nontemporal, int reverse);

#ifdef __cplusplus
}
#endif
#endif
