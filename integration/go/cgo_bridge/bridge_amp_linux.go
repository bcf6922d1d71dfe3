//go:build linux && amd64

package cgo_bridge

// Wrappers for the entry points libgometal_hip.so adds to the reference's C ABI: the mixed-precision
// (fp16-gradient) Adam step in its two forms, the loss-scale state they share, buffers placed at a phase, and
// an explicit wait.  Slices are marshalled exactly as ExecuteAdamStepMPSGraph does it (bridge.go:989-1011):
// one []C.uintptr_t per list, built per call, never retained by the C side.

/*
#include <stdint.h>
#include "gometal_hip.h"
*/
import "C"

import (
	"fmt"
	"unsafe"
)

// handleArray copies a slice of buffer handles into a C array (bridge.go:999-1010).
func handleArray(buffers []unsafe.Pointer) []C.uintptr_t {
	out := make([]C.uintptr_t, len(buffers))
	for i, b := range buffers {
		out[i] = C.uintptr_t(uintptr(b))
	}
	return out
}

// first returns the address of a handle array's first element, or nil for an empty (optional) list.
func first(a []C.uintptr_t) *C.uintptr_t {
	if len(a) == 0 {
		return nil
	}
	return &a[0]
}

func sizeArray(sizes []int) []C.int {
	out := make([]C.int, len(sizes))
	for i, s := range sizes {
		out[i] = C.int(s)
	}
	return out
}

// AllocateMetalBufferPhased is AllocateMetalBuffer (bridge.go:729-741) with the start of the buffer at
// phaseBytes modulo 2 MiB (a multiple of 256 below 2 MiB).  Freed with DeallocateMetalBuffer.
func AllocateMetalBufferPhased(device unsafe.Pointer, size int, deviceType DeviceType, phaseBytes int) (unsafe.Pointer, error) {
	buffer := C.gm_allocate_buffer_phased(C.uintptr_t(uintptr(device)), C.int(size), C.int(deviceType), C.int(phaseBytes))
	if buffer == 0 {
		return nil, fmt.Errorf("failed to allocate Metal buffer of size %d at phase %d", size, phaseBytes)
	}
	return unsafe.Pointer(uintptr(buffer)), nil
}

// Synchronize waits for every step enqueued on the library's stream (update steps return before they finish;
// every call that hands data to the host waits by itself).
func Synchronize(device unsafe.Pointer) error {
	if rc := C.gm_synchronize(C.uintptr_t(uintptr(device))); rc != 0 {
		return fmt.Errorf("device synchronisation failed with error code: %d", int(rc))
	}
	return nil
}

// BiasCorrections returns 1 - beta1^step and 1 - beta2^step exactly as the Adam and NAdam entry points compute
// them (the C library's powf in float32, bridge_optimizer.m:398-399).
func BiasCorrections(beta1, beta2 float32, step int) (bc1, bc2 float32) {
	var a, b C.float
	C.gm_bias_corrections(C.float(beta1), C.float(beta2), C.int(step), &a, &b)
	return float32(a), float32(b)
}

// NadamMuNext returns NAdam's momentum schedule at step + 1 as the entry point computes it (bridge_optimizer.m:2066).
func NadamMuNext(beta1 float32, step int) float32 {
	return float32(C.gm_nadam_mu_next(C.float(beta1), C.int(step)))
}

// CreateAMPState creates the device-resident loss-scale state of the mixed-precision step
// (defaults of training/model_trainer.go:258-270: 65536, 2, 0.5, 2000).
func CreateAMPState(device unsafe.Pointer, initialScale, growthFactor, backoffFactor float32, growthInterval int) (unsafe.Pointer, error) {
	state := C.gm_amp_state_create(C.uintptr_t(uintptr(device)), C.float(initialScale), C.float(growthFactor),
		C.float(backoffFactor), C.int(growthInterval))
	if state == 0 {
		return nil, fmt.Errorf("failed to create loss-scale state")
	}
	return unsafe.Pointer(uintptr(state)), nil
}

// DestroyAMPState waits for steps in flight and frees the state.
func DestroyAMPState(ampState unsafe.Pointer) {
	if ampState != nil {
		C.gm_amp_state_destroy(C.uintptr_t(uintptr(ampState)))
	}
}

// QueryAMPState waits for every step in flight and returns the loss scale, the clean-step counter, the
// number of steps applied (the optimizer's StepCount as the device counts it) and the number dropped.
func QueryAMPState(ampState unsafe.Pointer) (scale float32, growthTracker, appliedSteps, skippedSteps int, err error) {
	var sc C.float
	var gt, ap, sk C.int
	if rc := C.gm_amp_state_query(C.uintptr_t(uintptr(ampState)), &sc, &gt, &ap, &sk); rc != 0 {
		return 0, 0, 0, 0, fmt.Errorf("loss-scale state query failed with error code: %d", int(rc))
	}
	return float32(sc), int(gt), int(ap), int(sk), nil
}

// SetAMPState restores the loss scale and the clean-step counter (checkpoint resume).
func SetAMPState(ampState unsafe.Pointer, scale float32, growthTracker int) error {
	if rc := C.gm_amp_state_set(C.uintptr_t(uintptr(ampState)), C.float(scale), C.int(growthTracker)); rc != 0 {
		return fmt.Errorf("loss-scale state update failed with error code: %d", int(rc))
	}
	return nil
}

// SetAMPStepCount tells the device how many steps have been applied so far (the asynchronous steps take
// their bias corrections from the device's own count).
func SetAMPStepCount(ampState unsafe.Pointer, appliedSteps int) error {
	if rc := C.gm_amp_state_set_step_count(C.uintptr_t(uintptr(ampState)), C.int(appliedSteps)); rc != 0 {
		return fmt.Errorf("loss-scale state step count update failed with error code: %d", int(rc))
	}
	return nil
}

// AMPCurrentSet waits and returns which ping-pong set holds the current weights and moments (0: A, 1: B).
func AMPCurrentSet(ampState unsafe.Pointer) (int, error) {
	rc := C.gm_amp_state_current_set(C.uintptr_t(uintptr(ampState)))
	if rc < 0 {
		return 0, fmt.Errorf("loss-scale state query failed with error code: %d", int(rc))
	}
	return int(rc), nil
}

// SetAMPCurrentSet tells a newly created state which set is current.
func SetAMPCurrentSet(ampState unsafe.Pointer, currentSet int) error {
	if rc := C.gm_amp_state_set_current_set(C.uintptr_t(uintptr(ampState)), C.int(currentSet)); rc != 0 {
		return fmt.Errorf("loss-scale state update failed with error code: %d", int(rc))
	}
	return nil
}

func checkAMPLists(n int, lists [][]unsafe.Pointer, weight16Buffers []unsafe.Pointer, bufferSizes []int) error {
	for _, l := range lists {
		if len(l) != n {
			return fmt.Errorf("all buffer arrays must have the same length")
		}
	}
	if len(bufferSizes) != n || (len(weight16Buffers) != 0 && len(weight16Buffers) != n) {
		return fmt.Errorf("all buffer arrays must have the same length")
	}
	if n == 0 {
		return fmt.Errorf("buffer arrays must not be empty")
	}
	return nil
}

// ExecuteAdamAMPStep runs one mixed-precision Adam step in place and waits for it: fp16 gradients of the
// scaled loss, fp32 weights and moments, an fp16 copy of the new weights (weight16Buffers may be empty).
// stepCount is the bias-correction step of this step IF it is applied (the caller's StepCount + 1).
// skipped: a gradient held an inf / NaN, nothing was written and the loss scale was reduced.
func ExecuteAdamAMPStep(
	device unsafe.Pointer,
	weightBuffers, gradient16Buffers, momentumBuffers, varianceBuffers, weight16Buffers []unsafe.Pointer,
	bufferSizes []int,
	learningRate, beta1, beta2, epsilon, weightDecay float32,
	stepCount int,
	ampState unsafe.Pointer,
) (skipped bool, scale float32, growthTracker int, err error) {
	n := len(weightBuffers)
	if err := checkAMPLists(n, [][]unsafe.Pointer{gradient16Buffers, momentumBuffers, varianceBuffers}, weight16Buffers, bufferSizes); err != nil {
		return false, 0, 0, err
	}
	cW, cG, cM, cV, cH := handleArray(weightBuffers), handleArray(gradient16Buffers), handleArray(momentumBuffers),
		handleArray(varianceBuffers), handleArray(weight16Buffers)
	cSizes := sizeArray(bufferSizes)
	var sk, gt C.int
	var sc C.float
	result := C.execute_adam_amp_step(
		C.uintptr_t(uintptr(device)), &cW[0], &cG[0], &cM[0], &cV[0], first(cH),
		C.int(n), &cSizes[0],
		C.float(learningRate), C.float(beta1), C.float(beta2), C.float(epsilon), C.float(weightDecay),
		C.int(stepCount), C.uintptr_t(uintptr(ampState)), &sk, &sc, &gt,
	)
	if result != 0 {
		return false, 0, 0, fmt.Errorf("Adam mixed-precision step failed with error code: %d", int(result))
	}
	return sk != 0, float32(sc), int(gt), nil
}

// ExecuteAdamAMPStepAsync enqueues the same step and returns; the device counts applied steps itself
// (SetAMPStepCount), and QueryAMPState waits and reports.
func ExecuteAdamAMPStepAsync(
	device unsafe.Pointer,
	weightBuffers, gradient16Buffers, momentumBuffers, varianceBuffers, weight16Buffers []unsafe.Pointer,
	bufferSizes []int,
	learningRate, beta1, beta2, epsilon, weightDecay float32,
	ampState unsafe.Pointer,
) error {
	n := len(weightBuffers)
	if err := checkAMPLists(n, [][]unsafe.Pointer{gradient16Buffers, momentumBuffers, varianceBuffers}, weight16Buffers, bufferSizes); err != nil {
		return err
	}
	cW, cG, cM, cV, cH := handleArray(weightBuffers), handleArray(gradient16Buffers), handleArray(momentumBuffers),
		handleArray(varianceBuffers), handleArray(weight16Buffers)
	cSizes := sizeArray(bufferSizes)
	result := C.execute_adam_amp_step_async(
		C.uintptr_t(uintptr(device)), &cW[0], &cG[0], &cM[0], &cV[0], first(cH),
		C.int(n), &cSizes[0],
		C.float(learningRate), C.float(beta1), C.float(beta2), C.float(epsilon), C.float(weightDecay),
		C.uintptr_t(uintptr(ampState)),
	)
	if result != 0 {
		return fmt.Errorf("Adam mixed-precision step failed with error code: %d", int(result))
	}
	return nil
}

// AMPSet is one set of weights and moments of the ping-pong step.
type AMPSet struct {
	Weights, Momentum, Variance []unsafe.Pointer
}

// ExecuteAdamAMPStepFused runs the step in one pass over ping-pong state and waits for it: it reads the set
// that is current, writes the other one, and that one becomes current only if no gradient overflowed.
// currentSet (0: a, 1: b) is the current set after the step.
func ExecuteAdamAMPStepFused(
	device unsafe.Pointer,
	a, b AMPSet,
	gradient16Buffers, weight16Buffers []unsafe.Pointer,
	bufferSizes []int,
	learningRate, beta1, beta2, epsilon, weightDecay float32,
	stepCount int,
	ampState unsafe.Pointer,
) (skipped bool, scale float32, growthTracker int, currentSet int, err error) {
	n := len(a.Weights)
	lists := [][]unsafe.Pointer{a.Momentum, a.Variance, b.Weights, b.Momentum, b.Variance, gradient16Buffers}
	if err := checkAMPLists(n, lists, weight16Buffers, bufferSizes); err != nil {
		return false, 0, 0, 0, err
	}
	cWa, cMa, cVa := handleArray(a.Weights), handleArray(a.Momentum), handleArray(a.Variance)
	cWb, cMb, cVb := handleArray(b.Weights), handleArray(b.Momentum), handleArray(b.Variance)
	cG, cH := handleArray(gradient16Buffers), handleArray(weight16Buffers)
	cSizes := sizeArray(bufferSizes)
	var sk, gt, cur C.int
	var sc C.float
	result := C.execute_adam_amp_step_fused(
		C.uintptr_t(uintptr(device)), &cWa[0], &cMa[0], &cVa[0], &cWb[0], &cMb[0], &cVb[0], &cG[0], first(cH),
		C.int(n), &cSizes[0],
		C.float(learningRate), C.float(beta1), C.float(beta2), C.float(epsilon), C.float(weightDecay),
		C.int(stepCount), C.uintptr_t(uintptr(ampState)), &sk, &sc, &gt, &cur,
	)
	if result != 0 {
		return false, 0, 0, 0, fmt.Errorf("Adam mixed-precision step failed with error code: %d", int(result))
	}
	return sk != 0, float32(sc), int(gt), int(cur), nil
}

// ExecuteAdamAMPStepFusedAsync enqueues the one-pass step and returns.
func ExecuteAdamAMPStepFusedAsync(
	device unsafe.Pointer,
	a, b AMPSet,
	gradient16Buffers, weight16Buffers []unsafe.Pointer,
	bufferSizes []int,
	learningRate, beta1, beta2, epsilon, weightDecay float32,
	ampState unsafe.Pointer,
) error {
	n := len(a.Weights)
	lists := [][]unsafe.Pointer{a.Momentum, a.Variance, b.Weights, b.Momentum, b.Variance, gradient16Buffers}
	if err := checkAMPLists(n, lists, weight16Buffers, bufferSizes); err != nil {
		return err
	}
	cWa, cMa, cVa := handleArray(a.Weights), handleArray(a.Momentum), handleArray(a.Variance)
	cWb, cMb, cVb := handleArray(b.Weights), handleArray(b.Momentum), handleArray(b.Variance)
	cG, cH := handleArray(gradient16Buffers), handleArray(weight16Buffers)
	cSizes := sizeArray(bufferSizes)
	result := C.execute_adam_amp_step_fused_async(
		C.uintptr_t(uintptr(device)), &cWa[0], &cMa[0], &cVa[0], &cWb[0], &cMb[0], &cVb[0], &cG[0], first(cH),
		C.int(n), &cSizes[0],
		C.float(learningRate), C.float(beta1), C.float(beta2), C.float(epsilon), C.float(weightDecay),
		C.uintptr_t(uintptr(ampState)),
	)
	if result != 0 {
		return fmt.Errorf("Adam mixed-precision step failed with error code: %d", int(result))
	}
	return nil
}
