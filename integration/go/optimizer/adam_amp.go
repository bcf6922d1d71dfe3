//go:build linux && amd64

package optimizer

// Mixed-precision (fp16-gradient) Adam on *AdamOptimizerState: EnableMixedPrecision, EnablePingPong, StepAMP,
// StepAMPAsync, SyncAMP.  Additive to adam.go; the reference has the configuration of mixed precision
// (training/model_trainer.go:79-87, 258-270) and no step for it.
//
// The struct in adam.go:13-39 is left as it is: what these methods keep per optimizer lives in a side table
// keyed by the optimizer.  Three places of adam.go call into this file once it is present (each one line):
//
//	Step      (adam.go:177)  first line:   if err := adam.beforeStep(); err != nil { return err }
//	                         and passes adam.CurrentWeightBuffers(), adam.CurrentMomentumBuffers(),
//	                         adam.CurrentVarianceBuffers() where it passes the three slices (adam.go:213-218)
//	GetState / LoadState     (adam.go:329, 383) read and write adam.CurrentMomentumBuffers() /
//	                         adam.CurrentVarianceBuffers() instead of the slices
//	Cleanup   (adam.go:306)  first line:   adam.cleanupAMP()
//
// Without ping-pong state (the default) the Current* accessors return the optimizer's own slices, so the
// first and second hook only matter for the pending-step wait.

import (
	"fmt"
	"sync"
	"unsafe"

	"github.com/tsawler/go-metal/cgo_bridge"
	"github.com/tsawler/go-metal/memory"
)

// adamAMP is the mixed-precision side of one AdamOptimizerState.
type adamAMP struct {
	state         unsafe.Pointer // device-resident loss-scale state (cgo_bridge.CreateAMPState)
	LossScale     float32        // as of the last StepAMP / SyncAMP / EnableMixedPrecision
	GrowthTracker int
	pending       int  // asynchronous steps issued since the last SyncAMP
	countDirty    bool // StepCount changed on the host (Step, LoadState): tell the device before the next step
	pingPong      bool
	currentSet    int // 0: the optimizer's own buffers are current, 1: the shadows
	shadow        cgo_bridge.AMPSet
}

var ampTable sync.Map // *AdamOptimizerState -> *adamAMP

func (adam *AdamOptimizerState) ampLookup() *adamAMP {
	if v, ok := ampTable.Load(adam); ok {
		return v.(*adamAMP)
	}
	return nil
}

// EnableMixedPrecision creates the device-resident loss-scale state.  Call once before StepAMP; a second call
// replaces the state (steps in flight finish first, the current ping-pong set is carried over).
// Defaults of the reference's trainer: 65536, 2.0, 0.5, 2000.
func (adam *AdamOptimizerState) EnableMixedPrecision(initialScale, growthFactor, backoffFactor float32, growthInterval int) error {
	if adam.device == nil {
		return fmt.Errorf("device cannot be nil")
	}
	if !(initialScale > 0) {
		return fmt.Errorf("initial loss scale must be positive, got %f", initialScale)
	}
	if growthInterval <= 0 {
		return fmt.Errorf("growth interval must be positive, got %d", growthInterval)
	}
	amp := adam.ampLookup()
	if amp == nil {
		amp = &adamAMP{}
		ampTable.Store(adam, amp)
	}
	if amp.state != nil {
		if amp.pending > 0 {
			if err := adam.SyncAMP(); err != nil {
				return err
			}
		}
		cgo_bridge.DestroyAMPState(amp.state)
		amp.state = nil
	}
	state, err := cgo_bridge.CreateAMPState(adam.device, initialScale, growthFactor, backoffFactor, growthInterval)
	if err != nil {
		return fmt.Errorf("failed to create loss-scale state: %v", err)
	}
	amp.state = state
	if amp.pingPong && amp.currentSet != 0 {
		if err := cgo_bridge.SetAMPCurrentSet(state, amp.currentSet); err != nil {
			return fmt.Errorf("failed to carry the current ping-pong set over: %v", err)
		}
	}
	amp.LossScale = initialScale
	amp.GrowthTracker = 0
	amp.pending = 0
	amp.countDirty = true
	return nil
}

// EnablePingPong switches StepAMP / StepAMPAsync to the one-pass step: a second set of weight, momentum and
// variance buffers is allocated, every applied step reads the current set and writes the other, and a dropped
// step leaves the current set as it was because it was never written (28 bytes per parameter move instead of
// 30).  Call after SetWeightBuffers and EnableMixedPrecision.  From then on the current fp32 weights are where
// CurrentWeightBuffers says, which after an odd number of applied steps is NOT the caller's own buffers; the
// fp16 weight copy passed to StepAMP is always the caller's buffer and must start out as half of the weights.
// Not the default for that reason.
func (adam *AdamOptimizerState) EnablePingPong() error {
	amp := adam.ampLookup()
	if amp == nil || amp.state == nil {
		return fmt.Errorf("mixed precision is not enabled: call EnableMixedPrecision first")
	}
	if amp.pingPong {
		return nil
	}
	if adam.memoryManager == nil {
		return fmt.Errorf("memory manager cannot be nil")
	}
	for _, w := range adam.WeightBuffers {
		if w == nil {
			return fmt.Errorf("weight buffers are not set: call SetWeightBuffers first")
		}
	}
	n := len(adam.bufferSizes)
	lists := []*[]unsafe.Pointer{&amp.shadow.Weights, &amp.shadow.Momentum, &amp.shadow.Variance}
	phases := []int{memory.ShadowWeightPhase, memory.StatePhases[0], memory.StatePhases[1]}
	for k, list := range lists {
		*list = make([]unsafe.Pointer, n)
		for i, size := range adam.bufferSizes {
			(*list)[i] = adam.memoryManager.AllocateBufferAtPhase(size, phases[k])
			if (*list)[i] == nil {
				adam.releaseShadows(amp)
				return fmt.Errorf("failed to allocate ping-pong buffer for weight %d", i)
			}
		}
	}
	amp.pingPong = true
	amp.currentSet = 0
	return nil
}

func (adam *AdamOptimizerState) releaseShadows(amp *adamAMP) {
	for _, list := range []*[]unsafe.Pointer{&amp.shadow.Weights, &amp.shadow.Momentum, &amp.shadow.Variance} {
		for _, b := range *list {
			if b != nil {
				adam.memoryManager.ReleaseBuffer(b)
			}
		}
		*list = nil
	}
}

// PingPong reports whether the one-pass step is on.
func (adam *AdamOptimizerState) PingPong() bool {
	amp := adam.ampLookup()
	return amp != nil && amp.pingPong
}

func (adam *AdamOptimizerState) shadowIsCurrent() bool {
	amp := adam.ampLookup()
	if amp == nil || !amp.pingPong {
		return false
	}
	if amp.pending > 0 {
		_ = adam.SyncAMP()
	}
	return amp.currentSet == 1
}

// CurrentWeightBuffers returns the buffers that hold the current fp32 weights (the caller's own, or the
// shadows after an odd number of applied ping-pong steps).  Waits for steps in flight.
func (adam *AdamOptimizerState) CurrentWeightBuffers() []unsafe.Pointer {
	if adam.shadowIsCurrent() {
		return adam.ampLookup().shadow.Weights
	}
	return adam.WeightBuffers
}

// CurrentMomentumBuffers: as CurrentWeightBuffers, for the first moments.
func (adam *AdamOptimizerState) CurrentMomentumBuffers() []unsafe.Pointer {
	if adam.shadowIsCurrent() {
		return adam.ampLookup().shadow.Momentum
	}
	return adam.MomentumBuffers
}

// CurrentVarianceBuffers: as CurrentWeightBuffers, for the second moments.
func (adam *AdamOptimizerState) CurrentVarianceBuffers() []unsafe.Pointer {
	if adam.shadowIsCurrent() {
		return adam.ampLookup().shadow.Variance
	}
	return adam.VarianceBuffers
}

// SyncAMP waits for every mixed-precision step in flight and brings StepCount, the loss scale and the
// clean-step counter up to date.
func (adam *AdamOptimizerState) SyncAMP() error {
	amp := adam.ampLookup()
	if amp == nil || amp.state == nil {
		return fmt.Errorf("mixed precision is not enabled: call EnableMixedPrecision first")
	}
	scale, tracker, applied, _, err := cgo_bridge.QueryAMPState(amp.state)
	if err != nil {
		return fmt.Errorf("failed to read loss-scale state: %v", err)
	}
	amp.LossScale, amp.GrowthTracker = scale, tracker
	if amp.pending > 0 {
		adam.StepCount = uint64(applied) // the device counted the pending steps
	}
	if amp.pingPong {
		set, err := cgo_bridge.AMPCurrentSet(amp.state)
		if err != nil {
			return fmt.Errorf("failed to read the current ping-pong set: %v", err)
		}
		amp.currentSet = set
	}
	amp.pending = 0
	return nil
}

// LossScale returns the loss scale and the clean-step counter as of the last StepAMP / SyncAMP.
func (adam *AdamOptimizerState) LossScale() (scale float32, growthTracker int) {
	if amp := adam.ampLookup(); amp != nil {
		return amp.LossScale, amp.GrowthTracker
	}
	return 0, 0
}

func (adam *AdamOptimizerState) checkAMPArgs(gradient16Buffers, weight16Buffers []unsafe.Pointer) (*adamAMP, error) {
	if len(gradient16Buffers) != len(adam.WeightBuffers) {
		return nil, fmt.Errorf("gradient buffers length (%d) doesn't match weight buffers length (%d)",
			len(gradient16Buffers), len(adam.WeightBuffers))
	}
	if len(weight16Buffers) != 0 && len(weight16Buffers) != len(adam.WeightBuffers) {
		return nil, fmt.Errorf("fp16 weight buffers length (%d) doesn't match weight buffers length (%d)",
			len(weight16Buffers), len(adam.WeightBuffers))
	}
	amp := adam.ampLookup()
	if amp == nil || amp.state == nil {
		return nil, fmt.Errorf("mixed precision is not enabled: call EnableMixedPrecision first")
	}
	return amp, nil
}

func (adam *AdamOptimizerState) pushStepCount(amp *adamAMP) error {
	if amp.countDirty {
		if err := cgo_bridge.SetAMPStepCount(amp.state, int(adam.StepCount)); err != nil {
			return fmt.Errorf("failed to set the device step count: %v", err)
		}
		amp.countDirty = false
	}
	return nil
}

// StepAMP performs one mixed-precision Adam step and waits for it.  gradient16Buffers hold fp16 gradients of
// the loss multiplied by the current loss scale; weight16Buffers (may be nil) receive the fp16 copy of the
// new weights.  skipped: a gradient held an inf / NaN; weights, moments and the fp16 copy are unchanged, the
// loss scale was multiplied by the backoff factor, and StepCount did not advance (adam.go:183 counts every
// call; here only applied steps count, so the bias corrections stay those of the steps actually taken).
func (adam *AdamOptimizerState) StepAMP(gradient16Buffers, weight16Buffers []unsafe.Pointer) (skipped bool, err error) {
	amp, err := adam.checkAMPArgs(gradient16Buffers, weight16Buffers)
	if err != nil {
		return false, err
	}
	if amp.pending > 0 {
		if err := adam.SyncAMP(); err != nil {
			return false, err
		}
	}
	if err := adam.pushStepCount(amp); err != nil {
		return false, err
	}
	var scale float32
	var tracker int
	if amp.pingPong {
		a := cgo_bridge.AMPSet{Weights: adam.WeightBuffers, Momentum: adam.MomentumBuffers, Variance: adam.VarianceBuffers}
		var current int
		skipped, scale, tracker, current, err = cgo_bridge.ExecuteAdamAMPStepFused(adam.device, a, amp.shadow,
			gradient16Buffers, weight16Buffers, adam.bufferSizes, adam.LearningRate, adam.Beta1, adam.Beta2,
			adam.Epsilon, adam.WeightDecay, int(adam.StepCount+1), amp.state)
		if err == nil {
			amp.currentSet = current
		}
	} else {
		skipped, scale, tracker, err = cgo_bridge.ExecuteAdamAMPStep(adam.device, adam.WeightBuffers,
			gradient16Buffers, adam.MomentumBuffers, adam.VarianceBuffers, weight16Buffers, adam.bufferSizes,
			adam.LearningRate, adam.Beta1, adam.Beta2, adam.Epsilon, adam.WeightDecay, int(adam.StepCount+1), amp.state)
	}
	if err != nil {
		return false, fmt.Errorf("Adam mixed-precision step execution failed: %v", err)
	}
	amp.LossScale, amp.GrowthTracker = scale, tracker
	if !skipped {
		adam.StepCount++
	}
	return skipped, nil
}

// StepAMPAsync enqueues the same step and returns: the device counts applied steps itself, up to 7 steps run
// ahead of the host, and StepCount, the loss scale and the clean-step counter are brought up to date by SyncAMP
// (GetStepCount, GetState, LoadState, Step and StepAMP call it when steps are pending).
func (adam *AdamOptimizerState) StepAMPAsync(gradient16Buffers, weight16Buffers []unsafe.Pointer) error {
	amp, err := adam.checkAMPArgs(gradient16Buffers, weight16Buffers)
	if err != nil {
		return err
	}
	if err := adam.pushStepCount(amp); err != nil {
		return err
	}
	if amp.pingPong {
		a := cgo_bridge.AMPSet{Weights: adam.WeightBuffers, Momentum: adam.MomentumBuffers, Variance: adam.VarianceBuffers}
		err = cgo_bridge.ExecuteAdamAMPStepFusedAsync(adam.device, a, amp.shadow, gradient16Buffers, weight16Buffers,
			adam.bufferSizes, adam.LearningRate, adam.Beta1, adam.Beta2, adam.Epsilon, adam.WeightDecay, amp.state)
	} else {
		err = cgo_bridge.ExecuteAdamAMPStepAsync(adam.device, adam.WeightBuffers, gradient16Buffers,
			adam.MomentumBuffers, adam.VarianceBuffers, weight16Buffers, adam.bufferSizes, adam.LearningRate,
			adam.Beta1, adam.Beta2, adam.Epsilon, adam.WeightDecay, amp.state)
	}
	if err != nil {
		return fmt.Errorf("Adam mixed-precision step execution failed: %v", err)
	}
	amp.pending++
	return nil
}

// finishPendingAMP waits for asynchronous mixed-precision steps, if any (GetStepCount, step_count.go).
func (adam *AdamOptimizerState) finishPendingAMP() {
	if amp := adam.ampLookup(); amp != nil && amp.pending > 0 {
		_ = adam.SyncAMP()
	}
}

// beforeStep is the hook at the top of Step (adam.go:177): pending asynchronous steps finish first, and the
// device is told about the fp32 step's increment of StepCount before the next mixed-precision step.
func (adam *AdamOptimizerState) beforeStep() error {
	amp := adam.ampLookup()
	if amp == nil {
		return nil
	}
	if amp.pending > 0 {
		if err := adam.SyncAMP(); err != nil {
			return err
		}
	}
	amp.countDirty = true
	return nil
}

// cleanupAMP is the hook at the top of Cleanup (adam.go:306).
func (adam *AdamOptimizerState) cleanupAMP() {
	amp := adam.ampLookup()
	if amp == nil {
		return
	}
	if amp.state != nil {
		cgo_bridge.DestroyAMPState(amp.state) // waits for steps in flight
		amp.state = nil
	}
	if adam.memoryManager != nil {
		adam.releaseShadows(amp)
	}
	ampTable.Delete(adam)
}
