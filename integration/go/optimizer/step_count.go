package optimizer

// GetStepCount for the two optimizers that lack it in the reference (adam.go:266 and rmsprop.go:261 have
// GetStep only), so that *AdamOptimizerState and *RMSPropOptimizerState satisfy the Optimizer interface
// (interface.go:28-29) like the other four.  Additive: nothing else changes.

// GetStepCount returns the current optimization step number.  With mixed-precision steps still in flight
// (StepAMPAsync) it first waits for them: the device counts the steps it applied.
func (adam *AdamOptimizerState) GetStepCount() uint64 {
	adam.finishPendingAMP()
	return adam.StepCount
}

// GetStepCount returns the current optimization step number.
func (rmsprop *RMSPropOptimizerState) GetStepCount() uint64 {
	return rmsprop.StepCount
}
