//go:build !(linux && amd64)

package optimizer

// Builds without libgometal_hip.so have no mixed-precision step: nothing is ever pending.
func (adam *AdamOptimizerState) finishPendingAMP() {}
