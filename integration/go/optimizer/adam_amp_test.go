//go:build linux && amd64

package optimizer

// Device tests of the additions, in the style of adam_test.go: they need an MI355X and libgometal_hip.so and are
// skipped when no device can be created.  Results are held to the CPU oracle of this package bit for bit.

import (
	"math"
	"math/rand"
	"testing"
	"unsafe"

	"github.com/tsawler/go-metal/cgo_bridge"
	"github.com/tsawler/go-metal/memory"
)

func normal32(rng *rand.Rand, n int, std float64) []float32 {
	out := make([]float32, n)
	for i := range out {
		out[i] = float32(rng.NormFloat64() * std)
	}
	return out
}

// halfBytes packs fp16 bit patterns little-endian, padded to a multiple of four bytes.
func halfBytes(h []uint16) []byte {
	out := make([]byte, (2*len(h)+3)/4*4)
	for i, x := range h {
		out[2*i] = byte(x)
		out[2*i+1] = byte(x >> 8)
	}
	return out
}

// readHalves reads n fp16 bit patterns from a device buffer through the float32 copy.
func readHalves(t *testing.T, buffer unsafe.Pointer, n int) []uint16 {
	words, err := cgo_bridge.CopyMetalBufferToFloat32Array(buffer, (n+1)/2)
	if err != nil {
		t.Fatalf("read-back failed: %v", err)
	}
	out := make([]uint16, n)
	for i := range out {
		bits := math.Float32bits(words[i/2])
		out[i] = uint16(bits >> (16 * uint(i%2)))
	}
	return out
}

func sameBits(a, b []float32) int {
	for i := range a {
		if math.Float32bits(a[i]) != math.Float32bits(b[i]) {
			return i
		}
	}
	return -1
}

// TestAdamStepMatchesOracle: configuration 1 of the benchmark at reduced size, p / m / v after every step.
func TestAdamStepMatchesOracle(t *testing.T) {
	device, err := cgo_bridge.CreateMetalDevice()
	if err != nil {
		t.Skipf("device not available: %v", err)
	}
	defer cgo_bridge.DestroyMetalDevice(device)
	memory.InitializeGlobalMemoryManager(device)
	mm := memory.GetGlobalMemoryManager()

	shapes := [][]int{{300, 7}, {4097}, {1}}
	config := AdamConfig{LearningRate: 1e-3, Beta1: 0.9, Beta2: 0.999, Epsilon: 1e-8, WeightDecay: 1e-4}
	opt, err := NewAdamOptimizer(config, shapes, mm, device)
	if err != nil {
		t.Fatalf("NewAdamOptimizer: %v", err)
	}
	defer opt.Cleanup()

	rng := rand.New(rand.NewSource(1))
	n := len(shapes)
	w, m, v := make([][]float32, n), make([][]float32, n), make([][]float32, n)
	weights, grads := make([]unsafe.Pointer, n), make([]unsafe.Pointer, n)
	for i, shape := range shapes {
		numel := calculateTensorSize(shape)
		w[i], m[i], v[i] = normal32(rng, numel, 0.02), make([]float32, numel), make([]float32, numel)
		weights[i], grads[i] = mm.AllocateBuffer(4*numel), mm.AllocateBuffer(4*numel)
		defer mm.ReleaseBuffer(weights[i])
		defer mm.ReleaseBuffer(grads[i])
		if err := cgo_bridge.CopyFloat32ArrayToMetalBuffer(weights[i], w[i]); err != nil {
			t.Fatal(err)
		}
	}
	if err := opt.SetWeightBuffers(weights); err != nil {
		t.Fatal(err)
	}
	for step := 1; step <= 10; step++ {
		for i := range shapes {
			g := normal32(rng, len(w[i]), 1e-2)
			if err := cgo_bridge.CopyFloat32ArrayToMetalBuffer(grads[i], g); err != nil {
				t.Fatal(err)
			}
			OracleAdamStep(w[i], g, m[i], v[i], config.LearningRate, config.Beta1, config.Beta2, config.Epsilon,
				config.WeightDecay, step)
		}
		if err := opt.Step(grads); err != nil {
			t.Fatalf("Step %d: %v", step, err)
		}
		for i := range shapes {
			for name, pair := range map[string][2]interface{}{
				"weights":  {weights[i], w[i]},
				"momentum": {opt.MomentumBuffers[i], m[i]},
				"variance": {opt.VarianceBuffers[i], v[i]},
			} {
				want := pair[1].([]float32)
				got, err := cgo_bridge.CopyMetalBufferToFloat32Array(pair[0].(unsafe.Pointer), len(want))
				if err != nil {
					t.Fatal(err)
				}
				if k := sameBits(got, want); k >= 0 {
					t.Fatalf("step %d tensor %d %s[%d]: got %g want %g", step, i, name, k, got[k], want[k])
				}
			}
		}
	}
	if opt.GetStepCount() != 10 {
		t.Errorf("step count %d, want 10", opt.GetStepCount())
	}
}

// TestStepAMPMatchesOracle: clean steps, a dropped step (inf in the last element of the last tensor), growth of the
// scale at the interval; both forms of the step, waited for and run ahead.
func TestStepAMPMatchesOracle(t *testing.T) {
	device, err := cgo_bridge.CreateMetalDevice()
	if err != nil {
		t.Skipf("device not available: %v", err)
	}
	defer cgo_bridge.DestroyMetalDevice(device)
	memory.InitializeGlobalMemoryManager(device)
	mm := memory.GetGlobalMemoryManager()

	for _, pingPong := range []bool{false, true} {
		shapes := [][]int{{1000, 33}, {257}, {5}}
		config := AdamConfig{LearningRate: 1e-3, Beta1: 0.9, Beta2: 0.999, Epsilon: 1e-8, WeightDecay: 1e-4}
		opt, err := NewAdamOptimizer(config, shapes, mm, device)
		if err != nil {
			t.Fatalf("NewAdamOptimizer: %v", err)
		}
		rng := rand.New(rand.NewSource(2))
		n := len(shapes)
		w, m, v := make([][]float32, n), make([][]float32, n), make([][]float32, n)
		w16 := make([][]uint16, n)
		weights, grads16, weights16 := make([]unsafe.Pointer, n), make([]unsafe.Pointer, n), make([]unsafe.Pointer, n)
		for i, shape := range shapes {
			numel := calculateTensorSize(shape)
			w[i], m[i], v[i] = normal32(rng, numel, 0.02), make([]float32, numel), make([]float32, numel)
			w16[i] = make([]uint16, numel)
			for k := range w[i] {
				w16[i][k] = Float32ToFloat16(w[i][k]) // the ping-pong step wants the copy to start as half(weights)
			}
			weights[i], grads16[i], weights16[i] = mm.AllocateBuffer(4*numel), mm.AllocateBuffer(2*numel+2), mm.AllocateBuffer(2*numel+2)
			if err := cgo_bridge.CopyFloat32ArrayToMetalBuffer(weights[i], w[i]); err != nil {
				t.Fatal(err)
			}
			if err := cgo_bridge.CopyDataToMetalBuffer(weights16[i], halfBytes(w16[i])); err != nil {
				t.Fatal(err)
			}
		}
		if err := opt.SetWeightBuffers(weights); err != nil {
			t.Fatal(err)
		}
		if err := opt.EnableMixedPrecision(4096, 2, 0.5, 3); err != nil {
			t.Fatal(err)
		}
		if pingPong {
			if err := opt.EnablePingPong(); err != nil {
				t.Fatal(err)
			}
		}
		st := &OracleAMPState{Scale: 4096, GrowthFactor: 2, BackoffFactor: 0.5, GrowthInterval: 3}
		for step := 0; step < 12; step++ {
			g16 := make([][]uint16, n)
			for i := range shapes {
				g := normal32(rng, len(w[i]), 1e-4*float64(st.Scale))
				g16[i] = make([]uint16, len(g))
				for k := range g {
					g16[i][k] = Float32ToFloat16(g[k])
				}
			}
			if step == 2 || step == 7 {
				last := g16[n-1]
				last[len(last)-1] = 0xFC00 // -inf
			}
			for i := range shapes {
				if err := cgo_bridge.CopyDataToMetalBuffer(grads16[i], halfBytes(g16[i])); err != nil {
					t.Fatal(err)
				}
			}
			want := OracleAdamAMPStep(w, g16, m, v, w16, config.LearningRate, config.Beta1, config.Beta2,
				config.Epsilon, config.WeightDecay, st)
			if step%4 == 3 { // run ahead, then catch up
				if err := opt.StepAMPAsync(grads16, weights16); err != nil {
					t.Fatalf("StepAMPAsync %d: %v", step, err)
				}
				if err := opt.SyncAMP(); err != nil {
					t.Fatal(err)
				}
			} else {
				skipped, err := opt.StepAMP(grads16, weights16)
				if err != nil {
					t.Fatalf("StepAMP %d: %v", step, err)
				}
				if skipped != want {
					t.Fatalf("step %d: skipped %v, want %v", step, skipped, want)
				}
			}
			scale, tracker := opt.LossScale()
			if scale != st.Scale || tracker != st.GrowthTracker || opt.GetStepCount() != st.StepCount {
				t.Fatalf("step %d: scale %g tracker %d count %d, want %g %d %d", step, scale, tracker,
					opt.GetStepCount(), st.Scale, st.GrowthTracker, st.StepCount)
			}
			current, moments, variances := opt.CurrentWeightBuffers(), opt.CurrentMomentumBuffers(), opt.CurrentVarianceBuffers()
			for i := range shapes {
				for name, pair := range map[string][2]interface{}{
					"weights": {current[i], w[i]}, "momentum": {moments[i], m[i]}, "variance": {variances[i], v[i]},
				} {
					wantArr := pair[1].([]float32)
					got, err := cgo_bridge.CopyMetalBufferToFloat32Array(pair[0].(unsafe.Pointer), len(wantArr))
					if err != nil {
						t.Fatal(err)
					}
					if k := sameBits(got, wantArr); k >= 0 {
						t.Fatalf("pingPong %v step %d tensor %d %s[%d]: got %g want %g", pingPong, step, i, name, k, got[k], wantArr[k])
					}
				}
				got16 := readHalves(t, weights16[i], len(w16[i]))
				for k := range got16 {
					if got16[k] != w16[i][k] {
						t.Fatalf("pingPong %v step %d tensor %d fp16 copy[%d]: got %#04x want %#04x", pingPong, step, i, k, got16[k], w16[i][k])
					}
				}
			}
		}
		if st.StepCount != 10 {
			t.Fatalf("the schedule should have applied 10 steps, applied %d", st.StepCount)
		}
		opt.Cleanup()
		for i := range shapes {
			mm.ReleaseBuffer(weights[i])
			mm.ReleaseBuffer(grads16[i])
			mm.ReleaseBuffer(weights16[i])
		}
	}
}
