//go:build linux && amd64

package optimizer

// CPU oracle of the optimizer step: the update equations of cgo_bridge/bridge_optimizer.m evaluated on host
// slices, one IEEE binary32 operation per node of the reference's MPSGraph op chain, in the reference's order.
// It is what the GPU results are held to (bit for bit); the tests of this package use it, nothing else does.
//
// Every product and sum is written as its own statement with an explicit float32 conversion: a conversion
// rounds to float32 and keeps the compiler from fusing a multiply and an add into one FMA (which some GOAMD64
// levels and other architectures would otherwise do).  The host scalars (bias corrections, NAdam's momentum
// schedule) come from the library's own helpers, which evaluate them with the C library's powf exactly as
// the step entry points do (bridge_optimizer.m:398-399, 2066).

import (
	"math"

	"github.com/tsawler/go-metal/cgo_bridge"
)

const fltMin = 0x1p-126 // the smallest normal float32

func sqrt32(x float32) float32 { return float32(math.Sqrt(float64(x))) } // correctly rounded: sqrt of a float32 in float64, rounded once

// OracleSGDStep: bridge_optimizer.m:160-357.  m may be nil (no momentum buffer: the vanilla rule).
func OracleSGDStep(w, g, m []float32, lr, momentum, weightDecay float32, nesterov bool) {
	useMomentum := momentum > 0 && m != nil // :233
	for i := range w {
		wi, gi := w[i], g[i]
		if weightDecay > 0 { // :219-228
			decay := float32(wi * weightDecay)
			gi = float32(gi + decay)
		}
		if useMomentum {
			scaled := float32(m[i] * momentum) // :245
			mi := float32(scaled + gi)         // :248
			var upd float32
			if nesterov { // :257-267
				t1 := float32(momentum * mi)
				t2 := float32(t1 + gi)
				upd = float32(lr * t2)
			} else { // :270-272
				upd = float32(lr * mi)
			}
			w[i] = float32(wi - upd) // :276
			m[i] = mi
		} else { // :315-322
			upd := float32(lr * gi)
			w[i] = float32(wi - upd)
		}
	}
}

// adamElement: one element of bridge_optimizer.m:484-550; shared with the mixed-precision step.
func adamElement(w, m, v *float32, g, lr, beta1, beta2, oneMinusBeta1, oneMinusBeta2, eps, weightDecay, bc1, bc2 float32) {
	wi := *w
	mScaled := float32(*m * beta1)             // :484
	gScaled := float32(g * oneMinusBeta1)      // :487
	mi := float32(mScaled + gScaled)           // :490
	gSq := float32(g * g)                      // :495
	vScaled := float32(*v * beta2)             // :498
	gSqScaled := float32(gSq * oneMinusBeta2)  // :501
	vi := float32(vScaled + gSqScaled)         // :504
	mHat := float32(mi / bc1)                  // :509
	vHat := float32(vi / bc2)                  // :514
	root := sqrt32(vHat)                       // :519
	den := float32(root + eps)                 // :521
	upd := float32(mHat / den)                 // :526
	if weightDecay > 0 {                       // :531-540
		decay := float32(wi * weightDecay)
		upd = float32(upd + decay)
	}
	scaled := float32(upd * lr) // :543
	*w = float32(wi - scaled)   // :548
	*m = mi
	*v = vi
}

// OracleAdamStep: bridge_optimizer.m:360-641.  step is the step count AFTER the increment of adam.go:183.
func OracleAdamStep(w, g, m, v []float32, lr, beta1, beta2, eps, weightDecay float32, step int) {
	bc1, bc2 := cgo_bridge.BiasCorrections(beta1, beta2, step)
	omb1 := float32(1.0 - beta1) // :469
	omb2 := float32(1.0 - beta2) // :471
	for i := range w {
		adamElement(&w[i], &m[i], &v[i], g[i], lr, beta1, beta2, omb1, omb2, eps, weightDecay, bc1, bc2)
	}
}

// OracleRMSPropStep: bridge_optimizer.m:691-951.  mom / gavg may be nil when momentum is 0 / centered is false.
func OracleRMSPropStep(w, g, s, mom, gavg []float32, lr, alpha, eps, weightDecay, momentum float32, centered bool) {
	oma := float32(1.0 - alpha) // :773
	for i := range w {
		wi, gi := w[i], g[i]
		gSq := float32(gi * gi)            // :782
		sScaled := float32(s[i] * alpha)   // :785
		gSqScaled := float32(gSq * oma)    // :788
		si := float32(sScaled + gSqScaled) // :791
		var den float32
		if centered { // :797-824
			gaScaled := float32(gavg[i] * alpha)
			gTerm := float32(gi * oma)
			ga := float32(gaScaled + gTerm)
			gaSq := float32(ga * ga)
			variance := float32(si - gaSq)
			varEps := float32(variance + eps)
			den = sqrt32(varEps)
			gavg[i] = ga
		} else { // :827-830
			sEps := float32(si + eps)
			den = sqrt32(sEps)
		}
		upd := float32(gi / den) // :834
		if momentum > 0 {        // :839-854
			bScaled := float32(mom[i] * momentum)
			bi := float32(bScaled + upd)
			mom[i] = bi
			upd = bi
		}
		if weightDecay > 0 { // :857-866
			decay := float32(wi * weightDecay)
			upd = float32(upd + decay)
		}
		scaled := float32(upd * lr) // :869
		w[i] = float32(wi - scaled) // :874
		s[i] = si
	}
}

// OracleAdaGradStep: bridge_optimizer.m:1421-1588.
func OracleAdaGradStep(w, g, s []float32, lr, eps, weightDecay float32) {
	for i := range w {
		wi, gi := w[i], g[i]
		if weightDecay > 0 { // :1480-1488
			decay := float32(wi * weightDecay)
			gi = float32(gi + decay)
		}
		gSq := float32(gi * gi)    // :1492
		si := float32(s[i] + gSq)  // :1495
		root := sqrt32(si)         // :1501
		den := float32(root + eps) // :1503
		alr := float32(lr / den)   // :1506
		upd := float32(alr * gi)   // :1512
		w[i] = float32(wi - upd)   // :1515
		s[i] = si
	}
}

// OracleAdaDeltaStep: bridge_optimizer.m:1708-1925 (the OLD accumulated update feeds the numerator).
func OracleAdaDeltaStep(w, g, s, a []float32, rho, eps, weightDecay float32) {
	omr := float32(1.0 - rho)
	for i := range w {
		wi, gi, ai := w[i], g[i], a[i]
		if weightDecay > 0 { // :1773-1781
			decay := float32(wi * weightDecay)
			gi = float32(gi + decay)
		}
		gSq := float32(gi * gi)            // :1785
		sScaled := float32(s[i] * rho)     // :1788
		gSqScaled := float32(gSq * omr)    // :1791
		si := float32(sScaled + gSqScaled) // :1794
		sEps := float32(si + eps)          // :1800
		rmsG := sqrt32(sEps)               // :1803
		aEps := float32(ai + eps)          // :1807
		rmsU := sqrt32(aEps)               // :1810
		alr := float32(rmsU / rmsG)        // :1815
		d := float32(alr * gi)             // :1818
		negD := -d                         // :1821
		w[i] = float32(wi + negD)          // :1826
		dSq := float32(negD * negD)        // :1832
		aScaled := float32(ai * rho)       // :1835
		dSqScaled := float32(dSq * omr)    // :1838
		a[i] = float32(aScaled + dSqScaled) // :1841
		s[i] = si
	}
}

// OracleNadamStep: bridge_optimizer.m:2023-2280 (the momentum schedule is taken at step + 1, :2066).
func OracleNadamStep(w, g, m, v []float32, lr, beta1, beta2, eps, weightDecay float32, step int) {
	bc1, bc2 := cgo_bridge.BiasCorrections(beta1, beta2, step) // :2061-2062
	mu := cgo_bridge.NadamMuNext(beta1, step)                  // :2066
	oneMinusMu := float32(1.0 - mu)                            // :2153
	omb1 := float32(1.0 - beta1)
	omb2 := float32(1.0 - beta2)
	for i := range w {
		wi, gi := w[i], g[i]
		mScaled := float32(m[i] * beta1)      // :2114
		gScaled := float32(gi * omb1)         // :2117
		mi := float32(mScaled + gScaled)      // :2120
		gSq := float32(gi * gi)               // :2125
		vScaled := float32(v[i] * beta2)      // :2128
		gSqScaled := float32(gSq * omb2)      // :2131
		vi := float32(vScaled + gSqScaled)    // :2134
		vHat := float32(vi / bc2)             // :2139
		mHat := float32(mi / bc1)             // :2145
		gHat := float32(gi / bc1)             // :2148
		mTerm := float32(mHat * mu)           // :2158
		gTerm := float32(gHat * oneMinusMu)   // :2161
		mBar := float32(mTerm + gTerm)        // :2164
		root := sqrt32(vHat)                  // :2170
		den := float32(root + eps)            // :2171
		upd := float32(mBar / den)            // :2176
		if weightDecay > 0 {                  // :2181-2190
			decay := float32(wi * weightDecay)
			upd = float32(upd + decay)
		}
		scaled := float32(upd * lr) // :2193
		w[i] = float32(wi - scaled) // :2198
		m[i] = mi
		v[i] = vi
	}
}

// Float16ToFloat32 / Float32ToFloat16: the casts of bridge_memory.m:361-377 on bit patterns (exact widening;
// narrowing rounds to nearest, ties to even, overflows to infinity and quiets NaNs).
func Float16ToFloat32(h uint16) float32 {
	sign := (uint32(h) & 0x8000) << 16
	exp := (uint32(h) >> 10) & 0x1F
	man := uint32(h) & 0x3FF
	var u uint32
	switch {
	case exp == 0x1F:
		u = sign | 0x7F800000 | (man << 13)
	case exp != 0:
		u = sign | ((exp - 15 + 127) << 23) | (man << 13)
	case man == 0:
		u = sign
	default: // subnormal half: normalise
		e := uint32(0)
		man <<= 1
		for man&0x400 == 0 {
			e++
			man <<= 1
		}
		u = sign | ((127 - 15 - e) << 23) | ((man & 0x3FF) << 13)
	}
	return math.Float32frombits(u)
}

func Float32ToFloat16(x float32) uint16 {
	u := math.Float32bits(x)
	sign := (u >> 16) & 0x8000
	exp := (u >> 23) & 0xFF
	man := u & 0x7FFFFF
	if exp == 0xFF { // inf / NaN
		if man == 0 {
			return uint16(sign | 0x7C00)
		}
		return uint16(sign | 0x7E00 | (man >> 13)) // quiet NaN, top payload bits kept
	}
	e := int32(exp) - 127 + 15 // biased half exponent
	if e >= 0x1F {
		return uint16(sign | 0x7C00) // overflow before rounding
	}
	if e <= 0 { // subnormal half or zero
		if e < -10 {
			return uint16(sign)
		}
		full := man | 0x800000
		shift := uint32(14 - e) // 14..24
		q := full >> shift
		rem := full & ((1 << shift) - 1)
		halfway := uint32(1) << (shift - 1)
		if rem > halfway || (rem == halfway && q&1 != 0) {
			q++
		}
		return uint16(sign | q) // q may carry into the normal range
	}
	q := (uint32(e) << 10) | (man >> 13)
	rem := man & 0x1FFF
	if rem > 0x1000 || (rem == 0x1000 && q&1 != 0) {
		q++ // may carry up to infinity
	}
	return uint16(sign | q)
}

// OracleAMPState is the loss-scale state machine of the mixed-precision step (constants of
// training/model_trainer.go:258-270; rule of docs/tutorials/mixed-precision.md:610-629).
type OracleAMPState struct {
	Scale          float32
	GrowthTracker  int
	GrowthFactor   float32
	BackoffFactor  float32
	GrowthInterval int
	StepCount      uint64
}

// OracleAdamAMPStep runs one mixed-precision Adam step over a tensor list: fp16 gradients of the scaled loss
// (bit patterns), fp32 weights and moments, fp16 copy of the new weights.  Returns true when a gradient held
// an inf / NaN: nothing is written, the scale is multiplied by the backoff factor (it stays a normal number)
// and the clean-step counter is reset; otherwise StepCount advances, every element takes the Adam rule on
// float(g16) * (1 / scale), and the scale grows when the counter reaches the interval (never to +Inf).
func OracleAdamAMPStep(w [][]float32, g16 [][]uint16, m, v [][]float32, w16 [][]uint16,
	lr, beta1, beta2, eps, weightDecay float32, st *OracleAMPState) (skipped bool) {
	for _, g := range g16 {
		for _, h := range g {
			if h&0x7C00 == 0x7C00 {
				skipped = true
			}
		}
	}
	if skipped {
		next := float32(st.Scale * st.BackoffFactor)
		if next >= fltMin { // the scale stays a normal number
			st.Scale = next
		}
		st.GrowthTracker = 0
		return true
	}
	st.StepCount++
	bc1, bc2 := cgo_bridge.BiasCorrections(beta1, beta2, int(st.StepCount))
	omb1 := float32(1.0 - beta1)
	omb2 := float32(1.0 - beta2)
	invScale := float32(1.0 / st.Scale)
	for t := range w {
		for i := range w[t] {
			gi := float32(Float16ToFloat32(g16[t][i]) * invScale)
			adamElement(&w[t][i], &m[t][i], &v[t][i], gi, lr, beta1, beta2, omb1, omb2, eps, weightDecay, bc1, bc2)
			if w16 != nil && w16[t] != nil {
				w16[t][i] = Float32ToFloat16(w[t][i])
			}
		}
	}
	st.GrowthTracker++
	if st.GrowthTracker == st.GrowthInterval {
		next := float32(st.Scale * st.GrowthFactor)
		if next <= math.MaxFloat32 { // "up to maximum": never +Inf
			st.Scale = next
		}
		st.GrowthTracker = 0
	}
	return false
}
