//go:build linux && amd64

package memory

// Placement of optimizer state buffers.  Additive to manager.go.
//
// hipMalloc aligns large buffers to 2 MiB, so element i of a tensor's weight, gradient and state buffers has
// the same low address bits in all of them and lands on the same HBM channel at the same moment.  The
// optimizers therefore ask for their state buffers of the 16 MiB tier and above at phases of their own: the
// first, second and third state of a tensor start 512 KiB, 1.5 MiB and 1 MiB past a 2 MiB boundary (worth
// about half a point to a point of bandwidth for Adam over large tensors; 2 MiB of padding per buffer).
//
// The constructors call AllocateStateBuffer(size, j) where they call AllocateBuffer(size) for their j-th state
// (adam.go:104, 112 and the same loops in sgd.go, rmsprop.go, adagrad.go, adadelta.go, nadam.go).  Placed
// buffers are pooled apart from the others, by (size, phase); ReleaseBuffer (manager.go:299) gets one line at
// its top so that it hands them back to the right pool:
//
//	if mm.releasePlaced(buffer) { return }

import (
	"sync"
	"unsafe"

	"github.com/tsawler/go-metal/cgo_bridge"
)

// StatePhases: where the j-th state buffer of a tensor starts, in bytes modulo 2 MiB.
var StatePhases = [3]int{512 << 10, 1536 << 10, 1 << 20}

// ShadowWeightPhase: where the second weight set of the ping-pong mixed-precision step starts (its moments
// start at the phases of their counterparts).
const ShadowWeightPhase = 1 << 20

// PhasedMinBytes: buffers below the 16 MiB tier are not placed (their padding would outweigh them).
const PhasedMinBytes = 16 << 20

type placedKey struct {
	Size  int
	Phase int
}

// placedPools holds what manager.go's structs have no fields for: per manager, the free lists of placed
// buffers and the key each placed buffer in use belongs to.
type placedPools struct {
	mu   sync.Mutex
	free map[placedKey][]unsafe.Pointer
	used map[unsafe.Pointer]placedKey
}

var placedByManager sync.Map // *MemoryManager -> *placedPools

func (mm *MemoryManager) placed() *placedPools {
	if v, ok := placedByManager.Load(mm); ok {
		return v.(*placedPools)
	}
	v, _ := placedByManager.LoadOrStore(mm, &placedPools{
		free: make(map[placedKey][]unsafe.Pointer),
		used: make(map[unsafe.Pointer]placedKey),
	})
	return v.(*placedPools)
}

// AllocateStateBuffer is AllocateBuffer (manager.go:289-296) for the stateIndex-th state buffer of a tensor
// (0, 1 or 2): nil on failure, returned with ReleaseBuffer.
func (mm *MemoryManager) AllocateStateBuffer(size int, stateIndex int) unsafe.Pointer {
	phase := 0
	if stateIndex >= 0 && stateIndex < len(StatePhases) {
		phase = StatePhases[stateIndex]
	}
	return mm.AllocateBufferAtPhase(size, phase)
}

// AllocateBufferAtPhase is AllocateBuffer with the start of the buffer at `phase` bytes modulo 2 MiB (a
// multiple of 256).  Requests whose tier is below PhasedMinBytes, and phase 0, are ordinary allocations.
func (mm *MemoryManager) AllocateBufferAtPhase(size int, phase int) unsafe.Pointer {
	poolSize := mm.findPoolSize(size)
	if phase == 0 || poolSize < PhasedMinBytes {
		return mm.AllocateBuffer(size)
	}
	key := placedKey{Size: poolSize, Phase: phase}
	p := mm.placed()
	p.mu.Lock()
	if list := p.free[key]; len(list) > 0 {
		buffer := list[len(list)-1]
		p.free[key] = list[:len(list)-1]
		p.used[buffer] = key
		p.mu.Unlock()
		return buffer
	}
	p.mu.Unlock()
	buffer, err := cgo_bridge.AllocateMetalBufferPhased(mm.device, poolSize, cgo_bridge.GPU, phase)
	if err != nil {
		return nil
	}
	p.mu.Lock()
	p.used[buffer] = key
	p.mu.Unlock()
	return buffer
}

// releasePlaced takes a placed buffer back into its (size, phase) free list; false for any other buffer.
func (mm *MemoryManager) releasePlaced(buffer unsafe.Pointer) bool {
	v, ok := placedByManager.Load(mm)
	if !ok {
		return false
	}
	p := v.(*placedPools)
	p.mu.Lock()
	defer p.mu.Unlock()
	key, ok := p.used[buffer]
	if !ok {
		return false
	}
	delete(p.used, buffer)
	p.free[key] = append(p.free[key], buffer)
	return true
}
