// Host-side mirror of the Go package `memory` (memory/manager.go): a size-tiered pool of
// device buffers.  Same type and method names, same tier table and rounding, same "nil on
// failure" convention.  The buffers come from allocate_metal_buffer (hipMalloc on HBM).
//
// One deliberate difference: the per-pool buffer caps.  The reference caps a pool at
// 100 / 50 / 20 / 20 / 15 buffers by size class (memory/manager.go:210-224); 15 buffers of
// 64 MB cannot hold the optimizer state of a transformer-sized parameter list (28 tensors of
// 64 MB need 56 state buffers for Adam).  Here a pool may grow to the reference's cap or to
// the number of buffers that fit a byte budget (default 128 GiB of the GPU's 288 GB),
// whichever is larger.
#pragma once

#include "bridge.hpp"

#include <cstddef>
#include <deque>
#include <map>
#include <memory>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

namespace gometal {
namespace memory {

// memory/tensor.go:20-26
enum DeviceType : int { CPU = 0, GPU = 1, PersistentGPU = 2 };

// memory/manager.go:12-86
class BufferPool {
public:
    BufferPool(int bufferSize, int maxSize, DeviceType device, int phase = 0);
    ~BufferPool();
    std::pair<Pointer, Error> Get();
    void Return(Pointer buffer);
    void Stats(int *available, int *allocated, int *maxSize);

private:
    std::deque<Pointer> buffers_;   // available buffers (the Go channel)
    int maxSize_;
    int bufferSize_;
    DeviceType device_;
    int phase_;                     // where this pool's buffers start, in bytes modulo 2 MiB (0: wherever hipMalloc puts them)
    int allocated_ = 0;
    std::mutex mutex_;
};

// memory/manager.go:103-106
struct PoolKey {
    int Size;
    DeviceType Device;
    int Phase = 0;      // not in the reference: buffers placed at a phase are pooled apart from the others
    bool operator<(const PoolKey &o) const
    {
        if (Size != o.Size) return Size < o.Size;
        if (Device != o.Device) return Device < o.Device;
        return Phase < o.Phase;
    }
};

// Where the optimizers put the state buffers of a tensor: first, second and third state start at these
// phases (bytes modulo 2 MiB), away from the 2 MiB-aligned starts hipMalloc gives the weights and
// gradients, so that element i of a tensor's streams does not land on one HBM channel for all of
// them at once (measured on MI355X, Adam over 1.012B parameters: 83.1 % of peak against 82.0 %).
constexpr int kStatePhases[3] = {512 << 10, 1536 << 10, 1 << 20};
// The second set of the ping-pong mixed-precision step: its moments at the phases of their counterparts, its
// weights 1 MiB off.
constexpr int kShadowWeightPhase = 1 << 20;
// Placing a buffer costs 2 MiB of padding: only the tiers from 16 MiB up (an eighth more memory at
// most) are placed, smaller requests take the ordinary pools.
constexpr int kPhasedMinBytes = 16 << 20;

// memory/manager.go:88-240
class MemoryManager {
public:
    explicit MemoryManager(Pointer device);
    std::pair<Pointer, Error> GetBuffer(int size, DeviceType device, int phase = 0);
    void ReturnBuffer(Pointer buffer, int size, DeviceType device, int phase = 0);
    Pointer AllocateBuffer(int size);          // nullptr on failure (manager.go:289-296)
    // AllocateBuffer for the stateIndex-th state buffer of a tensor (0, 1, 2): large ones start at
    // kStatePhases[stateIndex]; ReleaseBuffer takes them back like any other.
    Pointer AllocateStateBuffer(int size, int stateIndex);
    // AllocateBuffer at a phase of the caller's choosing (bytes modulo 2 MiB, a multiple of 256).
    Pointer AllocateBufferAtPhase(int size, int phase);
    void ReleaseBuffer(Pointer buffer);        // manager.go:299-317
    std::map<PoolKey, std::string> Stats();
    int findPoolSize(int size) const;          // manager.go:172-180
    Pointer device() const { return device_; }

private:
    BufferPool *getOrCreatePool(const PoolKey &key);
    std::map<PoolKey, std::unique_ptr<BufferPool>> pools_;
    std::mutex poolsMutex_;
    Pointer device_;
    std::vector<int> poolSizes_;
    std::unordered_map<Pointer, int> bufferSizes_;
    std::unordered_map<Pointer, int> bufferPhases_;   // only buffers with a non-zero phase
    std::mutex bufferSizesMutex_;
};

// memory/manager.go:210-224, with the byte-budget extension described above.
int calculateMaxPoolSize(int bufferSize);
// The reference's cap table alone (memory/memory_test.go:242-255 pins these values).
int referenceMaxPoolSize(int bufferSize);
// Bytes a single pool may hold before Get() reports "buffer pool at capacity".
void SetPoolByteBudget(size_t bytes);

// memory/manager.go:242-258.  The first call wins, as with sync.Once.
void InitializeGlobalMemoryManager(Pointer device);
MemoryManager *GetGlobalMemoryManager();       // nullptr (Go: panic) before initialisation

// memory/manager.go:322-333
Pointer CreateMockDevice();
Pointer CreateMockCommandQueue();

}  // namespace memory
}  // namespace gometal
