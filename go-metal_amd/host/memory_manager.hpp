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
    BufferPool(int bufferSize, int maxSize, DeviceType device);
    ~BufferPool();
    std::pair<Pointer, Error> Get();
    void Return(Pointer buffer);
    void Stats(int *available, int *allocated, int *maxSize);

private:
    std::deque<Pointer> buffers_;   // available buffers (the Go channel)
    int maxSize_;
    int bufferSize_;
    DeviceType device_;
    int allocated_ = 0;
    std::mutex mutex_;
};

// memory/manager.go:103-106
struct PoolKey {
    int Size;
    DeviceType Device;
    bool operator<(const PoolKey &o) const { return Size != o.Size ? Size < o.Size : Device < o.Device; }
};

// memory/manager.go:88-240
class MemoryManager {
public:
    explicit MemoryManager(Pointer device);
    std::pair<Pointer, Error> GetBuffer(int size, DeviceType device);
    void ReturnBuffer(Pointer buffer, int size, DeviceType device);
    Pointer AllocateBuffer(int size);          // nullptr on failure (manager.go:289-296)
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
