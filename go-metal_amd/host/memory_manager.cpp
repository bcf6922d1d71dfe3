// Host-side mirror of memory/manager.go.
#include "memory_manager.hpp"

#include <atomic>
#include <cstdio>

namespace gometal {
namespace memory {

static std::atomic<size_t> g_pool_byte_budget{(size_t)128 << 30};

void SetPoolByteBudget(size_t bytes) { g_pool_byte_budget.store(bytes); }

// Default pool sizes: 1KB, 4KB, 16KB, 64KB, 256KB, 1MB, 4MB, 16MB, 64MB (manager.go:109-111)
static const int kDefaultPoolSizes[] = {1024, 4096, 16384, 65536, 262144, 1048576, 4194304, 16777216, 67108864};

int referenceMaxPoolSize(int bufferSize)
{
    if (bufferSize <= 4096) return 100;
    if (bufferSize <= 65536) return 50;
    if (bufferSize <= 1048576) return 20;
    if (bufferSize <= 16777216) return 20;
    return 15;
}

int calculateMaxPoolSize(int bufferSize)
{
    const int ref = referenceMaxPoolSize(bufferSize);
    if (bufferSize <= 0) return ref;
    const size_t by_budget = g_pool_byte_budget.load() / (size_t)bufferSize;
    const size_t capped = by_budget > 1000000 ? 1000000 : by_budget;
    return (int)capped > ref ? (int)capped : ref;
}

static std::pair<Pointer, Error> allocateMetalBuffer(int size, DeviceType device, int phase)
{
    // manager.go:263-281: the device comes from the global manager
    MemoryManager *global = GetGlobalMemoryManager();
    if (!global) return {nullptr, Errorf("global memory manager not initialized - call InitializeGlobalMemoryManager first")};
    cgo_bridge::DeviceType cgoDev;
    switch (device) {
    case CPU: cgoDev = cgo_bridge::CPU; break;
    case GPU: cgoDev = cgo_bridge::GPU; break;
    case PersistentGPU: cgoDev = cgo_bridge::PersistentGPU; break;
    default: cgoDev = cgo_bridge::GPU; break;
    }
    if (phase != 0) return cgo_bridge::AllocateMetalBufferPhased(global->device(), size, cgoDev, phase);
    return cgo_bridge::AllocateMetalBuffer(global->device(), size, cgoDev);
}

static void deallocateMetalBuffer(Pointer buffer) { cgo_bridge::DeallocateMetalBuffer(buffer); }

BufferPool::BufferPool(int bufferSize, int maxSize, DeviceType device, int phase)
    : maxSize_(maxSize), bufferSize_(bufferSize), device_(device), phase_(phase)
{
}

BufferPool::~BufferPool()
{
    for (Pointer p : buffers_) deallocateMetalBuffer(p);
}

std::pair<Pointer, Error> BufferPool::Get()
{
    {
        std::lock_guard<std::mutex> lk(mutex_);
        if (!buffers_.empty()) {
            Pointer p = buffers_.front();
            buffers_.pop_front();
            return {p, ""};
        }
        if (allocated_ >= maxSize_) return {nullptr, Errorf("buffer pool at capacity (%d)", maxSize_)};
        allocated_++;
    }
    auto [buffer, err] = allocateMetalBuffer(bufferSize_, device_, phase_);
    if (!err.empty()) {
        std::lock_guard<std::mutex> lk(mutex_);
        allocated_--;
        return {nullptr, Errorf("failed to allocate Metal buffer: %s", err.c_str())};
    }
    return {buffer, ""};
}

void BufferPool::Return(Pointer buffer)
{
    if (buffer == nullptr) return;
    bool pooled = false;
    {
        std::lock_guard<std::mutex> lk(mutex_);
        if ((int)buffers_.size() < maxSize_) {
            buffers_.push_back(buffer);
            pooled = true;
        } else {
            allocated_--;
        }
    }
    if (!pooled) deallocateMetalBuffer(buffer);   // pool is full
}

void BufferPool::Stats(int *available, int *allocated, int *maxSize)
{
    std::lock_guard<std::mutex> lk(mutex_);
    if (available) *available = (int)buffers_.size();
    if (allocated) *allocated = allocated_;
    if (maxSize) *maxSize = maxSize_;
}

MemoryManager::MemoryManager(Pointer device)
    : device_(device), poolSizes_(std::begin(kDefaultPoolSizes), std::end(kDefaultPoolSizes))
{
}

int MemoryManager::findPoolSize(int size) const
{
    for (int poolSize : poolSizes_)
        if (poolSize >= size) return poolSize;
    return size;   // larger than the largest tier: the requested size itself
}

BufferPool *MemoryManager::getOrCreatePool(const PoolKey &key)
{
    std::lock_guard<std::mutex> lk(poolsMutex_);
    auto it = pools_.find(key);
    if (it != pools_.end()) return it->second.get();
    auto pool = std::make_unique<BufferPool>(key.Size, calculateMaxPoolSize(key.Size), key.Device, key.Phase);
    BufferPool *raw = pool.get();
    pools_[key] = std::move(pool);
    return raw;
}

std::pair<Pointer, Error> MemoryManager::GetBuffer(int size, DeviceType device, int phase)
{
    const int poolSize = findPoolSize(size);
    if (poolSize < kPhasedMinBytes) phase = 0;
    BufferPool *pool = getOrCreatePool(PoolKey{poolSize, device, phase});
    auto [buffer, err] = pool->Get();
    if (!err.empty()) return {nullptr, err};
    std::lock_guard<std::mutex> lk(bufferSizesMutex_);
    bufferSizes_[buffer] = poolSize;
    if (phase != 0) bufferPhases_[buffer] = phase;
    return {buffer, ""};
}

void MemoryManager::ReturnBuffer(Pointer buffer, int size, DeviceType device, int phase)
{
    if (buffer == nullptr) return;
    const int poolSize = findPoolSize(size);
    if (poolSize < kPhasedMinBytes) phase = 0;
    const PoolKey key{poolSize, device, phase};
    BufferPool *pool = nullptr;
    {
        std::lock_guard<std::mutex> lk(poolsMutex_);
        auto it = pools_.find(key);
        if (it != pools_.end()) pool = it->second.get();
    }
    if (pool) pool->Return(buffer);
    else deallocateMetalBuffer(buffer);   // no pool exists, just deallocate
    std::lock_guard<std::mutex> lk(bufferSizesMutex_);
    bufferSizes_.erase(buffer);
    bufferPhases_.erase(buffer);
}

Pointer MemoryManager::AllocateBuffer(int size)
{
    auto [buffer, err] = GetBuffer(size, GPU);
    if (!err.empty()) return nullptr;
    return buffer;
}

Pointer MemoryManager::AllocateStateBuffer(int size, int stateIndex)
{
    const int phase = stateIndex >= 0 && stateIndex < 3 ? kStatePhases[stateIndex] : 0;
    auto [buffer, err] = GetBuffer(size, GPU, phase);
    if (!err.empty()) return nullptr;
    return buffer;
}

Pointer MemoryManager::AllocateBufferAtPhase(int size, int phase)
{
    auto [buffer, err] = GetBuffer(size, GPU, phase);
    if (!err.empty()) return nullptr;
    return buffer;
}

void MemoryManager::ReleaseBuffer(Pointer buffer)
{
    if (buffer == nullptr) return;
    int size = 0, phase = 0;
    bool exists = false;
    {
        std::lock_guard<std::mutex> lk(bufferSizesMutex_);
        auto it = bufferSizes_.find(buffer);
        if (it != bufferSizes_.end()) {
            size = it->second;
            exists = true;
        }
        auto ph = bufferPhases_.find(buffer);
        if (ph != bufferPhases_.end()) phase = ph->second;
    }
    if (!exists) {
        size = 4194304;   // 4MB default as fallback (manager.go:309-314)
        std::printf("Warning: releasing untracked buffer %p, using default size %d\n", buffer, size);
    }
    ReturnBuffer(buffer, size, GPU, phase);
}

std::map<PoolKey, std::string> MemoryManager::Stats()
{
    std::lock_guard<std::mutex> lk(poolsMutex_);
    std::map<PoolKey, std::string> stats;
    for (auto &kv : pools_) {
        int available, allocated, maxSize;
        kv.second->Stats(&available, &allocated, &maxSize);
        stats[kv.first] = Errorf("available=%d, allocated=%d, max=%d", available, allocated, maxSize);
    }
    return stats;
}

static MemoryManager *g_global = nullptr;
static std::once_flag g_global_once;

void InitializeGlobalMemoryManager(Pointer device)
{
    std::call_once(g_global_once, [device] { g_global = new MemoryManager(device); });
}

MemoryManager *GetGlobalMemoryManager() { return g_global; }

Pointer CreateMockDevice() { return reinterpret_cast<Pointer>((uintptr_t)0x1000); }
Pointer CreateMockCommandQueue() { return reinterpret_cast<Pointer>((uintptr_t)0x2000); }

}  // namespace memory
}  // namespace gometal
