// Host-side mirror of memory/tensor.go: a reference-counted tensor over a pooled device
// buffer, with GPU-side type conversion and GPU-to-GPU copy.  Same method names and error
// strings.  The Go code reaches the bridge through function variables to avoid an import
// cycle; here the calls are direct.
#pragma once

#include "memory_manager.hpp"

#include <atomic>
#include <string>
#include <vector>

namespace gometal {
namespace memory {

// memory/tensor.go:10-17
enum DataType : int { Float32 = 0, Int32 = 1, Float16 = 2, Int8 = 3 };

// memory/tensor.go:137-164.  -1 for an unsupported dtype (Go: panic).
int calculateSize(const std::vector<int> &shape, DataType dtype);

class Tensor {
public:
    // memory/tensor.go:41-66
    static std::pair<Tensor *, Error> NewTensor(const std::vector<int> &shape, DataType dtype, DeviceType device);

    Tensor *Retain();                 // tensor.go:69-75; nullptr if already released (Go: panic)
    void Release();                   // tensor.go:78-93
    Tensor *Clone() { return Retain(); }
    std::vector<int> Shape() const { return shape_; }
    DataType DType() const { return dtype_; }
    DeviceType Device() const { return device_; }
    Pointer MetalBuffer() const { return metalBuffer_; }   // nullptr after release (Go: panic)
    int Size() const { return size_; }
    int32_t RefCount() const { return released_ ? 0 : refCount_.load(); }
    std::pair<Tensor *, Error> ConvertTo(DataType dtype);      // tensor.go:166-186
    Error CopyFloat32Data(const std::vector<float> &data);     // tensor.go:189-206
    Error CopyInt32Data(const std::vector<int32_t> &data);     // tensor.go:209-226
    Error CopyFrom(const Tensor *src);                         // tensor.go:248-291
    std::pair<std::vector<float>, Error> ToFloat32Slice();     // tensor.go:341-360
    std::string String() const;                                // tensor.go:363-366

private:
    Tensor() = default;
    Pointer metalBuffer_ = nullptr;
    std::vector<int> shape_;
    DataType dtype_ = Float32;
    DeviceType device_ = GPU;
    std::atomic<int32_t> refCount_{1};
    bool released_ = false;
    bool pooled_ = true;
    uint64_t generation_ = 0;
    int size_ = 0;
};

// memory/tensor.go:306-308
Pointer GetDevice();

}  // namespace memory

namespace optimizer {
class Optimizer;
}

namespace engine {
// engine/training_engine.go:100-147: the thinnest caller of the hot path.  Tensors ->
// buffer handles -> SetWeightBuffers -> Step.  `what` names the optimizer in the error
// text ("Adam" in the reference).
Error ExecuteStepWithPrecomputedGradients(optimizer::Optimizer *opt, const std::vector<memory::Tensor *> &weightTensors,
                                          const std::vector<memory::Tensor *> &gradientTensors,
                                          const char *what = "Adam");
}  // namespace engine
}  // namespace gometal
