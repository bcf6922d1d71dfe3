// Host-side mirror of memory/tensor.go and of the precomputed-gradient step of
// engine/training_engine.go.
#include "tensor.hpp"

#include "optimizer.hpp"

#include "../../include/gometal_hip.h"

namespace gometal {
namespace memory {

static std::atomic<uint64_t> globalGeneration{0};

static std::string shapeString(const std::vector<int> &shape)   // Go's %v of []int
{
    std::string s = "[";
    for (size_t i = 0; i < shape.size(); i++) {
        if (i) s += " ";
        s += std::to_string(shape[i]);
    }
    return s + "]";
}

static int elementCount(const std::vector<int> &shape)
{
    int n = 1;
    for (int d : shape) n *= d;
    return n;
}

int calculateSize(const std::vector<int> &shape, DataType dtype)
{
    if (shape.empty()) return 0;
    int elementSize;
    switch (dtype) {
    case Float32:
    case Int32: elementSize = 4; break;
    case Float16: elementSize = 2; break;
    case Int8: elementSize = 1; break;
    default: return -1;
    }
    return elementCount(shape) * elementSize;
}

std::pair<Tensor *, Error> Tensor::NewTensor(const std::vector<int> &shape, DataType dtype, DeviceType device)
{
    const int size = calculateSize(shape, dtype);
    if (size < 0) return {nullptr, Errorf("unsupported data type: %d", (int)dtype)};
    MemoryManager *mm = GetGlobalMemoryManager();
    if (!mm)
        return {nullptr, Errorf("failed to allocate buffer: global memory manager not initialized - call "
                                "InitializeGlobalMemoryManager first")};
    auto [buffer, err] = mm->GetBuffer(size, device);
    if (!err.empty()) return {nullptr, Errorf("failed to allocate buffer: %s", err.c_str())};
    Tensor *t = new Tensor();
    t->metalBuffer_ = buffer;
    t->shape_ = shape;
    t->dtype_ = dtype;
    t->device_ = device;
    t->generation_ = globalGeneration.fetch_add(1) + 1;
    t->size_ = size;
    return {t, ""};
}

Tensor *Tensor::Retain()
{
    if (released_) return nullptr;
    refCount_.fetch_add(1);
    return this;
}

void Tensor::Release()
{
    if (released_) return;
    if (refCount_.fetch_sub(1) == 1) {
        if (pooled_ && metalBuffer_ != nullptr) GetGlobalMemoryManager()->ReturnBuffer(metalBuffer_, size_, device_);
        metalBuffer_ = nullptr;
        released_ = true;
        shape_.clear();
    }
}

std::pair<Tensor *, Error> Tensor::ConvertTo(DataType dtype)
{
    if (dtype_ == dtype) return {Retain(), ""};
    auto [newTensor, err] = NewTensor(shape_, dtype, device_);
    if (!err.empty()) return {nullptr, Errorf("failed to create converted tensor: %s", err.c_str())};
    Error cerr = cgo_bridge::ConvertTensorType(metalBuffer_, newTensor->metalBuffer_, shape_, (int)dtype_, (int)dtype,
                                               GetDevice());
    if (!cerr.empty()) {
        newTensor->Release();
        delete newTensor;
        return {nullptr, Errorf("failed to convert tensor type: %s", cerr.c_str())};
    }
    return {newTensor, ""};
}

Error Tensor::CopyFloat32Data(const std::vector<float> &data)
{
    if (dtype_ != Float32) return Errorf("tensor data type is %d, expected Float32 (%d)", (int)dtype_, (int)Float32);
    const int expected = elementCount(shape_);
    if ((int)data.size() != expected)
        return Errorf("data length %d doesn't match tensor shape %s (expected %d elements)", (int)data.size(),
                      shapeString(shape_).c_str(), expected);
    return cgo_bridge::CopyFloat32ArrayToMetalBuffer(metalBuffer_, data);
}

Error Tensor::CopyInt32Data(const std::vector<int32_t> &data)
{
    if (dtype_ != Int32) return Errorf("tensor data type is %d, expected Int32 (%d)", (int)dtype_, (int)Int32);
    const int expected = elementCount(shape_);
    if ((int)data.size() != expected)
        return Errorf("data length %d doesn't match tensor shape %s (expected %d elements)", (int)data.size(),
                      shapeString(shape_).c_str(), expected);
    if (data.empty()) return "";
    int rc = copy_int32_array_to_metal_buffer(reinterpret_cast<uintptr_t>(metalBuffer_),
                                              const_cast<int *>(reinterpret_cast<const int *>(data.data())),
                                              (int)data.size());
    if (rc != 0) return Errorf("failed to copy int32 array to Metal buffer with error code: %d", rc);
    return "";
}

Error Tensor::CopyFrom(const Tensor *src)
{
    if (src == nullptr) return Errorf("source tensor is nil");
    if (metalBuffer_ == nullptr) return Errorf("destination tensor has nil metal buffer");
    if (src->metalBuffer_ == nullptr) return Errorf("source tensor has nil metal buffer");
    if (shape_.size() != src->shape_.size())
        return Errorf("tensor shape dimensions don't match: dst %s vs src %s", shapeString(shape_).c_str(),
                      shapeString(src->shape_).c_str());
    for (size_t i = 0; i < shape_.size(); i++)
        if (shape_[i] != src->shape_[i])
            return Errorf("tensor shapes don't match: dst %s vs src %s", shapeString(shape_).c_str(),
                          shapeString(src->shape_).c_str());
    if (dtype_ != src->dtype_)
        return Errorf("tensor data types don't match: dst %d vs src %d", (int)dtype_, (int)src->dtype_);
    if (src->size_ != size_)
        return Errorf("tensor sizes don't match: dst %d bytes vs src %d bytes", size_, src->size_);
    return cgo_bridge::CopyTensorBufferSync(src->metalBuffer_, metalBuffer_, size_);
}

std::pair<std::vector<float>, Error> Tensor::ToFloat32Slice()
{
    if (dtype_ != Float32)
        return {{}, Errorf("tensor data type is %d, expected Float32 (%d)", (int)dtype_, (int)Float32)};
    const int expected = elementCount(shape_);
    if (expected <= 0) return {{}, Errorf("tensor has invalid shape: %s", shapeString(shape_).c_str())};
    return cgo_bridge::CopyMetalBufferToFloat32Array(metalBuffer_, expected);
}

std::string Tensor::String() const
{
    return Errorf("Tensor{shape=%s, dtype=%d, device=%d, refs=%d, gen=%llu}", shapeString(shape_).c_str(), (int)dtype_,
                  (int)device_, (int)RefCount(), (unsigned long long)generation_);
}

Pointer GetDevice()
{
    MemoryManager *mm = GetGlobalMemoryManager();
    return mm ? mm->device() : nullptr;
}

}  // namespace memory

namespace engine {

Error ExecuteStepWithPrecomputedGradients(optimizer::Optimizer *opt, const std::vector<memory::Tensor *> &weightTensors,
                                          const std::vector<memory::Tensor *> &gradientTensors, const char *what)
{
    if (opt == nullptr) return Errorf("%s optimizer not initialized", what);
    if (weightTensors.size() != gradientTensors.size())
        return Errorf("weight tensors (%d) and gradient tensors (%d) count mismatch", (int)weightTensors.size(),
                      (int)gradientTensors.size());
    std::vector<Pointer> weightBuffers(weightTensors.size());
    for (size_t i = 0; i < weightTensors.size(); i++) {
        if (weightTensors[i] == nullptr) return Errorf("weight tensor %d is nil", (int)i);
        weightBuffers[i] = weightTensors[i]->MetalBuffer();
    }
    Error err = opt->SetWeightBuffers(weightBuffers);
    if (!err.empty()) return Errorf("failed to set weight buffers: %s", err.c_str());
    std::vector<Pointer> gradientBuffers(gradientTensors.size());
    for (size_t i = 0; i < gradientTensors.size(); i++) {
        if (gradientTensors[i] == nullptr) return Errorf("gradient tensor %d is nil", (int)i);
        gradientBuffers[i] = gradientTensors[i]->MetalBuffer();
    }
    err = opt->Step(gradientBuffers);
    if (!err.empty()) return Errorf("%s optimization step failed: %s", what, err.c_str());
    return "";
}

}  // namespace engine
}  // namespace gometal
