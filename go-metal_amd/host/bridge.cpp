// Host-side mirror of cgo_bridge/bridge.go (optimizer and buffer wrappers).
#include "bridge.hpp"

#include "../../include/gometal_hip.h"

#include <cstdarg>
#include <cstdio>

namespace gometal {

Error Errorf(const char *fmt, ...)
{
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    return std::string(buf);
}

namespace cgo_bridge {

static inline uintptr_t H(Pointer p) { return reinterpret_cast<uintptr_t>(p); }
static inline Pointer P(uintptr_t h) { return reinterpret_cast<Pointer>(h); }

static std::vector<uintptr_t> handles(const std::vector<Pointer> &v, size_t n)
{
    std::vector<uintptr_t> out(n, 0);
    for (size_t i = 0; i < n && i < v.size(); i++) out[i] = H(v[i]);
    return out;
}

// Go indexes &slice[0]; an empty list has nothing to pass.
static const char *kEmptyList = "buffer arrays must not be empty";

std::pair<Pointer, Error> CreateMetalDevice()
{
    uintptr_t device = create_metal_device();
    if (device == 0) return {nullptr, Errorf("failed to create Metal device")};
    return {P(device), ""};
}

void DestroyMetalDevice(Pointer device)
{
    if (device != nullptr) destroy_metal_device(H(device));
}

std::pair<Pointer, Error> CreateCommandQueue(Pointer device)
{
    if (device == nullptr) return {nullptr, Errorf("device cannot be nil")};
    uintptr_t q = create_command_queue(H(device));
    if (q == 0) return {nullptr, Errorf("failed to create command queue")};
    return {P(q), ""};
}

void ReleaseCommandQueue(Pointer queue)
{
    if (queue != nullptr) release_command_queue(H(queue));
}

std::pair<Pointer, Error> AllocateMetalBuffer(Pointer device, int size, DeviceType deviceType)
{
    uintptr_t buffer = allocate_metal_buffer(H(device), size, (int)deviceType);
    if (buffer == 0) return {nullptr, Errorf("failed to allocate Metal buffer of size %d", size)};
    return {P(buffer), ""};
}

std::pair<Pointer, Error> AllocateMetalBufferPhased(Pointer device, int size, DeviceType deviceType, int phase)
{
    uintptr_t buffer = gm_allocate_buffer_phased(H(device), size, (int)deviceType, phase);
    if (buffer == 0) return {nullptr, Errorf("failed to allocate Metal buffer of size %d", size)};
    return {P(buffer), ""};
}

void DeallocateMetalBuffer(Pointer buffer)
{
    if (buffer != nullptr) deallocate_metal_buffer(H(buffer));
}

Error ZeroMetalBuffer(Pointer device, Pointer buffer, int size)
{
    int result = zero_metal_buffer(H(device), H(buffer), size);
    if (result != 0) return Errorf("failed to zero buffer with error code: %d", result);
    return "";
}

Error CopyFloat32ArrayToMetalBuffer(Pointer buffer, const std::vector<float> &data)
{
    if (data.empty()) return "";   // nothing to copy
    int result = copy_float32_array_to_metal_buffer(H(buffer), const_cast<float *>(data.data()), (int)data.size());
    if (result != 0) return Errorf("failed to copy float32 array to Metal buffer with error code: %d", result);
    return "";
}

std::pair<std::vector<float>, Error> CopyMetalBufferToFloat32Array(Pointer buffer, int numElements)
{
    if (numElements <= 0) return {{}, Errorf("invalid number of elements: %d", numElements)};
    std::vector<float> data((size_t)numElements);
    int result = copy_metal_buffer_to_float32_array(H(buffer), data.data(), numElements);
    if (result != 0)
        return {{}, Errorf("failed to copy Metal buffer to float32 array with error code: %d", result)};
    return {std::move(data), ""};
}

Error ConvertTensorType(Pointer srcBuffer, Pointer dstBuffer, const std::vector<int> &shape, int srcType,
                        int dstType, Pointer device)
{
    if (shape.empty()) return Errorf("shape cannot be empty");
    std::vector<int> cShape(shape);
    int result = convert_tensor_type(H(srcBuffer), H(dstBuffer), cShape.data(), (int)cShape.size(), srcType,
                                     dstType, H(device));
    if (result != 0) return Errorf("failed to convert tensor type with error code: %d", result);
    return "";
}

Error CopyTensorBufferSync(Pointer srcBuffer, Pointer dstBuffer, int size)
{
    if (srcBuffer == nullptr || dstBuffer == nullptr) return Errorf("source or destination buffer is nil");
    if (size <= 0) return Errorf("invalid copy size: %d", size);
    int result = copy_buffer_to_buffer_sync(H(srcBuffer), H(dstBuffer), 0, 0, size);
    if (result != 0) return Errorf("tensor buffer copy failed with error code: %d", result);
    return "";
}

Error ExecuteSGDStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                             const std::vector<Pointer> &gradientBuffers,
                             const std::vector<Pointer> &momentumBuffers, const std::vector<int> &bufferSizes,
                             float learningRate, float momentum, float weightDecay, bool nesterov,
                             int stepCount)
{
    if (weightBuffers.size() != gradientBuffers.size() || weightBuffers.size() != bufferSizes.size())
        return Errorf("weight, gradient, and buffer size arrays must have the same length");
    if (momentum > 0 && weightBuffers.size() != momentumBuffers.size())
        return Errorf("momentum buffers must have same length as weight buffers when momentum > 0");
    const size_t n = weightBuffers.size();
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n);
    // NULL entries for vanilla SGD (bridge.go:925-929)
    auto m = momentum > 0 ? handles(momentumBuffers, n) : std::vector<uintptr_t>(n, 0);
    std::vector<int> sizes(bufferSizes);
    int result = execute_sgd_step_mpsgraph(H(device), n ? w.data() : nullptr, n ? g.data() : nullptr,
                                           n ? m.data() : nullptr, (int)n, n ? sizes.data() : nullptr,
                                           learningRate, momentum, weightDecay, nesterov ? 1 : 0, stepCount);
    if (result != 0) return Errorf("SGD step execution failed with error code: %d", result);
    return "";
}

Error ExecuteAdamStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                              const std::vector<Pointer> &gradientBuffers,
                              const std::vector<Pointer> &momentumBuffers,
                              const std::vector<Pointer> &varianceBuffers, const std::vector<int> &bufferSizes,
                              float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                              int stepCount)
{
    const size_t n = weightBuffers.size();
    if (n != gradientBuffers.size() || n != momentumBuffers.size() || n != varianceBuffers.size() ||
        n != bufferSizes.size())
        return Errorf("all buffer arrays must have the same length");
    if (n == 0) return Errorf("%s", kEmptyList);
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n), m = handles(momentumBuffers, n),
         v = handles(varianceBuffers, n);
    std::vector<int> sizes(bufferSizes);
    int result = execute_adam_step_mpsgraph(H(device), w.data(), g.data(), m.data(), v.data(), (int)n,
                                            sizes.data(), learningRate, beta1, beta2, epsilon, weightDecay,
                                            stepCount);
    if (result != 0) return Errorf("Adam MPSGraph step failed with error code: %d", result);
    return "";
}

Error ExecuteRMSPropStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                                 const std::vector<Pointer> &gradientBuffers,
                                 const std::vector<Pointer> &squaredGradAvgBuffers,
                                 const std::vector<Pointer> &momentumBuffers,
                                 const std::vector<Pointer> &gradientAvgBuffers,
                                 const std::vector<int> &bufferSizes, float learningRate, float alpha,
                                 float epsilon, float weightDecay, float momentum, bool centered,
                                 int stepCount)
{
    const size_t n = weightBuffers.size();
    if (n != gradientBuffers.size() || n != squaredGradAvgBuffers.size() || n != bufferSizes.size())
        return Errorf("weight, gradient, squared gradient average, and buffer size arrays must have the same length");
    if (n == 0) return Errorf("%s", kEmptyList);
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n), s = handles(squaredGradAvgBuffers, n);
    // optional buffers: 0 unless the variant is on and the caller supplied one (bridge.go:1900-1911)
    auto b = momentum > 0.0f ? handles(momentumBuffers, n) : std::vector<uintptr_t>(n, 0);
    auto ga = centered ? handles(gradientAvgBuffers, n) : std::vector<uintptr_t>(n, 0);
    std::vector<int> sizes(bufferSizes);
    int result = execute_rmsprop_step_mpsgraph(H(device), w.data(), g.data(), s.data(), b.data(), ga.data(), (int)n,
                                               sizes.data(), learningRate, alpha, epsilon, weightDecay, momentum,
                                               centered, stepCount);
    if (result != 0) return Errorf("RMSProp MPSGraph step failed with error code: %d", result);
    return "";
}

static Error adagrad_common(bool pooled, Pointer device, const std::vector<Pointer> &weightBuffers,
                            const std::vector<Pointer> &gradientBuffers,
                            const std::vector<Pointer> &squaredGradAvgBuffers, int numWeights,
                            const std::vector<int> &bufferSizes, float learningRate, float epsilon,
                            float weightDecay, Pointer commandPool)
{
    if (device == nullptr) return Errorf("device cannot be nil");
    if ((int)weightBuffers.size() != numWeights || (int)gradientBuffers.size() != numWeights ||
        (int)squaredGradAvgBuffers.size() != numWeights || (int)bufferSizes.size() != numWeights)
        return Errorf("buffer count mismatch: weights=%d, gradients=%d, squared_grad_avg=%d, sizes=%d, expected=%d",
                      (int)weightBuffers.size(), (int)gradientBuffers.size(), (int)squaredGradAvgBuffers.size(),
                      (int)bufferSizes.size(), numWeights);
    if (numWeights <= 0) return Errorf("%s", kEmptyList);
    const size_t n = (size_t)numWeights;
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n), s = handles(squaredGradAvgBuffers, n);
    std::vector<int> sizes(bufferSizes);
    int result;
    if (pooled) {
        result = execute_adagrad_step_mpsgraph_pooled(H(device), w.data(), g.data(), s.data(), numWeights,
                                                      sizes.data(), learningRate, epsilon, weightDecay,
                                                      H(commandPool));
        if (result != 0) return Errorf("AdaGrad MPSGraph pooled step failed with error code: %d", result);
    } else {
        result = execute_adagrad_step_mpsgraph(H(device), w.data(), g.data(), s.data(), numWeights, sizes.data(),
                                               learningRate, epsilon, weightDecay);
        if (result != 0) return Errorf("AdaGrad MPSGraph step failed with error code: %d", result);
    }
    return "";
}

Error ExecuteAdaGradStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                                 const std::vector<Pointer> &gradientBuffers,
                                 const std::vector<Pointer> &squaredGradAvgBuffers, int numWeights,
                                 const std::vector<int> &bufferSizes, float learningRate, float epsilon,
                                 float weightDecay)
{
    return adagrad_common(false, device, weightBuffers, gradientBuffers, squaredGradAvgBuffers, numWeights,
                          bufferSizes, learningRate, epsilon, weightDecay, nullptr);
}

Error ExecuteAdaGradStepMPSGraphPooled(Pointer device, const std::vector<Pointer> &weightBuffers,
                                       const std::vector<Pointer> &gradientBuffers,
                                       const std::vector<Pointer> &squaredGradAvgBuffers, int numWeights,
                                       const std::vector<int> &bufferSizes, float learningRate,
                                       float epsilon, float weightDecay, Pointer commandPool)
{
    return adagrad_common(true, device, weightBuffers, gradientBuffers, squaredGradAvgBuffers, numWeights,
                          bufferSizes, learningRate, epsilon, weightDecay, commandPool);
}

static Error adadelta_common(bool pooled, Pointer device, const std::vector<Pointer> &weightBuffers,
                             const std::vector<Pointer> &gradientBuffers,
                             const std::vector<Pointer> &squaredGradAvgBuffers,
                             const std::vector<Pointer> &squaredUpdateAvgBuffers, int numWeights,
                             const std::vector<int> &bufferSizes, float rho, float epsilon, float weightDecay,
                             Pointer commandPool)
{
    if (device == nullptr) return Errorf("device cannot be nil");
    if ((int)weightBuffers.size() != numWeights || (int)gradientBuffers.size() != numWeights ||
        (int)squaredGradAvgBuffers.size() != numWeights || (int)squaredUpdateAvgBuffers.size() != numWeights ||
        (int)bufferSizes.size() != numWeights)
        return Errorf("buffer count mismatch: weights=%d, gradients=%d, squared_grad_avg=%d, "
                      "squared_update_avg=%d, sizes=%d, expected=%d",
                      (int)weightBuffers.size(), (int)gradientBuffers.size(), (int)squaredGradAvgBuffers.size(),
                      (int)squaredUpdateAvgBuffers.size(), (int)bufferSizes.size(), numWeights);
    if (numWeights <= 0) return Errorf("%s", kEmptyList);
    const size_t n = (size_t)numWeights;
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n), s = handles(squaredGradAvgBuffers, n),
         a = handles(squaredUpdateAvgBuffers, n);
    std::vector<int> sizes(bufferSizes);
    int result;
    if (pooled) {
        result = execute_adadelta_step_mpsgraph_pooled(H(device), w.data(), g.data(), s.data(), a.data(), numWeights,
                                                       sizes.data(), rho, epsilon, weightDecay, H(commandPool));
        if (result != 0) return Errorf("AdaDelta MPSGraph pooled step failed with error code: %d", result);
    } else {
        result = execute_adadelta_step_mpsgraph(H(device), w.data(), g.data(), s.data(), a.data(), numWeights,
                                                sizes.data(), rho, epsilon, weightDecay);
        if (result != 0) return Errorf("AdaDelta MPSGraph step failed with error code: %d", result);
    }
    return "";
}

Error ExecuteAdaDeltaStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                                  const std::vector<Pointer> &gradientBuffers,
                                  const std::vector<Pointer> &squaredGradAvgBuffers,
                                  const std::vector<Pointer> &squaredUpdateAvgBuffers, int numWeights,
                                  const std::vector<int> &bufferSizes, float rho, float epsilon,
                                  float weightDecay)
{
    return adadelta_common(false, device, weightBuffers, gradientBuffers, squaredGradAvgBuffers,
                           squaredUpdateAvgBuffers, numWeights, bufferSizes, rho, epsilon, weightDecay, nullptr);
}

Error ExecuteAdaDeltaStepMPSGraphPooled(Pointer device, const std::vector<Pointer> &weightBuffers,
                                        const std::vector<Pointer> &gradientBuffers,
                                        const std::vector<Pointer> &squaredGradAvgBuffers,
                                        const std::vector<Pointer> &squaredUpdateAvgBuffers, int numWeights,
                                        const std::vector<int> &bufferSizes, float rho, float epsilon,
                                        float weightDecay, Pointer commandPool)
{
    return adadelta_common(true, device, weightBuffers, gradientBuffers, squaredGradAvgBuffers,
                           squaredUpdateAvgBuffers, numWeights, bufferSizes, rho, epsilon, weightDecay,
                           commandPool);
}

Error ExecuteNadamStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                               const std::vector<Pointer> &gradientBuffers,
                               const std::vector<Pointer> &momentumBuffers,
                               const std::vector<Pointer> &varianceBuffers, const std::vector<int> &bufferSizes,
                               float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                               int stepCount)
{
    const size_t n = weightBuffers.size();
    if (n != gradientBuffers.size() || n != momentumBuffers.size() || n != varianceBuffers.size() ||
        n != bufferSizes.size())
        return Errorf("all buffer arrays must have the same length");
    if (n == 0) return Errorf("%s", kEmptyList);
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n), m = handles(momentumBuffers, n),
         v = handles(varianceBuffers, n);
    std::vector<int> sizes(bufferSizes);
    int result = execute_nadam_step_mpsgraph(H(device), w.data(), g.data(), m.data(), v.data(), (int)n,
                                             sizes.data(), learningRate, beta1, beta2, epsilon, weightDecay,
                                             stepCount);
    if (result != 0) return Errorf("Nadam MPSGraph step failed with error code: %d", result);
    return "";
}

std::pair<float, Error> ExecuteLBFGSStepMPSGraph(
    Pointer device, const std::vector<Pointer> &weightBuffers, const std::vector<Pointer> &gradientBuffers,
    const std::vector<Pointer> &oldGradientBuffers, const std::vector<Pointer> &searchDirBuffers,
    const std::vector<std::vector<Pointer>> &sVectors, const std::vector<std::vector<Pointer>> &yVectors,
    const std::vector<Pointer> &rhoBuffers, Pointer alphaBuffer, int numWeights,
    const std::vector<int> &bufferSizes, int historySize, int historyCount, int historyIndex,
    float initialStep, float c1, float c2, int maxLineSearch, float currentLoss, float prevLoss,
    Pointer commandPool, bool usePooling)
{
    // bridge.go:1963-1970
    const size_t n = numWeights > 0 ? (size_t)numWeights : 0;
    if (weightBuffers.size() != n || gradientBuffers.size() != n || oldGradientBuffers.size() != n ||
        searchDirBuffers.size() != n || bufferSizes.size() != n || numWeights < 0)
        return {0.0f, Errorf("buffer arrays must have length %d", numWeights)};
    if (n == 0) return {0.0f, Errorf("%s", kEmptyList)};
    // Go would panic indexing a short history slice; here it is an error.
    if (historySize <= 0 || sVectors.size() != (size_t)historySize || yVectors.size() != (size_t)historySize ||
        rhoBuffers.size() != (size_t)historySize)
        return {0.0f, Errorf("history arrays must have length %d", historySize)};
    auto w = handles(weightBuffers, n), g = handles(gradientBuffers, n), o = handles(oldGradientBuffers, n),
         d = handles(searchDirBuffers, n), rho = handles(rhoBuffers, (size_t)historySize);
    // flattened [hist0_weight0, hist0_weight1, ..., hist1_weight0, ...]  (bridge.go:1988-1999)
    std::vector<uintptr_t> sFlat((size_t)historySize * n), yFlat((size_t)historySize * n);
    for (int h = 0; h < historySize; h++) {
        if (sVectors[h].size() != n || yVectors[h].size() != n)
            return {0.0f, Errorf("history arrays must have %d buffers per entry", numWeights)};
        for (size_t i = 0; i < n; i++) {
            sFlat[(size_t)h * n + i] = reinterpret_cast<uintptr_t>(sVectors[h][i]);
            yFlat[(size_t)h * n + i] = reinterpret_cast<uintptr_t>(yVectors[h][i]);
        }
    }
    std::vector<int> sizes(bufferSizes);
    float stepSize = 0.0f;
    int result;
    if (usePooling && commandPool != nullptr)
        result = execute_lbfgs_step_mpsgraph_pooled(
            H(device), w.data(), g.data(), o.data(), d.data(), sFlat.data(), yFlat.data(), rho.data(),
            H(alphaBuffer), numWeights, sizes.data(), historySize, historyCount, historyIndex, initialStep, c1,
            c2, maxLineSearch, currentLoss, prevLoss, H(commandPool), &stepSize);
    else
        result = execute_lbfgs_step_mpsgraph(
            H(device), w.data(), g.data(), o.data(), d.data(), sFlat.data(), yFlat.data(), rho.data(),
            H(alphaBuffer), numWeights, sizes.data(), historySize, historyCount, historyIndex, initialStep, c1,
            c2, maxLineSearch, currentLoss, prevLoss, &stepSize);
    if (result != 0) return {0.0f, Errorf("L-BFGS MPSGraph step failed with error code: %d", result)};
    return {stepSize, ""};
}

Error ExecuteAdamAMPStep(Pointer device, const std::vector<Pointer> &weightBuffers,
                         const std::vector<Pointer> &gradient16Buffers,
                         const std::vector<Pointer> &momentumBuffers,
                         const std::vector<Pointer> &varianceBuffers,
                         const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                         float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                         int stepCount, Pointer ampState, bool *skipped, float *scale, int *growthTracker)
{
    const size_t n = weightBuffers.size();
    if (n != gradient16Buffers.size() || n != momentumBuffers.size() || n != varianceBuffers.size() ||
        n != bufferSizes.size() || (!weight16Buffers.empty() && weight16Buffers.size() != n))
        return Errorf("all buffer arrays must have the same length");
    if (n == 0) return Errorf("%s", kEmptyList);
    auto w = handles(weightBuffers, n), g = handles(gradient16Buffers, n), m = handles(momentumBuffers, n),
         v = handles(varianceBuffers, n), h = handles(weight16Buffers, n);
    std::vector<int> sizes(bufferSizes);
    int sk = 0;
    int result = execute_adam_amp_step(H(device), w.data(), g.data(), m.data(), v.data(),
                                       weight16Buffers.empty() ? nullptr : h.data(), (int)n, sizes.data(),
                                       learningRate, beta1, beta2, epsilon, weightDecay, stepCount, H(ampState),
                                       &sk, scale, growthTracker);
    if (result != 0) return Errorf("Adam mixed-precision step failed with error code: %d", result);
    if (skipped) *skipped = sk != 0;
    return "";
}

Error ExecuteAdamAMPStepAsync(Pointer device, const std::vector<Pointer> &weightBuffers,
                              const std::vector<Pointer> &gradient16Buffers,
                              const std::vector<Pointer> &momentumBuffers,
                              const std::vector<Pointer> &varianceBuffers,
                              const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                              float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                              Pointer ampState)
{
    const size_t n = weightBuffers.size();
    if (n != gradient16Buffers.size() || n != momentumBuffers.size() || n != varianceBuffers.size() ||
        n != bufferSizes.size() || (!weight16Buffers.empty() && weight16Buffers.size() != n))
        return Errorf("all buffer arrays must have the same length");
    if (n == 0) return Errorf("%s", kEmptyList);
    auto w = handles(weightBuffers, n), g = handles(gradient16Buffers, n), m = handles(momentumBuffers, n),
         v = handles(varianceBuffers, n), h = handles(weight16Buffers, n);
    std::vector<int> sizes(bufferSizes);
    int result = execute_adam_amp_step_async(H(device), w.data(), g.data(), m.data(), v.data(),
                                             weight16Buffers.empty() ? nullptr : h.data(), (int)n, sizes.data(),
                                             learningRate, beta1, beta2, epsilon, weightDecay, H(ampState));
    if (result != 0) return Errorf("Adam mixed-precision step failed with error code: %d", result);
    return "";
}

static Error checkFusedLists(const std::vector<Pointer> setA[3], const std::vector<Pointer> setB[3],
                             const std::vector<Pointer> &gradient16Buffers,
                             const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes)
{
    const size_t n = setA[0].size();
    for (int k = 0; k < 3; k++)
        if (setA[k].size() != n || setB[k].size() != n) return Errorf("all buffer arrays must have the same length");
    if (n != gradient16Buffers.size() || n != bufferSizes.size() ||
        (!weight16Buffers.empty() && weight16Buffers.size() != n))
        return Errorf("all buffer arrays must have the same length");
    if (n == 0) return Errorf("%s", kEmptyList);
    return "";
}

Error ExecuteAdamAMPStepFused(Pointer device, const std::vector<Pointer> setA[3], const std::vector<Pointer> setB[3],
                              const std::vector<Pointer> &gradient16Buffers,
                              const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                              float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                              int stepCount, Pointer ampState, bool *skipped, float *scale, int *growthTracker,
                              int *currentSet)
{
    if (Error e = checkFusedLists(setA, setB, gradient16Buffers, weight16Buffers, bufferSizes); !e.empty()) return e;
    const size_t n = setA[0].size();
    auto wa = handles(setA[0], n), ma = handles(setA[1], n), va = handles(setA[2], n);
    auto wb = handles(setB[0], n), mb = handles(setB[1], n), vb = handles(setB[2], n);
    auto g = handles(gradient16Buffers, n), h = handles(weight16Buffers, n);
    std::vector<int> sizes(bufferSizes);
    int sk = 0;
    int result = execute_adam_amp_step_fused(H(device), wa.data(), ma.data(), va.data(), wb.data(), mb.data(), vb.data(),
                                             g.data(), weight16Buffers.empty() ? nullptr : h.data(), (int)n,
                                             sizes.data(), learningRate, beta1, beta2, epsilon, weightDecay, stepCount,
                                             H(ampState), &sk, scale, growthTracker, currentSet);
    if (result != 0) return Errorf("Adam mixed-precision step failed with error code: %d", result);
    if (skipped) *skipped = sk != 0;
    return "";
}

Error ExecuteAdamAMPStepFusedAsync(Pointer device, const std::vector<Pointer> setA[3],
                                   const std::vector<Pointer> setB[3], const std::vector<Pointer> &gradient16Buffers,
                                   const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                                   float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                                   Pointer ampState)
{
    if (Error e = checkFusedLists(setA, setB, gradient16Buffers, weight16Buffers, bufferSizes); !e.empty()) return e;
    const size_t n = setA[0].size();
    auto wa = handles(setA[0], n), ma = handles(setA[1], n), va = handles(setA[2], n);
    auto wb = handles(setB[0], n), mb = handles(setB[1], n), vb = handles(setB[2], n);
    auto g = handles(gradient16Buffers, n), h = handles(weight16Buffers, n);
    std::vector<int> sizes(bufferSizes);
    int result = execute_adam_amp_step_fused_async(H(device), wa.data(), ma.data(), va.data(), wb.data(), mb.data(),
                                                   vb.data(), g.data(), weight16Buffers.empty() ? nullptr : h.data(),
                                                   (int)n, sizes.data(), learningRate, beta1, beta2, epsilon,
                                                   weightDecay, H(ampState));
    if (result != 0) return Errorf("Adam mixed-precision step failed with error code: %d", result);
    return "";
}

}  // namespace cgo_bridge
}  // namespace gometal
