// Host-side mirror of the Go package `cgo_bridge` (cgo_bridge/bridge.go), limited
// to the wrappers the `optimizer` and `memory` packages call.  Same function
// names, argument order, validation and error strings as the Go wrappers; an
// empty Error plays the role of Go's nil error.  Each wrapper marshals its
// arguments and calls the C ABI in include/gometal_hip.h, exactly where the Go
// wrapper calls C.<function>.
#pragma once

#include <cstdint>
#include <string>
#include <utility>
#include <vector>

namespace gometal {

using Error = std::string;                 // "" == nil
using Pointer = void *;                    // Go's unsafe.Pointer
Error Errorf(const char *fmt, ...) __attribute__((format(printf, 1, 2)));

namespace cgo_bridge {

// cgo_bridge/bridge.go:623-629
enum DeviceType : int { CPU = 0, GPU = 1, PersistentGPU = 2 };

std::pair<Pointer, Error> CreateMetalDevice();                                      // bridge.go:632
void DestroyMetalDevice(Pointer device);                                            // bridge.go:641
std::pair<Pointer, Error> CreateCommandQueue(Pointer device);                       // bridge.go:1676
void ReleaseCommandQueue(Pointer queue);                                            // bridge.go:1690
std::pair<Pointer, Error> AllocateMetalBuffer(Pointer device, int size, DeviceType deviceType);  // bridge.go:729
// allocate_metal_buffer with the buffer's start placed at `phase` bytes modulo 2 MiB (no counterpart in the reference)
std::pair<Pointer, Error> AllocateMetalBufferPhased(Pointer device, int size, DeviceType deviceType, int phase);
void DeallocateMetalBuffer(Pointer buffer);                                         // bridge.go:744
Error ZeroMetalBuffer(Pointer device, Pointer buffer, int size);                    // bridge.go:1039
Error CopyFloat32ArrayToMetalBuffer(Pointer buffer, const std::vector<float> &data);  // bridge.go:1069
std::pair<std::vector<float>, Error> CopyMetalBufferToFloat32Array(Pointer buffer, int numElements);  // bridge.go:1107
Error ConvertTensorType(Pointer srcBuffer, Pointer dstBuffer, const std::vector<int> &shape, int srcType,
                        int dstType, Pointer device);                               // bridge.go:1151
Error CopyTensorBufferSync(Pointer srcBuffer, Pointer dstBuffer, int size);         // bridge.go:2358

// bridge.go:892
Error ExecuteSGDStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                             const std::vector<Pointer> &gradientBuffers,
                             const std::vector<Pointer> &momentumBuffers, const std::vector<int> &bufferSizes,
                             float learningRate, float momentum, float weightDecay, bool nesterov,
                             int stepCount);
// bridge.go:975
Error ExecuteAdamStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                              const std::vector<Pointer> &gradientBuffers,
                              const std::vector<Pointer> &momentumBuffers,
                              const std::vector<Pointer> &varianceBuffers, const std::vector<int> &bufferSizes,
                              float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                              int stepCount);
// bridge.go:1861
Error ExecuteRMSPropStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                                 const std::vector<Pointer> &gradientBuffers,
                                 const std::vector<Pointer> &squaredGradAvgBuffers,
                                 const std::vector<Pointer> &momentumBuffers,
                                 const std::vector<Pointer> &gradientAvgBuffers,
                                 const std::vector<int> &bufferSizes, float learningRate, float alpha,
                                 float epsilon, float weightDecay, float momentum, bool centered,
                                 int stepCount);
// bridge.go:2067, 2120
Error ExecuteAdaGradStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                                 const std::vector<Pointer> &gradientBuffers,
                                 const std::vector<Pointer> &squaredGradAvgBuffers, int numWeights,
                                 const std::vector<int> &bufferSizes, float learningRate, float epsilon,
                                 float weightDecay);
Error ExecuteAdaGradStepMPSGraphPooled(Pointer device, const std::vector<Pointer> &weightBuffers,
                                       const std::vector<Pointer> &gradientBuffers,
                                       const std::vector<Pointer> &squaredGradAvgBuffers, int numWeights,
                                       const std::vector<int> &bufferSizes, float learningRate,
                                       float epsilon, float weightDecay, Pointer commandPool);
// bridge.go:2175, 2233
Error ExecuteAdaDeltaStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                                  const std::vector<Pointer> &gradientBuffers,
                                  const std::vector<Pointer> &squaredGradAvgBuffers,
                                  const std::vector<Pointer> &squaredUpdateAvgBuffers, int numWeights,
                                  const std::vector<int> &bufferSizes, float rho, float epsilon,
                                  float weightDecay);
Error ExecuteAdaDeltaStepMPSGraphPooled(Pointer device, const std::vector<Pointer> &weightBuffers,
                                        const std::vector<Pointer> &gradientBuffers,
                                        const std::vector<Pointer> &squaredGradAvgBuffers,
                                        const std::vector<Pointer> &squaredUpdateAvgBuffers, int numWeights,
                                        const std::vector<int> &bufferSizes, float rho, float epsilon,
                                        float weightDecay, Pointer commandPool);
// bridge.go:2294
Error ExecuteNadamStepMPSGraph(Pointer device, const std::vector<Pointer> &weightBuffers,
                               const std::vector<Pointer> &gradientBuffers,
                               const std::vector<Pointer> &momentumBuffers,
                               const std::vector<Pointer> &varianceBuffers, const std::vector<int> &bufferSizes,
                               float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                               int stepCount);

// bridge.go:1939.  sVectors / yVectors are [historySize][numWeights]; returns the step size.
std::pair<float, Error> ExecuteLBFGSStepMPSGraph(
    Pointer device, const std::vector<Pointer> &weightBuffers, const std::vector<Pointer> &gradientBuffers,
    const std::vector<Pointer> &oldGradientBuffers, const std::vector<Pointer> &searchDirBuffers,
    const std::vector<std::vector<Pointer>> &sVectors, const std::vector<std::vector<Pointer>> &yVectors,
    const std::vector<Pointer> &rhoBuffers, Pointer alphaBuffer, int numWeights,
    const std::vector<int> &bufferSizes, int historySize, int historyCount, int historyIndex,
    float initialStep, float c1, float c2, int maxLineSearch, float currentLoss, float prevLoss,
    Pointer commandPool, bool usePooling);

// Addition (no Go counterpart): the mixed-precision Adam step.  weight16Buffers may be
// empty.  On success *skipped tells whether the step was dropped for an inf / NaN gradient.
Error ExecuteAdamAMPStep(Pointer device, const std::vector<Pointer> &weightBuffers,
                         const std::vector<Pointer> &gradient16Buffers,
                         const std::vector<Pointer> &momentumBuffers,
                         const std::vector<Pointer> &varianceBuffers,
                         const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                         float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                         int stepCount, Pointer ampState, bool *skipped, float *scale, int *growthTracker);

// The same step without the read-back (execute_adam_amp_step_async).
Error ExecuteAdamAMPStepAsync(Pointer device, const std::vector<Pointer> &weightBuffers,
                              const std::vector<Pointer> &gradient16Buffers,
                              const std::vector<Pointer> &momentumBuffers,
                              const std::vector<Pointer> &varianceBuffers,
                              const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                              float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                              Pointer ampState);

// The one-pass step over ping-pong state (execute_adam_amp_step_fused): set A / set B of weights,
// momentum and variance; *currentSet (may be null) receives which set is current after the step.
Error ExecuteAdamAMPStepFused(Pointer device, const std::vector<Pointer> setA[3], const std::vector<Pointer> setB[3],
                              const std::vector<Pointer> &gradient16Buffers,
                              const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                              float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                              int stepCount, Pointer ampState, bool *skipped, float *scale, int *growthTracker,
                              int *currentSet);
Error ExecuteAdamAMPStepFusedAsync(Pointer device, const std::vector<Pointer> setA[3],
                                   const std::vector<Pointer> setB[3], const std::vector<Pointer> &gradient16Buffers,
                                   const std::vector<Pointer> &weight16Buffers, const std::vector<int> &bufferSizes,
                                   float learningRate, float beta1, float beta2, float epsilon, float weightDecay,
                                   Pointer ampState);

}  // namespace cgo_bridge
}  // namespace gometal
