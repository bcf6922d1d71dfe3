// Host-side mirror of the Go package `optimizer` (optimizer/*.go): the state objects that
// own hyper-parameters, step counters and device-resident state buffers, and drive the C ABI.
// Type names, method names, argument meaning, validation order and error strings follow the
// Go sources; an empty Error is Go's nil.  L-BFGS lives in lbfgs.hpp.
#pragma once

#include "bridge.hpp"
#include "memory_manager.hpp"

#include <cstdint>
#include <map>
#include <memory>
#include <string>
#include <variant>
#include <vector>

namespace gometal {

namespace checkpoints {
// checkpoints/checkpoint.go:81-86
struct OptimizerTensor {
    std::string Name;
    std::vector<int> Shape;
    std::vector<float> Data;
    std::string StateType;
};
}  // namespace checkpoints

namespace optimizer {

// A value of Go's map[string]interface{}.  GetState stores float32 / uint64 / bool (as the Go
// code does); after a JSON round trip every number is a float64, which is the only numeric
// type LoadState accepts (optimizer/adam.go:397-414).
using ParamValue = std::variant<double, float, bool, uint64_t, std::string>;

// optimizer/interface.go:47-51
struct OptimizerState {
    std::string Type;
    std::map<std::string, ParamValue> Parameters;
    std::vector<checkpoints::OptimizerTensor> StateData;

    // encoding/json shape: {"type":..,"parameters":{..},"state_data":[{"name","shape","data","state_type"}]}
    // Fails on a non-finite value, as json.Marshal does ("json: unsupported value: NaN").
    std::pair<std::string, Error> ToJSON() const;
    static std::pair<OptimizerState, Error> FromJSON(const std::string &text);

    // The reference stores this object under the key "optimizer_state" of its JSON checkpoint
    // (checkpoints/checkpoint.go:38-52, written by saveJSON :133-157).  FromCheckpointJSON pulls
    // it out of such a file's text (error if the checkpoint has none); ToCheckpointJSON writes a
    // checkpoint document that carries only the optimizer state and the metadata block
    // (framework "go-metal", version "1.0.0"), which the reference's loadJSON decodes.
    static std::pair<OptimizerState, Error> FromCheckpointJSON(const std::string &text);
    std::pair<std::string, Error> ToCheckpointJSON() const;
};

// optimizer/interface.go:13-43
class Optimizer {
public:
    virtual ~Optimizer() = default;
    virtual Error Step(const std::vector<Pointer> &gradientBuffers) = 0;
    virtual std::pair<std::unique_ptr<OptimizerState>, Error> GetState() = 0;
    virtual Error LoadState(const OptimizerState *state) = 0;
    virtual uint64_t GetStepCount() = 0;
    virtual void UpdateLearningRate(float lr) = 0;
    virtual Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) = 0;
    virtual void SetCommandPool(Pointer commandPool) = 0;
    virtual void Cleanup() = 0;
};

// ---- helpers: optimizer/interface.go:56-84, state_helpers.go:14-74, adam.go:142-148, 237-251 ----
int extractBufferIndex(const std::string &name);
Error validateStateType(const std::string &optimizerType, const OptimizerState *state);
int calculateTensorSize(const std::vector<int> &shape);
std::pair<std::unique_ptr<checkpoints::OptimizerTensor>, Error> extractBufferState(
    Pointer buffer, int bufferSize, const std::string &name, const std::string &stateType);
Error restoreBufferState(Pointer buffer, const std::vector<float> &data, int bufferSize, const std::string &name);
float extractFloat32Param(const std::map<std::string, ParamValue> &params, const std::string &key, float defaultValue);
bool extractBoolParam(const std::map<std::string, ParamValue> &params, const std::string &key, bool defaultValue);
uint64_t extractUint64Param(const std::map<std::string, ParamValue> &params, const std::string &key,
                            uint64_t defaultValue);

// optimizer/adam.go:236-251: x^y by repeated multiplication for small non-negative integer y
// (a helper the Go package keeps and tests but does not call; bias corrections are formed
// natively with powf).
float pow(float x, float y);

using Shapes = std::vector<std::vector<int>>;

// ------------------------------------------------------------------ SGD (optimizer/sgd.go) ----
struct SGDConfig {
    float LearningRate, Momentum, WeightDecay;
    bool Nesterov;
};
SGDConfig DefaultSGDConfig();

class SGDOptimizerState : public Optimizer {
public:
    float LearningRate = 0, Momentum = 0, WeightDecay = 0;
    bool Nesterov = false;
    std::vector<Pointer> MomentumBuffers, WeightBuffers;
    uint64_t StepCount = 0;

    Error Step(const std::vector<Pointer> &gradientBuffers) override;
    std::pair<std::unique_ptr<OptimizerState>, Error> GetState() override;
    Error LoadState(const OptimizerState *state) override;
    uint64_t GetStepCount() override { return StepCount; }
    uint64_t GetStep() { return StepCount; }
    void UpdateLearningRate(float lr) override { LearningRate = lr; }
    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) override;
    void SetCommandPool(Pointer commandPool) override;
    void Cleanup() override;

    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
};
std::pair<std::unique_ptr<SGDOptimizerState>, Error> NewSGDOptimizer(const SGDConfig &config,
                                                                     const Shapes &weightShapes,
                                                                     memory::MemoryManager *memoryManager,
                                                                     Pointer device);

// ---------------------------------------------------------------- Adam (optimizer/adam.go) ----
struct AdamConfig {
    float LearningRate, Beta1, Beta2, Epsilon, WeightDecay;
};
AdamConfig DefaultAdamConfig();

struct AdamStats {
    uint64_t StepCount;
    float LearningRate, Beta1, Beta2, Epsilon, WeightDecay;
    int NumParameters, TotalBufferSize;
};

class AdamOptimizerState : public Optimizer {
public:
    float LearningRate = 0, Beta1 = 0, Beta2 = 0, Epsilon = 0, WeightDecay = 0;
    std::vector<Pointer> MomentumBuffers, VarianceBuffers, WeightBuffers;
    uint64_t StepCount = 0;

    ~AdamOptimizerState() override;
    Error Step(const std::vector<Pointer> &gradientBuffers) override;
    std::pair<std::unique_ptr<OptimizerState>, Error> GetState() override;
    Error LoadState(const OptimizerState *state) override;
    uint64_t GetStepCount() override;                         // additive: the Go type only has GetStep
    uint64_t GetStep() { return GetStepCount(); }
    AdamStats GetStats();
    void UpdateLearningRate(float lr) override { LearningRate = lr; }
    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) override;
    void SetCommandPool(Pointer commandPool) override;
    void Cleanup() override;

    // ---- mixed precision (additive; constants from training/model_trainer.go:258-270) ----
    // Creates the device-resident loss-scale state.  Call before StepAMP.  A further call replaces the state
    // (steps in flight finish first; with ping-pong state on, the new state is told which set is current).
    Error EnableMixedPrecision(float initialScale = 65536.0f, float growthFactor = 2.0f,
                               float backoffFactor = 0.5f, int growthInterval = 2000);
    // One step on fp16 gradients of the scaled loss.  Returns skipped = true (and leaves
    // StepCount, weights and moments untouched) when a gradient holds inf / NaN.
    // weight16Buffers may be empty (no fp16 weight copy).  Updates in place unless EnablePingPong
    // was called: the caller's own fp32 weight buffers hold the current weights after every step.
    // Returns when the outcome is known; the update completes on the library's stream like an fp32 Step.
    std::pair<bool, Error> StepAMP(const std::vector<Pointer> &gradient16Buffers,
                                   const std::vector<Pointer> &weight16Buffers);
    // The same step without waiting for it: no result is returned, and up to 7 steps run ahead
    // of the host.  StepCount, LossScale and GrowthTracker are brought up to date by SyncAMP
    // (GetStepCount, GetState, LoadState, Step and StepAMP call it when steps are pending).
    Error StepAMPAsync(const std::vector<Pointer> &gradient16Buffers,
                       const std::vector<Pointer> &weight16Buffers);
    // Waits for the pending steps; *skippedSteps (may be null) receives how many steps have
    // been dropped since EnableMixedPrecision.
    Error SyncAMP(uint64_t *skippedSteps = nullptr);
    // Switches StepAMP / StepAMPAsync to the one-pass step over ping-pong state: a second set of weight,
    // momentum and variance buffers is taken from the memory manager, and every applied step makes the set it
    // wrote the current one.  Call after SetWeightBuffers and EnableMixedPrecision.  From then on the weights
    // live in CurrentWeightBuffers() (the caller's own buffers after an even number of applied steps, the
    // shadow set after an odd number); GetState / LoadState read and write the current moments; the fp16
    // weight copy passed to StepAMP must start out as half of the weights (ConvertTo(Float16)).
    Error EnablePingPong();
    bool PingPong() const { return pingPong; }
    // The buffers holding the current fp32 weights / moments (waits for pending asynchronous steps).
    const std::vector<Pointer> &CurrentWeightBuffers();
    const std::vector<Pointer> &CurrentMomentumBuffers();
    const std::vector<Pointer> &CurrentVarianceBuffers();
    float LossScale = 0.0f;     // as of the last StepAMP / SyncAMP / EnableMixedPrecision / LoadState
    int GrowthTracker = 0;

    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
    Pointer ampState = nullptr;
    int ampPending = 0;            // asynchronous steps issued since the last SyncAMP
    bool ampCountDirty = false;    // StepCount changed on the host since the device last saw it
    bool pingPong = false;
    int currentSet = 0;            // 0: WeightBuffers / MomentumBuffers / VarianceBuffers are current, 1: the shadows
    std::vector<Pointer> ShadowWeightBuffers, ShadowMomentumBuffers, ShadowVarianceBuffers;

private:
    Error refreshCurrentSet();     // after asynchronous steps: asks the device which set is current
};
std::pair<std::unique_ptr<AdamOptimizerState>, Error> NewAdamOptimizer(const AdamConfig &config,
                                                                       const Shapes &weightShapes,
                                                                       memory::MemoryManager *memoryManager,
                                                                       Pointer device);

// ---------------------------------------------------------- RMSProp (optimizer/rmsprop.go) ----
struct RMSPropConfig {
    float LearningRate, Alpha, Epsilon, WeightDecay, Momentum;
    bool Centered;
};
RMSPropConfig DefaultRMSPropConfig();

struct RMSPropStats {
    uint64_t StepCount;
    float LearningRate, Alpha, Epsilon, WeightDecay, Momentum;
    bool Centered;
    int NumParameters, TotalBufferSize;
};

class RMSPropOptimizerState : public Optimizer {
public:
    float LearningRate = 0, Alpha = 0, Epsilon = 0, WeightDecay = 0, Momentum = 0;
    bool Centered = false;
    std::vector<Pointer> SquaredGradAvgBuffers, MomentumBuffers, GradientAvgBuffers, WeightBuffers;
    uint64_t StepCount = 0;

    Error Step(const std::vector<Pointer> &gradientBuffers) override;
    std::pair<std::unique_ptr<OptimizerState>, Error> GetState() override;
    Error LoadState(const OptimizerState *state) override;
    uint64_t GetStepCount() override { return StepCount; }   // additive: the Go type only has GetStep
    uint64_t GetStep() { return StepCount; }
    RMSPropStats GetStats();
    void UpdateLearningRate(float lr) override { LearningRate = lr; }
    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) override;
    void SetCommandPool(Pointer commandPool) override;
    void Cleanup() override;

    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
};
std::pair<std::unique_ptr<RMSPropOptimizerState>, Error> NewRMSPropOptimizer(const RMSPropConfig &config,
                                                                             const Shapes &weightShapes,
                                                                             memory::MemoryManager *memoryManager,
                                                                             Pointer device);

// ---------------------------------------------------------- AdaGrad (optimizer/adagrad.go) ----
struct AdaGradConfig {
    float LearningRate, Epsilon, WeightDecay;
};
AdaGradConfig DefaultAdaGradConfig();

class AdaGradOptimizerState : public Optimizer {
public:
    std::vector<Pointer> WeightBuffers;

    Error Step(const std::vector<Pointer> &gradientBuffers) override;
    std::pair<std::unique_ptr<OptimizerState>, Error> GetState() override;
    Error LoadState(const OptimizerState *state) override;
    uint64_t GetStepCount() override { return currentStep; }
    uint64_t GetStep() { return currentStep; }
    std::map<std::string, ParamValue> GetStats();
    void UpdateLearningRate(float lr) override { config.LearningRate = lr; }
    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) override;
    void SetCommandPool(Pointer pool) override;
    void Cleanup() override;

    AdaGradConfig config{};
    std::vector<Pointer> squaredGradAvgBuffers;
    uint64_t currentStep = 0;
    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
    bool logProgress = true;     // the Go Step prints a line every 10 steps (adagrad.go:165-167)

private:
    void cleanup();
};
std::pair<std::unique_ptr<AdaGradOptimizerState>, Error> NewAdaGradOptimizer(const AdaGradConfig &config,
                                                                             const Shapes &weightShapes,
                                                                             memory::MemoryManager *memoryManager,
                                                                             Pointer device);

// -------------------------------------------------------- AdaDelta (optimizer/adadelta.go) ----
struct AdaDeltaConfig {
    float Rho, Epsilon, WeightDecay;
};
AdaDeltaConfig DefaultAdaDeltaConfig();

class AdaDeltaOptimizerState : public Optimizer {
public:
    std::vector<Pointer> WeightBuffers;

    Error Step(const std::vector<Pointer> &gradientBuffers) override;
    std::pair<std::unique_ptr<OptimizerState>, Error> GetState() override;
    Error LoadState(const OptimizerState *state) override;
    uint64_t GetStepCount() override { return currentStep; }
    uint64_t GetStep() { return currentStep; }
    std::map<std::string, ParamValue> GetStats();
    void UpdateLearningRate(float) override {}   // AdaDelta has no learning rate (adadelta.go:222-225)
    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) override;
    void SetCommandPool(Pointer pool) override;
    void Cleanup() override;

    AdaDeltaConfig config{};
    std::vector<Pointer> squaredGradAvgBuffers, squaredUpdateAvgBuffers;
    uint64_t currentStep = 0;
    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
    bool logProgress = true;     // adadelta.go:188-190

private:
    void cleanup();
};
std::pair<std::unique_ptr<AdaDeltaOptimizerState>, Error> NewAdaDeltaOptimizer(const AdaDeltaConfig &config,
                                                                               const Shapes &weightShapes,
                                                                               memory::MemoryManager *memoryManager,
                                                                               Pointer device);

// -------------------------------------------------------------- Nadam (optimizer/nadam.go) ----
struct NadamConfig {
    float LearningRate, Beta1, Beta2, Epsilon, WeightDecay;
};
NadamConfig DefaultNadamConfig();

class NadamOptimizerState : public Optimizer {
public:
    std::vector<Pointer> WeightBuffers;

    Error Step(const std::vector<Pointer> &gradientBuffers) override;
    std::pair<std::unique_ptr<OptimizerState>, Error> GetState() override;
    Error LoadState(const OptimizerState *state) override;
    uint64_t GetStepCount() override { return currentStep; }
    uint64_t GetStep() { return currentStep; }
    std::map<std::string, ParamValue> GetStats();
    void UpdateLearningRate(float lr) override { config.LearningRate = lr; }
    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers) override;
    void SetCommandPool(Pointer commandPool) override;
    void Cleanup() override;

    NadamConfig config{};
    std::vector<Pointer> momentumBuffers, varianceBuffers;
    uint64_t currentStep = 0;
    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
};
std::pair<std::unique_ptr<NadamOptimizerState>, Error> NewNadamOptimizer(const NadamConfig &config,
                                                                         const Shapes &weightShapes,
                                                                         memory::MemoryManager *memoryManager,
                                                                         Pointer device);

}  // namespace optimizer
}  // namespace gometal
