// Host-side mirror of the Go package `optimizer` (see optimizer.hpp).
#include "optimizer.hpp"

#include "../../include/gometal_hip.h"

#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace gometal {
namespace optimizer {

using checkpoints::OptimizerTensor;
using StateResult = std::pair<std::unique_ptr<OptimizerState>, Error>;

// ------------------------------------------------------------------------ helpers ----

// optimizer/interface.go:56-76: the decimal integer after the last underscore
// (fmt.Sscanf "%d": optional sign, at least one digit, trailing text ignored).
int extractBufferIndex(const std::string &name)
{
    const size_t us = name.rfind('_');
    if (us == std::string::npos) return -1;
    const char *p = name.c_str() + us + 1;
    const char *q = p;
    if (*q == '+' || *q == '-') q++;
    if (!std::isdigit((unsigned char)*q)) return -1;
    return (int)std::strtol(p, nullptr, 10);
}

// optimizer/interface.go:79-84
Error validateStateType(const std::string &optimizerType, const OptimizerState *state)
{
    if (state->Type != optimizerType)
        return Errorf("state type mismatch: expected %s, got %s", optimizerType.c_str(), state->Type.c_str());
    return "";
}

// optimizer/adam.go:237-251
float pow(float x, float y)
{
    if (y == 0) return 1.0f;
    if (y == 1) return x;
    float result = 1.0f;
    for (int i = 0; i < (int)y; i++) result *= x;
    return result;
}

// optimizer/adam.go:142-148
int calculateTensorSize(const std::vector<int> &shape)
{
    int size = 1;
    for (int dim : shape) size *= dim;
    return size;
}

// optimizer/state_helpers.go:14-32
std::pair<std::unique_ptr<OptimizerTensor>, Error> extractBufferState(Pointer buffer, int bufferSize,
                                                                      const std::string &name,
                                                                      const std::string &stateType)
{
    if (buffer == nullptr) return {nullptr, ""};
    const int numElements = bufferSize / 4;
    auto [data, err] = cgo_bridge::CopyMetalBufferToFloat32Array(buffer, numElements);
    if (!err.empty()) return {nullptr, Errorf("failed to read %s: %s", name.c_str(), err.c_str())};
    auto t = std::make_unique<OptimizerTensor>();
    t->Name = name;
    t->Shape = {(int)data.size()};
    t->Data = std::move(data);
    t->StateType = stateType;
    return {std::move(t), ""};
}

// optimizer/state_helpers.go:35-50
Error restoreBufferState(Pointer buffer, const std::vector<float> &data, int bufferSize, const std::string &name)
{
    if (buffer == nullptr) return Errorf("%s buffer is nil", name.c_str());
    const int expectedElements = bufferSize / 4;
    if ((int)data.size() != expectedElements)
        return Errorf("data size mismatch for %s: expected %d elements, got %d", name.c_str(), expectedElements,
                      (int)data.size());
    Error err = cgo_bridge::CopyFloat32ArrayToMetalBuffer(buffer, data);
    if (!err.empty()) return Errorf("failed to restore %s: %s", name.c_str(), err.c_str());
    return "";
}

static const double *asFloat64(const std::map<std::string, ParamValue> &params, const std::string &key)
{
    auto it = params.find(key);
    if (it == params.end()) return nullptr;
    return std::get_if<double>(&it->second);
}

// optimizer/state_helpers.go:53-74: only a float64 (what encoding/json produces) is accepted
float extractFloat32Param(const std::map<std::string, ParamValue> &params, const std::string &key, float defaultValue)
{
    if (const double *v = asFloat64(params, key)) return (float)*v;
    return defaultValue;
}

bool extractBoolParam(const std::map<std::string, ParamValue> &params, const std::string &key, bool defaultValue)
{
    auto it = params.find(key);
    if (it != params.end())
        if (const bool *b = std::get_if<bool>(&it->second)) return *b;
    return defaultValue;
}

// Go's uint64(float64) of a value outside the target range is implementation-defined; in C++ it
// is undefined behaviour.  Out-of-range counts saturate and NaN counts as zero.
static uint64_t toUint64(double v)
{
    if (!(v >= 0.0)) return 0;                                   // negative or NaN
    if (v >= 18446744073709551616.0) return UINT64_MAX;
    return (uint64_t)v;
}

static int toInt(double v)
{
    if (std::isnan(v)) return 0;
    if (v <= -2147483648.0) return INT32_MIN;
    if (v >= 2147483647.0) return INT32_MAX;
    return (int)v;
}

uint64_t extractUint64Param(const std::map<std::string, ParamValue> &params, const std::string &key,
                            uint64_t defaultValue)
{
    if (const double *v = asFloat64(params, key)) return toUint64(*v);
    return defaultValue;
}

// step_count as AdaGrad / AdaDelta / Nadam read it: float64, else uint64 (adagrad.go:258-262)
static void loadStepCountLenient(const std::map<std::string, ParamValue> &params, uint64_t &step)
{
    auto it = params.find("step_count");
    if (it == params.end()) return;
    if (const double *d = std::get_if<double>(&it->second)) step = toUint64(*d);
    else if (const uint64_t *u = std::get_if<uint64_t>(&it->second)) step = *u;
}

static void setFloat(const std::map<std::string, ParamValue> &params, const char *key, float &field)
{
    if (const double *v = asFloat64(params, key)) field = (float)*v;
}

static Error checkCommon(memory::MemoryManager *memoryManager, Pointer device, const Shapes &weightShapes)
{
    if (memoryManager == nullptr) return Errorf("memory manager cannot be nil");
    if (device == nullptr) return Errorf("device cannot be nil");
    if (weightShapes.empty()) return Errorf("no weight shapes provided");
    return "";
}

static Error setWeights(std::vector<Pointer> &dst, const std::vector<Pointer> &src)
{
    if (src.size() != dst.size())
        return Errorf("expected %d weight buffers, got %d", (int)dst.size(), (int)src.size());
    dst = src;
    return "";
}

static Error checkGradients(const std::vector<Pointer> &gradientBuffers, const std::vector<Pointer> &weightBuffers)
{
    if (gradientBuffers.size() != weightBuffers.size())
        return Errorf("gradient buffers length (%d) doesn't match weight buffers length (%d)",
                      (int)gradientBuffers.size(), (int)weightBuffers.size());
    return "";
}

static void releaseAll(memory::MemoryManager *mm, std::vector<Pointer> &buffers)
{
    for (Pointer &b : buffers) {
        if (b != nullptr) {
            if (mm) mm->ReleaseBuffer(b);
            b = nullptr;
        }
    }
}

// Reads every non-nil buffer of one state kind into tensors named <prefix>_<i>.
static Error readBuffers(const std::vector<Pointer> &buffers, const std::vector<int> &sizes, const char *prefix,
                         const char *stateType, const char *what, std::vector<OptimizerTensor> &out)
{
    for (size_t i = 0; i < buffers.size(); i++) {
        if (buffers[i] == nullptr) continue;
        auto [data, err] = cgo_bridge::CopyMetalBufferToFloat32Array(buffers[i], sizes[i] / 4);
        if (!err.empty()) return Errorf("failed to read %s buffer %d: %s", what, (int)i, err.c_str());
        OptimizerTensor t;
        t.Name = std::string(prefix) + "_" + std::to_string(i);
        t.Shape = {(int)data.size()};
        t.Data = std::move(data);
        t.StateType = stateType;
        out.push_back(std::move(t));
    }
    return "";
}

// The common part of every LoadState loop body: index and length validation.
static Error checkTensor(const OptimizerTensor &tensor, const std::vector<int> &bufferSizes, int &idx)
{
    idx = extractBufferIndex(tensor.Name);
    if (idx < 0 || idx >= (int)bufferSizes.size())
        return Errorf("invalid buffer index in tensor name: %s", tensor.Name.c_str());
    const int expectedElements = bufferSizes[idx] / 4;
    if ((int)tensor.Data.size() != expectedElements)
        return Errorf("data size mismatch for %s: expected %d elements, got %d", tensor.Name.c_str(),
                      expectedElements, (int)tensor.Data.size());
    return "";
}

static Error writeBuffer(Pointer buffer, const OptimizerTensor &tensor, int idx, const char *what)
{
    if (buffer == nullptr) return Errorf("%s buffer %d is nil", what, idx);
    Error err = cgo_bridge::CopyFloat32ArrayToMetalBuffer(buffer, tensor.Data);
    if (!err.empty()) return Errorf("failed to restore %s buffer %d: %s", what, idx, err.c_str());
    return "";
}

// ---------------------------------------------------------------------------- SGD ----

SGDConfig DefaultSGDConfig() { return SGDConfig{0.01f, 0.0f, 0.0f, false}; }

std::pair<std::unique_ptr<SGDOptimizerState>, Error> NewSGDOptimizer(const SGDConfig &config,
                                                                     const Shapes &weightShapes,
                                                                     memory::MemoryManager *memoryManager,
                                                                     Pointer device)
{
    if (Error e = checkCommon(memoryManager, device, weightShapes); !e.empty()) return {nullptr, e};
    if (config.LearningRate < 0) return {nullptr, Errorf("learning rate cannot be negative: %f", config.LearningRate)};
    if (config.Momentum < 0) return {nullptr, Errorf("momentum cannot be negative: %f", config.Momentum)};
    if (config.Momentum > 1.0f)
        return {nullptr, Errorf("momentum cannot be greater than 1.0: %f", config.Momentum)};
    if (config.WeightDecay < 0) return {nullptr, Errorf("weight decay cannot be negative: %f", config.WeightDecay)};

    const size_t n = weightShapes.size();
    auto sgd = std::make_unique<SGDOptimizerState>();
    sgd->LearningRate = config.LearningRate;
    sgd->Momentum = config.Momentum;
    sgd->WeightDecay = config.WeightDecay;
    sgd->Nesterov = config.Nesterov;
    sgd->WeightBuffers.assign(n, nullptr);
    sgd->memoryManager = memoryManager;
    sgd->device = device;
    sgd->bufferSizes.assign(n, 0);

    if (config.Momentum > 0) {                       // momentum buffers only when used (sgd.go:105-133)
        sgd->MomentumBuffers.assign(n, nullptr);
        for (size_t i = 0; i < n; i++) {
            const int size = calculateTensorSize(weightShapes[i]) * 4;
            sgd->bufferSizes[i] = size;
            Pointer momentumBuffer = memoryManager->AllocateStateBuffer(size, 0);
            if (momentumBuffer == nullptr) {
                releaseAll(memoryManager, sgd->MomentumBuffers);
                return {nullptr, Errorf("failed to allocate momentum buffer for weight %d", (int)i)};
            }
            sgd->MomentumBuffers[i] = momentumBuffer;
            Error err = cgo_bridge::ZeroMetalBuffer(device, momentumBuffer, size);
            if (!err.empty()) {
                releaseAll(memoryManager, sgd->MomentumBuffers);
                return {nullptr, Errorf("failed to zero momentum buffer for weight %d: %s", (int)i, err.c_str())};
            }
        }
    } else {
        for (size_t i = 0; i < n; i++) sgd->bufferSizes[i] = calculateTensorSize(weightShapes[i]) * 4;
    }
    return {std::move(sgd), ""};
}

Error SGDOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    return setWeights(WeightBuffers, weightBuffers);
}

Error SGDOptimizerState::Step(const std::vector<Pointer> &gradientBuffers)
{
    if (Error e = checkGradients(gradientBuffers, WeightBuffers); !e.empty()) return e;
    StepCount++;                                     // before the call; stays on error (sgd_test.go:694-720)
    Error err = cgo_bridge::ExecuteSGDStepMPSGraph(device, WeightBuffers, gradientBuffers, MomentumBuffers,
                                                   bufferSizes, LearningRate, Momentum, WeightDecay, Nesterov,
                                                   (int)StepCount);
    if (!err.empty()) return Errorf("SGD step execution failed: %s", err.c_str());
    return "";
}

void SGDOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = (pool != nullptr);
}

void SGDOptimizerState::Cleanup()
{
    if (!MomentumBuffers.empty() && memoryManager != nullptr) releaseAll(memoryManager, MomentumBuffers);
    MomentumBuffers.clear();
    WeightBuffers.clear();
    bufferSizes.clear();
}

StateResult SGDOptimizerState::GetState()
{
    auto st = std::make_unique<OptimizerState>();
    if (Momentum > 0 && !MomentumBuffers.empty()) {
        for (size_t i = 0; i < MomentumBuffers.size(); i++) {
            auto [tensor, err] = extractBufferState(MomentumBuffers[i], bufferSizes[i],
                                                    "momentum_" + std::to_string(i), "momentum");
            if (!err.empty()) return {nullptr, err};
            if (tensor) st->StateData.push_back(std::move(*tensor));
        }
    }
    st->Type = "SGD";
    st->Parameters = {{"learning_rate", LearningRate}, {"momentum", Momentum}, {"weight_decay", WeightDecay},
                      {"nesterov", Nesterov},          {"step_count", StepCount}};
    return {std::move(st), ""};
}

Error SGDOptimizerState::LoadState(const OptimizerState *state)
{
    if (Error e = validateStateType("SGD", state); !e.empty()) return e;
    LearningRate = extractFloat32Param(state->Parameters, "learning_rate", LearningRate);
    Momentum = extractFloat32Param(state->Parameters, "momentum", Momentum);
    WeightDecay = extractFloat32Param(state->Parameters, "weight_decay", WeightDecay);
    Nesterov = extractBoolParam(state->Parameters, "nesterov", Nesterov);
    StepCount = extractUint64Param(state->Parameters, "step_count", StepCount);
    for (const OptimizerTensor &tensor : state->StateData) {
        if (tensor.StateType != "momentum") continue;
        const int idx = extractBufferIndex(tensor.Name);
        if (idx < 0 || idx >= (int)bufferSizes.size())
            return Errorf("invalid buffer index in tensor name: %s", tensor.Name.c_str());
        if (MomentumBuffers.empty() || MomentumBuffers[idx] == nullptr)
            return Errorf("momentum buffer %d not allocated", idx);
        if (Error e = restoreBufferState(MomentumBuffers[idx], tensor.Data, bufferSizes[idx], tensor.Name); !e.empty())
            return e;
    }
    return "";
}

// --------------------------------------------------------------------------- Adam ----

AdamConfig DefaultAdamConfig() { return AdamConfig{0.001f, 0.9f, 0.999f, 1e-8f, 0.0f}; }

// Allocates and zeroes the (first, second) state buffers of every tensor with the
// unwinding order of adam.go:98-135 / nadam.go:109-146.
static Error allocateMoments(memory::MemoryManager *mm, Pointer device, const Shapes &weightShapes,
                             std::vector<Pointer> &first, std::vector<Pointer> &second,
                             std::vector<int> &bufferSizes)
{
    const size_t n = weightShapes.size();
    auto unwind = [&](Error e) {
        releaseAll(mm, first);
        releaseAll(mm, second);
        return e;
    };
    for (size_t i = 0; i < n; i++) {
        const int size = calculateTensorSize(weightShapes[i]) * 4;
        bufferSizes[i] = size;
        // (the two moments of a tensor start at phases of their own: memory_manager.hpp, kStatePhases)
        Pointer momentumBuffer = mm->AllocateStateBuffer(size, 0);
        if (momentumBuffer == nullptr)
            return unwind(Errorf("failed to allocate momentum buffer for weight %d", (int)i));
        first[i] = momentumBuffer;
        Pointer varianceBuffer = mm->AllocateStateBuffer(size, 1);
        if (varianceBuffer == nullptr)
            return unwind(Errorf("failed to allocate variance buffer for weight %d", (int)i));
        second[i] = varianceBuffer;
        Error err = cgo_bridge::ZeroMetalBuffer(device, momentumBuffer, size);
        if (!err.empty())
            return unwind(Errorf("failed to zero momentum buffer for weight %d: %s", (int)i, err.c_str()));
        err = cgo_bridge::ZeroMetalBuffer(device, varianceBuffer, size);
        if (!err.empty())
            return unwind(Errorf("failed to zero variance buffer for weight %d: %s", (int)i, err.c_str()));
    }
    return "";
}

std::pair<std::unique_ptr<AdamOptimizerState>, Error> NewAdamOptimizer(const AdamConfig &config,
                                                                       const Shapes &weightShapes,
                                                                       memory::MemoryManager *memoryManager,
                                                                       Pointer device)
{
    if (Error e = checkCommon(memoryManager, device, weightShapes); !e.empty()) return {nullptr, e};
    const size_t n = weightShapes.size();
    auto adam = std::make_unique<AdamOptimizerState>();
    adam->LearningRate = config.LearningRate;
    adam->Beta1 = config.Beta1;
    adam->Beta2 = config.Beta2;
    adam->Epsilon = config.Epsilon;
    adam->WeightDecay = config.WeightDecay;
    adam->MomentumBuffers.assign(n, nullptr);
    adam->VarianceBuffers.assign(n, nullptr);
    adam->WeightBuffers.assign(n, nullptr);
    adam->memoryManager = memoryManager;
    adam->device = device;
    adam->bufferSizes.assign(n, 0);
    if (Error e = allocateMoments(memoryManager, device, weightShapes, adam->MomentumBuffers,
                                  adam->VarianceBuffers, adam->bufferSizes);
        !e.empty())
        return {nullptr, e};
    return {std::move(adam), ""};
}

AdamOptimizerState::~AdamOptimizerState()
{
    if (ampState) gm_amp_state_destroy(reinterpret_cast<uintptr_t>(ampState));
}

Error AdamOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    return setWeights(WeightBuffers, weightBuffers);
}

uint64_t AdamOptimizerState::GetStepCount()
{
    if (ampPending > 0) (void)SyncAMP();     // pending asynchronous steps: the device holds the count
    return StepCount;
}

Error AdamOptimizerState::Step(const std::vector<Pointer> &gradientBuffers)
{
    if (Error e = checkGradients(gradientBuffers, WeightBuffers); !e.empty()) return e;
    if (ampPending > 0)
        if (Error e = SyncAMP(); !e.empty()) return e;
    StepCount++;
    ampCountDirty = true;
    // As in adam.go:191-227 the pooled entry point is not used even when a pool is set.
    // (with ping-pong state the fp32 step updates whichever set is current, in place)
    Error err = cgo_bridge::ExecuteAdamStepMPSGraph(device, CurrentWeightBuffers(), gradientBuffers,
                                                    CurrentMomentumBuffers(), CurrentVarianceBuffers(), bufferSizes,
                                                    LearningRate, Beta1, Beta2, Epsilon, WeightDecay, (int)StepCount);
    if (!err.empty()) return Errorf("Adam step execution failed: %s", err.c_str());
    return "";
}

Error AdamOptimizerState::EnableMixedPrecision(float initialScale, float growthFactor, float backoffFactor,
                                               int growthInterval)
{
    if (device == nullptr) return Errorf("device cannot be nil");
    if (!(initialScale > 0)) return Errorf("initial loss scale must be positive, got %f", initialScale);
    if (growthInterval <= 0) return Errorf("growth interval must be positive, got %d", growthInterval);
    if (ampState) {
        // a second call replaces the loss-scale state; steps still in flight finish first, and with ping-pong
        // state on, the new device state is told which set is current (a fresh one would say set A)
        if (ampPending > 0)
            if (Error e = SyncAMP(); !e.empty()) return e;
        gm_amp_state_destroy(reinterpret_cast<uintptr_t>(ampState));
    }
    ampState = reinterpret_cast<Pointer>(gm_amp_state_create(reinterpret_cast<uintptr_t>(device), initialScale,
                                                             growthFactor, backoffFactor, growthInterval));
    if (ampState == nullptr) return Errorf("failed to create loss-scale state: %s", gm_last_error());
    if (pingPong && currentSet != 0 &&
        gm_amp_state_set_current_set(reinterpret_cast<uintptr_t>(ampState), currentSet) != 0)
        return Errorf("failed to carry the current ping-pong set over: %s", gm_last_error());
    LossScale = initialScale;
    GrowthTracker = 0;
    ampPending = 0;
    ampCountDirty = true;
    return "";
}

Error AdamOptimizerState::EnablePingPong()
{
    if (ampState == nullptr) return Errorf("mixed precision is not enabled: call EnableMixedPrecision first");
    if (pingPong) return "";
    if (memoryManager == nullptr) return Errorf("memory manager cannot be nil");
    for (Pointer w : WeightBuffers)
        if (w == nullptr) return Errorf("weight buffers are not set: call SetWeightBuffers first");
    std::vector<Pointer> *lists[3] = {&ShadowWeightBuffers, &ShadowMomentumBuffers, &ShadowVarianceBuffers};
    const int phases[3] = {memory::kShadowWeightPhase, memory::kStatePhases[0], memory::kStatePhases[1]};
    for (int k = 0; k < 3; k++) {
        auto *list = lists[k];
        list->assign(bufferSizes.size(), nullptr);
        for (size_t i = 0; i < bufferSizes.size(); i++) {
            (*list)[i] = memoryManager->AllocateBufferAtPhase(bufferSizes[i], phases[k]);
            if ((*list)[i] == nullptr) {
                for (auto *undo : lists) {
                    releaseAll(memoryManager, *undo);
                    undo->clear();
                }
                return Errorf("failed to allocate ping-pong buffer for weight %d", (int)i);
            }
        }
    }
    pingPong = true;
    currentSet = 0;
    return "";
}

Error AdamOptimizerState::refreshCurrentSet()
{
    if (!pingPong) return "";
    if (ampPending > 0)
        if (Error e = SyncAMP(); !e.empty()) return e;
    return "";
}

const std::vector<Pointer> &AdamOptimizerState::CurrentWeightBuffers()
{
    (void)refreshCurrentSet();
    return pingPong && currentSet == 1 ? ShadowWeightBuffers : WeightBuffers;
}

const std::vector<Pointer> &AdamOptimizerState::CurrentMomentumBuffers()
{
    (void)refreshCurrentSet();
    return pingPong && currentSet == 1 ? ShadowMomentumBuffers : MomentumBuffers;
}

const std::vector<Pointer> &AdamOptimizerState::CurrentVarianceBuffers()
{
    (void)refreshCurrentSet();
    return pingPong && currentSet == 1 ? ShadowVarianceBuffers : VarianceBuffers;
}

Error AdamOptimizerState::SyncAMP(uint64_t *skippedSteps)
{
    if (ampState == nullptr) return Errorf("mixed precision is not enabled: call EnableMixedPrecision first");
    int applied = 0, skipped = 0;
    if (gm_amp_state_query(reinterpret_cast<uintptr_t>(ampState), &LossScale, &GrowthTracker, &applied, &skipped) != 0)
        return Errorf("failed to read loss-scale state: %s", gm_last_error());
    if (ampPending > 0) StepCount = (uint64_t)applied;     // the device counted the pending steps
    if (pingPong) {
        const int set = gm_amp_state_current_set(reinterpret_cast<uintptr_t>(ampState));
        if (set < 0) return Errorf("failed to read the current ping-pong set: %s", gm_last_error());
        currentSet = set;
    }
    ampPending = 0;
    if (skippedSteps) *skippedSteps = (uint64_t)skipped;
    return "";
}

Error AdamOptimizerState::StepAMPAsync(const std::vector<Pointer> &gradient16Buffers,
                                       const std::vector<Pointer> &weight16Buffers)
{
    if (Error e = checkGradients(gradient16Buffers, WeightBuffers); !e.empty()) return e;
    if (!weight16Buffers.empty() && weight16Buffers.size() != WeightBuffers.size())
        return Errorf("fp16 weight buffers length (%d) doesn't match weight buffers length (%d)",
                      (int)weight16Buffers.size(), (int)WeightBuffers.size());
    if (ampState == nullptr) return Errorf("mixed precision is not enabled: call EnableMixedPrecision first");
    if (ampCountDirty) {
        if (gm_amp_state_set_step_count(reinterpret_cast<uintptr_t>(ampState), (int)StepCount) != 0)
            return Errorf("failed to set the device step count: %s", gm_last_error());
        ampCountDirty = false;
    }
    Error err;
    if (pingPong) {
        const std::vector<Pointer> a[3] = {WeightBuffers, MomentumBuffers, VarianceBuffers};
        const std::vector<Pointer> b[3] = {ShadowWeightBuffers, ShadowMomentumBuffers, ShadowVarianceBuffers};
        err = cgo_bridge::ExecuteAdamAMPStepFusedAsync(device, a, b, gradient16Buffers, weight16Buffers, bufferSizes,
                                                       LearningRate, Beta1, Beta2, Epsilon, WeightDecay, ampState);
    } else {
        err = cgo_bridge::ExecuteAdamAMPStepAsync(device, WeightBuffers, gradient16Buffers, MomentumBuffers,
                                                  VarianceBuffers, weight16Buffers, bufferSizes, LearningRate,
                                                  Beta1, Beta2, Epsilon, WeightDecay, ampState);
    }
    if (!err.empty()) return Errorf("Adam mixed-precision step execution failed: %s", err.c_str());
    ampPending++;
    return "";
}

std::pair<bool, Error> AdamOptimizerState::StepAMP(const std::vector<Pointer> &gradient16Buffers,
                                                   const std::vector<Pointer> &weight16Buffers)
{
    if (Error e = checkGradients(gradient16Buffers, WeightBuffers); !e.empty()) return {false, e};
    if (!weight16Buffers.empty() && weight16Buffers.size() != WeightBuffers.size())
        return {false, Errorf("fp16 weight buffers length (%d) doesn't match weight buffers length (%d)",
                              (int)weight16Buffers.size(), (int)WeightBuffers.size())};
    if (ampState == nullptr) return {false, Errorf("mixed precision is not enabled: call EnableMixedPrecision first")};
    if (ampPending > 0)
        if (Error e = SyncAMP(); !e.empty()) return {false, e};
    if (ampCountDirty) {
        if (gm_amp_state_set_step_count(reinterpret_cast<uintptr_t>(ampState), (int)StepCount) != 0)
            return {false, Errorf("failed to set the device step count: %s", gm_last_error())};
        ampCountDirty = false;
    }
    bool skipped = false;
    // StepCount advances only when the step is applied: the bias corrections are taken at StepCount + 1.
    Error err;
    if (pingPong) {
        const std::vector<Pointer> a[3] = {WeightBuffers, MomentumBuffers, VarianceBuffers};
        const std::vector<Pointer> b[3] = {ShadowWeightBuffers, ShadowMomentumBuffers, ShadowVarianceBuffers};
        err = cgo_bridge::ExecuteAdamAMPStepFused(device, a, b, gradient16Buffers, weight16Buffers, bufferSizes,
                                                  LearningRate, Beta1, Beta2, Epsilon, WeightDecay, (int)(StepCount + 1),
                                                  ampState, &skipped, &LossScale, &GrowthTracker, &currentSet);
    } else {
        err = cgo_bridge::ExecuteAdamAMPStep(device, WeightBuffers, gradient16Buffers, MomentumBuffers,
                                             VarianceBuffers, weight16Buffers, bufferSizes, LearningRate, Beta1,
                                             Beta2, Epsilon, WeightDecay, (int)(StepCount + 1), ampState, &skipped,
                                             &LossScale, &GrowthTracker);
    }
    if (!err.empty()) return {false, Errorf("Adam mixed-precision step execution failed: %s", err.c_str())};
    if (!skipped) StepCount++;
    return {skipped, ""};
}

void AdamOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = (pool != nullptr);
}

AdamStats AdamOptimizerState::GetStats()
{
    int total = 0;
    for (int size : bufferSizes) total += size * 2;   // momentum + variance buffers
    return AdamStats{StepCount, LearningRate, Beta1, Beta2, Epsilon, WeightDecay, (int)WeightBuffers.size(), total};
}

void AdamOptimizerState::Cleanup()
{
    if (memoryManager != nullptr) {
        releaseAll(memoryManager, MomentumBuffers);
        releaseAll(memoryManager, VarianceBuffers);
        releaseAll(memoryManager, ShadowWeightBuffers);
        releaseAll(memoryManager, ShadowMomentumBuffers);
        releaseAll(memoryManager, ShadowVarianceBuffers);
    }
    MomentumBuffers.clear();
    VarianceBuffers.clear();
    ShadowWeightBuffers.clear();
    ShadowMomentumBuffers.clear();
    ShadowVarianceBuffers.clear();
    pingPong = false;
    currentSet = 0;
    WeightBuffers.clear();
    bufferSizes.clear();
}

StateResult AdamOptimizerState::GetState()
{
    if (ampPending > 0)
        if (Error e = SyncAMP(); !e.empty()) return {nullptr, e};
    auto st = std::make_unique<OptimizerState>();
    if (Error e = readBuffers(CurrentMomentumBuffers(), bufferSizes, "momentum", "momentum", "momentum", st->StateData); !e.empty())
        return {nullptr, e};
    if (Error e = readBuffers(CurrentVarianceBuffers(), bufferSizes, "variance", "variance", "variance", st->StateData); !e.empty())
        return {nullptr, e};
    st->Type = "Adam";
    st->Parameters = {{"learning_rate", LearningRate}, {"beta1", Beta1},
                      {"beta2", Beta2},                {"epsilon", Epsilon},
                      {"weight_decay", WeightDecay},   {"step_count", StepCount}};
    if (ampState) {   // additive keys, present only when mixed precision is on
        st->Parameters["loss_scale"] = LossScale;
        st->Parameters["growth_tracker"] = (uint64_t)GrowthTracker;
    }
    return {std::move(st), ""};
}

Error AdamOptimizerState::LoadState(const OptimizerState *state)
{
    if (Error e = validateStateType("Adam", state); !e.empty()) return e;
    if (ampPending > 0)
        if (Error e = SyncAMP(); !e.empty()) return e;
    ampCountDirty = true;
    setFloat(state->Parameters, "learning_rate", LearningRate);
    setFloat(state->Parameters, "beta1", Beta1);
    setFloat(state->Parameters, "beta2", Beta2);
    setFloat(state->Parameters, "epsilon", Epsilon);
    setFloat(state->Parameters, "weight_decay", WeightDecay);
    if (const double *sc = asFloat64(state->Parameters, "step_count")) StepCount = toUint64(*sc);
    if (ampState) {
        const double *ls = asFloat64(state->Parameters, "loss_scale");
        const double *gt = asFloat64(state->Parameters, "growth_tracker");
        if (ls || gt) {
            if (ls) LossScale = (float)*ls;
            if (gt) GrowthTracker = toInt(*gt);
            if (gm_amp_state_set(reinterpret_cast<uintptr_t>(ampState), LossScale, GrowthTracker) != 0)
                return Errorf("failed to restore loss-scale state: %s", gm_last_error());
        }
    }
    for (const OptimizerTensor &tensor : state->StateData) {
        int idx;
        if (Error e = checkTensor(tensor, bufferSizes, idx); !e.empty()) return e;
        Error e;
        if (tensor.StateType == "momentum") e = writeBuffer(CurrentMomentumBuffers()[idx], tensor, idx, "momentum");
        else if (tensor.StateType == "variance") e = writeBuffer(CurrentVarianceBuffers()[idx], tensor, idx, "variance");
        else e = Errorf("unknown state type: %s", tensor.StateType.c_str());
        if (!e.empty()) return e;
    }
    return "";
}

// ------------------------------------------------------------------------ RMSProp ----

RMSPropConfig DefaultRMSPropConfig() { return RMSPropConfig{0.01f, 0.99f, 1e-8f, 0.0f, 0.0f, false}; }

std::pair<std::unique_ptr<RMSPropOptimizerState>, Error> NewRMSPropOptimizer(const RMSPropConfig &config,
                                                                             const Shapes &weightShapes,
                                                                             memory::MemoryManager *memoryManager,
                                                                             Pointer device)
{
    if (Error e = checkCommon(memoryManager, device, weightShapes); !e.empty()) return {nullptr, e};
    const size_t n = weightShapes.size();
    auto r = std::make_unique<RMSPropOptimizerState>();
    r->LearningRate = config.LearningRate;
    r->Alpha = config.Alpha;
    r->Epsilon = config.Epsilon;
    r->WeightDecay = config.WeightDecay;
    r->Momentum = config.Momentum;
    r->Centered = config.Centered;
    r->SquaredGradAvgBuffers.assign(n, nullptr);
    r->MomentumBuffers.assign(n, nullptr);
    r->GradientAvgBuffers.assign(n, nullptr);
    r->WeightBuffers.assign(n, nullptr);
    r->memoryManager = memoryManager;
    r->device = device;
    r->bufferSizes.assign(n, 0);
    auto unwind = [&](Error e) {
        releaseAll(memoryManager, r->SquaredGradAvgBuffers);
        releaseAll(memoryManager, r->MomentumBuffers);
        releaseAll(memoryManager, r->GradientAvgBuffers);
        return std::pair<std::unique_ptr<RMSPropOptimizerState>, Error>{nullptr, e};
    };
    for (size_t i = 0; i < n; i++) {
        const int size = calculateTensorSize(weightShapes[i]) * 4;
        r->bufferSizes[i] = size;
        Pointer s = memoryManager->AllocateStateBuffer(size, 0);
        if (s == nullptr)
            return unwind(Errorf("failed to allocate squared gradient average buffer for weight %d", (int)i));
        r->SquaredGradAvgBuffers[i] = s;
        if (config.Momentum > 0.0f) {
            Pointer b = memoryManager->AllocateStateBuffer(size, 1);
            if (b == nullptr) return unwind(Errorf("failed to allocate momentum buffer for weight %d", (int)i));
            r->MomentumBuffers[i] = b;
        }
        if (config.Centered) {
            Pointer ga = memoryManager->AllocateStateBuffer(size, 2);
            if (ga == nullptr)
                return unwind(Errorf("failed to allocate gradient average buffer for weight %d", (int)i));
            r->GradientAvgBuffers[i] = ga;
        }
        Error err = cgo_bridge::ZeroMetalBuffer(device, s, size);
        if (!err.empty())
            return unwind(Errorf("failed to zero squared gradient average buffer for weight %d: %s", (int)i,
                                 err.c_str()));
        if (r->MomentumBuffers[i] != nullptr) {
            err = cgo_bridge::ZeroMetalBuffer(device, r->MomentumBuffers[i], size);
            if (!err.empty())
                return unwind(Errorf("failed to zero momentum buffer for weight %d: %s", (int)i, err.c_str()));
        }
        if (r->GradientAvgBuffers[i] != nullptr) {
            err = cgo_bridge::ZeroMetalBuffer(device, r->GradientAvgBuffers[i], size);
            if (!err.empty())
                return unwind(Errorf("failed to zero gradient average buffer for weight %d: %s", (int)i,
                                     err.c_str()));
        }
    }
    return {std::move(r), ""};
}

Error RMSPropOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    return setWeights(WeightBuffers, weightBuffers);
}

Error RMSPropOptimizerState::Step(const std::vector<Pointer> &gradientBuffers)
{
    if (Error e = checkGradients(gradientBuffers, WeightBuffers); !e.empty()) return e;
    StepCount++;
    Error err = cgo_bridge::ExecuteRMSPropStepMPSGraph(device, WeightBuffers, gradientBuffers,
                                                       SquaredGradAvgBuffers, MomentumBuffers, GradientAvgBuffers,
                                                       bufferSizes, LearningRate, Alpha, Epsilon, WeightDecay,
                                                       Momentum, Centered, (int)StepCount);
    if (!err.empty()) return Errorf("RMSProp step execution failed: %s", err.c_str());
    return "";
}

void RMSPropOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = (pool != nullptr);
}

RMSPropStats RMSPropOptimizerState::GetStats()
{
    int total = 0;
    for (int size : bufferSizes) {
        total += size;
        if (Momentum > 0.0f) total += size;
        if (Centered) total += size;
    }
    return RMSPropStats{StepCount, LearningRate, Alpha, Epsilon, WeightDecay, Momentum, Centered,
                        (int)WeightBuffers.size(), total};
}

void RMSPropOptimizerState::Cleanup()
{
    if (memoryManager != nullptr) {
        releaseAll(memoryManager, SquaredGradAvgBuffers);
        releaseAll(memoryManager, MomentumBuffers);
        releaseAll(memoryManager, GradientAvgBuffers);
    }
    SquaredGradAvgBuffers.clear();
    MomentumBuffers.clear();
    GradientAvgBuffers.clear();
    WeightBuffers.clear();
    bufferSizes.clear();
}

StateResult RMSPropOptimizerState::GetState()
{
    auto st = std::make_unique<OptimizerState>();
    if (Error e = readBuffers(SquaredGradAvgBuffers, bufferSizes, "squared_grad_avg", "squared_grad_avg",
                              "squared grad avg", st->StateData);
        !e.empty())
        return {nullptr, e};
    if (Momentum > 0)
        if (Error e = readBuffers(MomentumBuffers, bufferSizes, "momentum", "momentum", "momentum", st->StateData);
            !e.empty())
            return {nullptr, e};
    if (Centered)
        if (Error e = readBuffers(GradientAvgBuffers, bufferSizes, "gradient_avg", "gradient_avg", "gradient avg",
                                  st->StateData);
            !e.empty())
            return {nullptr, e};
    st->Type = "RMSProp";
    st->Parameters = {{"learning_rate", LearningRate}, {"alpha", Alpha},       {"epsilon", Epsilon},
                      {"weight_decay", WeightDecay},   {"momentum", Momentum}, {"centered", Centered},
                      {"step_count", StepCount}};
    return {std::move(st), ""};
}

Error RMSPropOptimizerState::LoadState(const OptimizerState *state)
{
    if (Error e = validateStateType("RMSProp", state); !e.empty()) return e;
    setFloat(state->Parameters, "learning_rate", LearningRate);
    setFloat(state->Parameters, "alpha", Alpha);
    setFloat(state->Parameters, "epsilon", Epsilon);
    setFloat(state->Parameters, "weight_decay", WeightDecay);
    setFloat(state->Parameters, "momentum", Momentum);
    Centered = extractBoolParam(state->Parameters, "centered", Centered);
    if (const double *sc = asFloat64(state->Parameters, "step_count")) StepCount = toUint64(*sc);
    for (const OptimizerTensor &tensor : state->StateData) {
        int idx;
        if (Error e = checkTensor(tensor, bufferSizes, idx); !e.empty()) return e;
        Error e;
        if (tensor.StateType == "squared_grad_avg")
            e = writeBuffer(SquaredGradAvgBuffers[idx], tensor, idx, "squared grad avg");
        else if (tensor.StateType == "momentum") e = writeBuffer(MomentumBuffers[idx], tensor, idx, "momentum");
        else if (tensor.StateType == "gradient_avg")
            e = writeBuffer(GradientAvgBuffers[idx], tensor, idx, "gradient avg");
        else e = Errorf("unknown state type: %s", tensor.StateType.c_str());
        if (!e.empty()) return e;
    }
    return "";
}

// ------------------------------------------------------------------------ AdaGrad ----

AdaGradConfig DefaultAdaGradConfig() { return AdaGradConfig{0.01f, 1e-10f, 0.0f}; }

std::pair<std::unique_ptr<AdaGradOptimizerState>, Error> NewAdaGradOptimizer(const AdaGradConfig &config,
                                                                             const Shapes &weightShapes,
                                                                             memory::MemoryManager *memoryManager,
                                                                             Pointer device)
{
    if (Error e = checkCommon(memoryManager, device, weightShapes); !e.empty()) return {nullptr, e};
    const size_t n = weightShapes.size();
    auto a = std::make_unique<AdaGradOptimizerState>();
    a->config = config;
    a->squaredGradAvgBuffers.assign(n, nullptr);
    a->WeightBuffers.assign(n, nullptr);
    a->memoryManager = memoryManager;
    a->device = device;
    a->bufferSizes.assign(n, 0);
    for (size_t i = 0; i < n; i++) {
        a->bufferSizes[i] = calculateTensorSize(weightShapes[i]) * 4;
        Pointer s = memoryManager->AllocateStateBuffer(a->bufferSizes[i], 0);
        if (s == nullptr) {
            a->Cleanup();
            return {nullptr, Errorf("failed to allocate squared gradient average buffer for weight %d", (int)i)};
        }
        a->squaredGradAvgBuffers[i] = s;
        Error err = cgo_bridge::ZeroMetalBuffer(device, s, a->bufferSizes[i]);
        if (!err.empty()) {
            a->Cleanup();
            return {nullptr, Errorf("failed to zero squared gradient average buffer: %s", err.c_str())};
        }
    }
    return {std::move(a), ""};
}

void AdaGradOptimizerState::cleanup() { releaseAll(memoryManager, squaredGradAvgBuffers); }
void AdaGradOptimizerState::Cleanup() { cleanup(); }

Error AdaGradOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    return setWeights(WeightBuffers, weightBuffers);
}

Error AdaGradOptimizerState::Step(const std::vector<Pointer> &gradientBuffers)
{
    if (Error e = checkGradients(gradientBuffers, WeightBuffers); !e.empty()) return e;
    currentStep++;
    Error err;
    if (usePooling && commandPool != nullptr)
        err = cgo_bridge::ExecuteAdaGradStepMPSGraphPooled(device, WeightBuffers, gradientBuffers,
                                                           squaredGradAvgBuffers, (int)WeightBuffers.size(),
                                                           bufferSizes, config.LearningRate, config.Epsilon,
                                                           config.WeightDecay, commandPool);
    else
        err = cgo_bridge::ExecuteAdaGradStepMPSGraph(device, WeightBuffers, gradientBuffers, squaredGradAvgBuffers,
                                                     (int)WeightBuffers.size(), bufferSizes, config.LearningRate,
                                                     config.Epsilon, config.WeightDecay);
    if (!err.empty()) return Errorf("AdaGrad step failed: %s", err.c_str());
    if (logProgress && currentStep % 10 == 0)
        std::printf("AdaGrad step %llu completed, lr=%.6f\n", (unsigned long long)currentStep, config.LearningRate);
    return "";
}

void AdaGradOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = (pool != nullptr);
}

std::map<std::string, ParamValue> AdaGradOptimizerState::GetStats()
{
    return {{"step", currentStep},
            {"learning_rate", config.LearningRate},
            {"epsilon", config.Epsilon},
            {"weight_decay", config.WeightDecay}};
}

StateResult AdaGradOptimizerState::GetState()
{
    auto st = std::make_unique<OptimizerState>();
    if (Error e = readBuffers(squaredGradAvgBuffers, bufferSizes, "squared_grad_avg", "squared_grad_avg",
                              "squared gradient average", st->StateData);
        !e.empty())
        return {nullptr, e};
    st->Type = "AdaGrad";
    st->Parameters = {{"learning_rate", config.LearningRate},
                      {"epsilon", config.Epsilon},
                      {"weight_decay", config.WeightDecay},
                      {"step_count", currentStep}};
    return {std::move(st), ""};
}

Error AdaGradOptimizerState::LoadState(const OptimizerState *state)
{
    if (Error e = validateStateType("AdaGrad", state); !e.empty()) return e;
    setFloat(state->Parameters, "learning_rate", config.LearningRate);
    setFloat(state->Parameters, "epsilon", config.Epsilon);
    setFloat(state->Parameters, "weight_decay", config.WeightDecay);
    loadStepCountLenient(state->Parameters, currentStep);
    for (const OptimizerTensor &tensor : state->StateData) {
        int idx;
        if (Error e = checkTensor(tensor, bufferSizes, idx); !e.empty()) return e;
        Error e;
        if (tensor.StateType == "squared_grad_avg")
            e = writeBuffer(squaredGradAvgBuffers[idx], tensor, idx, "squared gradient average");
        else e = Errorf("unknown state type: %s", tensor.StateType.c_str());
        if (!e.empty()) return e;
    }
    return "";
}

// ----------------------------------------------------------------------- AdaDelta ----

AdaDeltaConfig DefaultAdaDeltaConfig() { return AdaDeltaConfig{0.95f, 1e-6f, 0.0f}; }

std::pair<std::unique_ptr<AdaDeltaOptimizerState>, Error> NewAdaDeltaOptimizer(const AdaDeltaConfig &config,
                                                                               const Shapes &weightShapes,
                                                                               memory::MemoryManager *memoryManager,
                                                                               Pointer device)
{
    if (Error e = checkCommon(memoryManager, device, weightShapes); !e.empty()) return {nullptr, e};
    if (config.Rho <= 0 || config.Rho >= 1) return {nullptr, Errorf("rho must be in range (0, 1), got %f", config.Rho)};
    const size_t n = weightShapes.size();
    auto a = std::make_unique<AdaDeltaOptimizerState>();
    a->config = config;
    a->squaredGradAvgBuffers.assign(n, nullptr);
    a->squaredUpdateAvgBuffers.assign(n, nullptr);
    a->WeightBuffers.assign(n, nullptr);
    a->memoryManager = memoryManager;
    a->device = device;
    a->bufferSizes.assign(n, 0);
    for (size_t i = 0; i < n; i++) {
        a->bufferSizes[i] = calculateTensorSize(weightShapes[i]) * 4;
        Pointer s = memoryManager->AllocateStateBuffer(a->bufferSizes[i], 0);
        if (s == nullptr) {
            a->Cleanup();
            return {nullptr, Errorf("failed to allocate squared gradient average buffer for weight %d", (int)i)};
        }
        a->squaredGradAvgBuffers[i] = s;
        Pointer u = memoryManager->AllocateStateBuffer(a->bufferSizes[i], 1);
        if (u == nullptr) {
            a->Cleanup();
            return {nullptr, Errorf("failed to allocate squared update average buffer for weight %d", (int)i)};
        }
        a->squaredUpdateAvgBuffers[i] = u;
        Error err = cgo_bridge::ZeroMetalBuffer(device, s, a->bufferSizes[i]);
        if (!err.empty()) {
            a->Cleanup();
            return {nullptr, Errorf("failed to zero squared gradient average buffer: %s", err.c_str())};
        }
        err = cgo_bridge::ZeroMetalBuffer(device, u, a->bufferSizes[i]);
        if (!err.empty()) {
            a->Cleanup();
            return {nullptr, Errorf("failed to zero squared update average buffer: %s", err.c_str())};
        }
    }
    return {std::move(a), ""};
}

void AdaDeltaOptimizerState::cleanup()
{
    releaseAll(memoryManager, squaredGradAvgBuffers);
    releaseAll(memoryManager, squaredUpdateAvgBuffers);
}
void AdaDeltaOptimizerState::Cleanup() { cleanup(); }

Error AdaDeltaOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    return setWeights(WeightBuffers, weightBuffers);
}

Error AdaDeltaOptimizerState::Step(const std::vector<Pointer> &gradientBuffers)
{
    if (Error e = checkGradients(gradientBuffers, WeightBuffers); !e.empty()) return e;
    currentStep++;
    Error err;
    if (usePooling && commandPool != nullptr)
        err = cgo_bridge::ExecuteAdaDeltaStepMPSGraphPooled(device, WeightBuffers, gradientBuffers,
                                                            squaredGradAvgBuffers, squaredUpdateAvgBuffers,
                                                            (int)WeightBuffers.size(), bufferSizes, config.Rho,
                                                            config.Epsilon, config.WeightDecay, commandPool);
    else
        err = cgo_bridge::ExecuteAdaDeltaStepMPSGraph(device, WeightBuffers, gradientBuffers, squaredGradAvgBuffers,
                                                      squaredUpdateAvgBuffers, (int)WeightBuffers.size(),
                                                      bufferSizes, config.Rho, config.Epsilon, config.WeightDecay);
    if (!err.empty()) return Errorf("AdaDelta step failed: %s", err.c_str());
    if (logProgress && currentStep % 10 == 0)
        std::printf("AdaDelta step %llu completed, rho=%.3f\n", (unsigned long long)currentStep, config.Rho);
    return "";
}

void AdaDeltaOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = (pool != nullptr);
}

std::map<std::string, ParamValue> AdaDeltaOptimizerState::GetStats()
{
    return {{"step", currentStep}, {"rho", config.Rho}, {"epsilon", config.Epsilon},
            {"weight_decay", config.WeightDecay}};
}

StateResult AdaDeltaOptimizerState::GetState()
{
    auto st = std::make_unique<OptimizerState>();
    if (Error e = readBuffers(squaredGradAvgBuffers, bufferSizes, "squared_grad_avg", "squared_grad_avg",
                              "squared gradient average", st->StateData);
        !e.empty())
        return {nullptr, e};
    if (Error e = readBuffers(squaredUpdateAvgBuffers, bufferSizes, "squared_update_avg", "squared_update_avg",
                              "squared update average", st->StateData);
        !e.empty())
        return {nullptr, e};
    st->Type = "AdaDelta";
    st->Parameters = {{"rho", config.Rho}, {"epsilon", config.Epsilon}, {"weight_decay", config.WeightDecay},
                      {"step_count", currentStep}};
    return {std::move(st), ""};
}

Error AdaDeltaOptimizerState::LoadState(const OptimizerState *state)
{
    if (Error e = validateStateType("AdaDelta", state); !e.empty()) return e;
    setFloat(state->Parameters, "rho", config.Rho);
    setFloat(state->Parameters, "epsilon", config.Epsilon);
    setFloat(state->Parameters, "weight_decay", config.WeightDecay);
    loadStepCountLenient(state->Parameters, currentStep);
    for (const OptimizerTensor &tensor : state->StateData) {
        int idx;
        if (Error e = checkTensor(tensor, bufferSizes, idx); !e.empty()) return e;
        Error e;
        if (tensor.StateType == "squared_grad_avg")
            e = writeBuffer(squaredGradAvgBuffers[idx], tensor, idx, "squared gradient average");
        else if (tensor.StateType == "squared_update_avg")
            e = writeBuffer(squaredUpdateAvgBuffers[idx], tensor, idx, "squared update average");
        else e = Errorf("unknown state type: %s", tensor.StateType.c_str());
        if (!e.empty()) return e;
    }
    return "";
}

// -------------------------------------------------------------------------- Nadam ----

NadamConfig DefaultNadamConfig() { return NadamConfig{0.002f, 0.9f, 0.999f, 1e-8f, 0.0f}; }

std::pair<std::unique_ptr<NadamOptimizerState>, Error> NewNadamOptimizer(const NadamConfig &config,
                                                                         const Shapes &weightShapes,
                                                                         memory::MemoryManager *memoryManager,
                                                                         Pointer device)
{
    if (Error e = checkCommon(memoryManager, device, weightShapes); !e.empty()) return {nullptr, e};
    if (config.LearningRate <= 0)
        return {nullptr, Errorf("learning rate must be positive, got %f", config.LearningRate)};
    if (config.Beta1 < 0 || config.Beta1 >= 1) return {nullptr, Errorf("beta1 must be in [0, 1), got %f", config.Beta1)};
    if (config.Beta2 < 0 || config.Beta2 >= 1) return {nullptr, Errorf("beta2 must be in [0, 1), got %f", config.Beta2)};
    if (config.Epsilon <= 0) return {nullptr, Errorf("epsilon must be positive, got %e", config.Epsilon)};
    if (config.WeightDecay < 0)
        return {nullptr, Errorf("weight decay must be non-negative, got %f", config.WeightDecay)};
    const size_t n = weightShapes.size();
    auto nadam = std::make_unique<NadamOptimizerState>();
    nadam->config = config;
    nadam->momentumBuffers.assign(n, nullptr);
    nadam->varianceBuffers.assign(n, nullptr);
    nadam->WeightBuffers.assign(n, nullptr);
    nadam->memoryManager = memoryManager;
    nadam->device = device;
    nadam->bufferSizes.assign(n, 0);
    if (Error e = allocateMoments(memoryManager, device, weightShapes, nadam->momentumBuffers,
                                  nadam->varianceBuffers, nadam->bufferSizes);
        !e.empty())
        return {nullptr, e};
    return {std::move(nadam), ""};
}

Error NadamOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    return setWeights(WeightBuffers, weightBuffers);
}

Error NadamOptimizerState::Step(const std::vector<Pointer> &gradientBuffers)
{
    if (Error e = checkGradients(gradientBuffers, WeightBuffers); !e.empty()) return e;
    currentStep++;
    // nadam.go:189-222: the pooled and non-pooled branches make the same call
    Error err = cgo_bridge::ExecuteNadamStepMPSGraph(device, WeightBuffers, gradientBuffers, momentumBuffers,
                                                     varianceBuffers, bufferSizes, config.LearningRate,
                                                     config.Beta1, config.Beta2, config.Epsilon, config.WeightDecay,
                                                     (int)currentStep);
    if (!err.empty()) return Errorf("Nadam step execution failed: %s", err.c_str());
    return "";
}

void NadamOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = (pool != nullptr);
}

std::map<std::string, ParamValue> NadamOptimizerState::GetStats()
{
    return {{"step", currentStep},        {"learning_rate", config.LearningRate}, {"beta1", config.Beta1},
            {"beta2", config.Beta2},      {"epsilon", config.Epsilon},            {"weight_decay", config.WeightDecay}};
}

void NadamOptimizerState::Cleanup()
{
    releaseAll(memoryManager, momentumBuffers);
    releaseAll(memoryManager, varianceBuffers);
    momentumBuffers.clear();
    varianceBuffers.clear();
    WeightBuffers.clear();
    bufferSizes.clear();
}

StateResult NadamOptimizerState::GetState()
{
    auto st = std::make_unique<OptimizerState>();
    if (Error e = readBuffers(momentumBuffers, bufferSizes, "momentum", "momentum", "momentum", st->StateData); !e.empty())
        return {nullptr, e};
    if (Error e = readBuffers(varianceBuffers, bufferSizes, "variance", "variance", "variance", st->StateData); !e.empty())
        return {nullptr, e};
    st->Type = "Nadam";
    st->Parameters = {{"learning_rate", config.LearningRate}, {"beta1", config.Beta1},
                      {"beta2", config.Beta2},                {"epsilon", config.Epsilon},
                      {"weight_decay", config.WeightDecay},   {"step_count", currentStep}};
    return {std::move(st), ""};
}

Error NadamOptimizerState::LoadState(const OptimizerState *state)
{
    if (Error e = validateStateType("Nadam", state); !e.empty()) return e;
    setFloat(state->Parameters, "learning_rate", config.LearningRate);
    setFloat(state->Parameters, "beta1", config.Beta1);
    setFloat(state->Parameters, "beta2", config.Beta2);
    setFloat(state->Parameters, "epsilon", config.Epsilon);
    setFloat(state->Parameters, "weight_decay", config.WeightDecay);
    loadStepCountLenient(state->Parameters, currentStep);
    for (const OptimizerTensor &tensor : state->StateData) {
        int idx;
        if (Error e = checkTensor(tensor, bufferSizes, idx); !e.empty()) return e;
        Error e;
        if (tensor.StateType == "momentum") e = writeBuffer(momentumBuffers[idx], tensor, idx, "momentum");
        else if (tensor.StateType == "variance") e = writeBuffer(varianceBuffers[idx], tensor, idx, "variance");
        else e = Errorf("unknown state type: %s", tensor.StateType.c_str());
        if (!e.empty()) return e;
    }
    return "";
}

}  // namespace optimizer
}  // namespace gometal
