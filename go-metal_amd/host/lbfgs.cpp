// optimizer/lbfgs.go on the HIP bridge.
#include "lbfgs.hpp"

#include <cstdio>

namespace gometal {
namespace optimizer {

LBFGSConfig DefaultLBFGSConfig() { return LBFGSConfig{10, 1e-4f, 20, 1e-4f, 0.9f, 1.0f}; }

std::pair<std::unique_ptr<LBFGSOptimizerState>, Error> NewLBFGSOptimizer(const LBFGSConfig &config,
                                                                         const Shapes &weightShapes,
                                                                         memory::MemoryManager *memoryManager,
                                                                         Pointer device)
{
    if (memoryManager == nullptr) return {nullptr, Errorf("memory manager cannot be nil")};
    if (device == nullptr) return {nullptr, Errorf("device cannot be nil")};
    if (weightShapes.empty()) return {nullptr, Errorf("no weight shapes provided")};
    if (config.HistorySize <= 0)
        return {nullptr, Errorf("history size must be positive, got %d", config.HistorySize)};

    const size_t n = weightShapes.size();
    const int m = config.HistorySize;
    auto l = std::make_unique<LBFGSOptimizerState>();
    l->config = config;
    l->sVectors.assign((size_t)m, {});
    l->yVectors.assign((size_t)m, {});
    l->rhoBuffers.assign((size_t)m, nullptr);
    l->oldGradients.assign(n, nullptr);
    l->searchDir.assign(n, nullptr);
    l->WeightBuffers.assign(n, nullptr);
    l->memoryManager = memoryManager;
    l->device = device;
    l->bufferSizes.assign(n, 0);
    for (size_t i = 0; i < n; i++) l->bufferSizes[i] = calculateTensorSize(weightShapes[i]) * 4;

    auto fail = [&](Error e) {
        l->Cleanup();
        return std::pair<std::unique_ptr<LBFGSOptimizerState>, Error>{nullptr, std::move(e)};
    };
    auto zero = [&](Pointer b, int size) { return cgo_bridge::ZeroMetalBuffer(device, b, size); };

    for (int h = 0; h < m; h++) {
        l->sVectors[h].assign(n, nullptr);
        l->yVectors[h].assign(n, nullptr);
        for (size_t i = 0; i < n; i++) {
            const int size = l->bufferSizes[i];
            Pointer s = memoryManager->AllocateBuffer(size);
            if (s == nullptr)
                return fail(Errorf("failed to allocate s vector buffer for history %d, weight %d", h, (int)i));
            l->sVectors[h][i] = s;
            Pointer y = memoryManager->AllocateBuffer(size);
            if (y == nullptr)
                return fail(Errorf("failed to allocate y vector buffer for history %d, weight %d", h, (int)i));
            l->yVectors[h][i] = y;
            if (Error e = zero(s, size); !e.empty()) return fail(Errorf("failed to zero s buffer: %s", e.c_str()));
            if (Error e = zero(y, size); !e.empty()) return fail(Errorf("failed to zero y buffer: %s", e.c_str()));
        }
        Pointer rho = memoryManager->AllocateBuffer(4);
        if (rho == nullptr) return fail(Errorf("failed to allocate rho buffer for history %d", h));
        l->rhoBuffers[h] = rho;
        // The Go constructor leaves rho as allocated (a fresh Metal buffer reads as zeros; a
        // pooled one keeps its last contents).  Cleared here so that a recycled buffer cannot
        // smuggle a stale value into the first recursion.
        if (Error e = zero(rho, 4); !e.empty()) return fail(Errorf("failed to zero rho buffer: %s", e.c_str()));
    }

    const int alphaSize = m * 4;
    l->alphaBuffer = memoryManager->AllocateBuffer(alphaSize);
    if (l->alphaBuffer == nullptr) return fail(Errorf("failed to allocate alpha buffer"));
    if (Error e = zero(l->alphaBuffer, alphaSize); !e.empty())
        return fail(Errorf("failed to zero alpha buffer: %s", e.c_str()));

    for (size_t i = 0; i < n; i++) {
        const int size = l->bufferSizes[i];
        Pointer og = memoryManager->AllocateBuffer(size);
        if (og == nullptr) return fail(Errorf("failed to allocate old gradient buffer for weight %d", (int)i));
        l->oldGradients[i] = og;
        Pointer sd = memoryManager->AllocateBuffer(size);
        if (sd == nullptr) return fail(Errorf("failed to allocate search direction buffer for weight %d", (int)i));
        l->searchDir[i] = sd;
        if (Error e = zero(og, size); !e.empty())
            return fail(Errorf("failed to zero old gradient buffer: %s", e.c_str()));
        if (Error e = zero(sd, size); !e.empty())
            return fail(Errorf("failed to zero search direction buffer: %s", e.c_str()));
    }
    return {std::move(l), ""};
}

void LBFGSOptimizerState::cleanup()
{
    if (memoryManager == nullptr) return;
    auto release = [&](Pointer &b) {
        if (b != nullptr) memoryManager->ReleaseBuffer(b);
        b = nullptr;      // a second Cleanup releases nothing (the Go version would release twice)
    };
    for (auto &h : sVectors)
        for (auto &b : h) release(b);
    for (auto &h : yVectors)
        for (auto &b : h) release(b);
    for (auto &b : rhoBuffers) release(b);
    release(alphaBuffer);
    for (auto &b : oldGradients) release(b);
    for (auto &b : searchDir) release(b);
}

Error LBFGSOptimizerState::SetWeightBuffers(const std::vector<Pointer> &weightBuffers)
{
    if (weightBuffers.size() != WeightBuffers.size())
        return Errorf("expected %d weight buffers, got %d", (int)WeightBuffers.size(), (int)weightBuffers.size());
    WeightBuffers = weightBuffers;
    return "";
}

Error LBFGSOptimizerState::Step(const std::vector<Pointer> &gradientBuffers, float currentLoss)
{
    if (gradientBuffers.size() != WeightBuffers.size())
        return Errorf("gradient buffers length (%d) doesn't match weight buffers length (%d)",
                      (int)gradientBuffers.size(), (int)WeightBuffers.size());
    currentStep++;
    auto [stepSize, err] = cgo_bridge::ExecuteLBFGSStepMPSGraph(
        device, WeightBuffers, gradientBuffers, oldGradients, searchDir, sVectors, yVectors, rhoBuffers,
        alphaBuffer, (int)WeightBuffers.size(), bufferSizes, config.HistorySize, historyCount, historyIndex,
        config.InitialStep, config.C1, config.C2, config.MaxLineSearch, currentLoss, prevLoss, commandPool,
        usePooling);
    if (!err.empty()) return Errorf("L-BFGS step failed: %s", err.c_str());
    lastStepSize = stepSize;

    historyIndex = (historyIndex + 1) % config.HistorySize;
    if (historyCount < config.HistorySize) historyCount++;
    prevLoss = currentLoss;

    if (logProgress && currentStep % 10 == 0)
        std::printf("L-BFGS step %llu: loss=%.6f, step_size=%.6f, history=%d/%d\n",
                    (unsigned long long)currentStep, currentLoss, stepSize, historyCount, config.HistorySize);
    return "";
}

void LBFGSOptimizerState::SetCommandPool(Pointer pool)
{
    commandPool = pool;
    usePooling = pool != nullptr;
}

std::map<std::string, ParamValue> LBFGSOptimizerState::GetStats() const
{
    return {{"step", (uint64_t)currentStep},
            {"history_size", (uint64_t)config.HistorySize},
            {"history_used", (uint64_t)historyCount},
            {"prev_loss", prevLoss}};
}

Error LBFGSOptimizerState::UpdateLearningRate(float)
{
    return Errorf("L-BFGS does not use a fixed learning rate; it uses line search");
}

}  // namespace optimizer
}  // namespace gometal
