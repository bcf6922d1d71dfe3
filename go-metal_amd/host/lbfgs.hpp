// Host-side mirror of optimizer/lbfgs.go: the L-BFGS state object (ring of s / y history
// tensors, one rho buffer per slot, alpha buffer, previous gradients, search direction) that
// drives execute_lbfgs_step_mpsgraph.  Names, allocation order, validation order and error
// strings follow the Go source.  Like the Go type it is not an optimizer.Optimizer: Step
// also takes the current loss.
#pragma once

#include "optimizer.hpp"

namespace gometal {
namespace optimizer {

// optimizer/lbfgs.go:45-64
struct LBFGSConfig {
    int HistorySize;
    float LineSearchTol;
    int MaxLineSearch;
    float C1, C2, InitialStep;
};
LBFGSConfig DefaultLBFGSConfig();

// optimizer/lbfgs.go:12-42
class LBFGSOptimizerState {
public:
    std::vector<Pointer> WeightBuffers;

    Error SetWeightBuffers(const std::vector<Pointer> &weightBuffers);              // lbfgs.go:235
    Error Step(const std::vector<Pointer> &gradientBuffers, float currentLoss);     // lbfgs.go:245
    void SetCommandPool(Pointer pool);                                              // lbfgs.go:304
    uint64_t GetStep() const { return currentStep; }                                // lbfgs.go:310
    std::map<std::string, ParamValue> GetStats() const;                             // lbfgs.go:315
    void Cleanup() { cleanup(); }                                                   // lbfgs.go:325
    Error UpdateLearningRate(float newLR);                                          // lbfgs.go:330

    LBFGSConfig config{};
    std::vector<std::vector<Pointer>> sVectors, yVectors;    // [HistorySize][numWeights]
    std::vector<Pointer> rhoBuffers;                         // one 4-byte buffer per history slot
    Pointer alphaBuffer = nullptr;
    std::vector<Pointer> oldGradients, searchDir;
    uint64_t currentStep = 0;
    int historyCount = 0, historyIndex = 0;
    memory::MemoryManager *memoryManager = nullptr;
    Pointer device = nullptr;
    std::vector<int> bufferSizes;
    Pointer commandPool = nullptr;
    bool usePooling = false;
    float prevLoss = 0, prevGradNorm = 0;
    float lastStepSize = 0;      // what the native step reported (the Go code only prints it)
    bool logProgress = true;     // the Go Step prints a line every 10 steps (lbfgs.go:295-298)

private:
    void cleanup();
};

// optimizer/lbfgs.go:67-193
std::pair<std::unique_ptr<LBFGSOptimizerState>, Error> NewLBFGSOptimizer(const LBFGSConfig &config,
                                                                         const Shapes &weightShapes,
                                                                         memory::MemoryManager *memoryManager,
                                                                         Pointer device);

}  // namespace optimizer
}  // namespace gometal
