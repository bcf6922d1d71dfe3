// Host-side mirror of training/scheduler.go: learning-rate schedules.  Pure host arithmetic
// in float64, as in the reference; the result reaches the kernels through
// Optimizer::UpdateLearningRate, and because the learning rate is a kernel argument (not a
// device constant) a schedule costs nothing per step.
#pragma once

#include <memory>
#include <string>

namespace gometal {
namespace training {

// training/scheduler.go:9-16
class LRScheduler {
public:
    virtual ~LRScheduler() = default;
    virtual double GetLR(int epoch, int step, double baseLR) = 0;
    virtual std::string GetName() = 0;
};

// training/scheduler.go:19-46
struct StepLRScheduler : LRScheduler {
    int StepSize;
    double Gamma;
    StepLRScheduler(int stepSize, double gamma);
    double GetLR(int epoch, int step, double baseLR) override;
    std::string GetName() override { return "StepLR"; }
};

// training/scheduler.go:49-69
struct ExponentialLRScheduler : LRScheduler {
    double Gamma;
    explicit ExponentialLRScheduler(double gamma);
    double GetLR(int epoch, int step, double baseLR) override;
    std::string GetName() override { return "ExponentialLR"; }
};

// training/scheduler.go:72-102
struct CosineAnnealingLRScheduler : LRScheduler {
    int TMax;
    double EtaMin;
    CosineAnnealingLRScheduler(int tMax, double etaMin);
    double GetLR(int epoch, int step, double baseLR) override;
    std::string GetName() override { return "CosineAnnealingLR"; }
};

// training/scheduler.go:105-184
struct ReduceLROnPlateauScheduler : LRScheduler {
    double Factor;
    int Patience;
    double Threshold;
    std::string Mode;
    ReduceLROnPlateauScheduler(double factor, int patience, double threshold, const std::string &mode);
    double Step(double metric, double currentLR);   // once per epoch with the validation metric
    double GetLR(int epoch, int step, double baseLR) override;
    std::string GetName() override { return "ReduceLROnPlateau"; }

private:
    double bestMetric = 0;
    int badEpochs = 0;
    double currentLR = 0;
    bool initialized = false;
};

// training/scheduler.go:187-195
struct NoOpScheduler : LRScheduler {
    double GetLR(int, int, double baseLR) override { return baseLR; }
    std::string GetName() override { return "ConstantLR"; }
};

}  // namespace training
}  // namespace gometal
