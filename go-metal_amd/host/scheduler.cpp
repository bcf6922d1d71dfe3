// Host-side mirror of training/scheduler.go.
#include "scheduler.hpp"

#include <cmath>

namespace gometal {
namespace training {

StepLRScheduler::StepLRScheduler(int stepSize, double gamma)
{
    if (stepSize <= 0) stepSize = 30;               // default: reduce every 30 epochs
    if (gamma <= 0 || gamma >= 1) gamma = 0.1;      // default: reduce by 10x
    StepSize = stepSize;
    Gamma = gamma;
}

double StepLRScheduler::GetLR(int epoch, int, double baseLR)
{
    const int times = epoch / StepSize;
    return baseLR * std::pow(Gamma, (double)times);
}

ExponentialLRScheduler::ExponentialLRScheduler(double gamma)
{
    if (gamma <= 0 || gamma >= 1) gamma = 0.95;     // default: 5 % reduction per epoch
    Gamma = gamma;
}

double ExponentialLRScheduler::GetLR(int epoch, int, double baseLR) { return baseLR * std::pow(Gamma, (double)epoch); }

CosineAnnealingLRScheduler::CosineAnnealingLRScheduler(int tMax, double etaMin)
{
    if (tMax <= 0) tMax = 100;
    if (etaMin < 0) etaMin = 0;
    TMax = tMax;
    EtaMin = etaMin;
}

double CosineAnnealingLRScheduler::GetLR(int epoch, int, double baseLR)
{
    if (epoch >= TMax) return EtaMin;
    const double pi = 3.14159265358979323846264338327950288;
    return EtaMin + (baseLR - EtaMin) * (1 + std::cos(pi * (double)epoch / (double)TMax)) / 2;
}

ReduceLROnPlateauScheduler::ReduceLROnPlateauScheduler(double factor, int patience, double threshold,
                                                       const std::string &mode)
{
    if (factor <= 0 || factor >= 1) factor = 0.1;
    if (patience <= 0) patience = 10;
    if (threshold < 0) threshold = 1e-4;
    Factor = factor;
    Patience = patience;
    Threshold = threshold;
    Mode = (mode != "min" && mode != "max") ? "min" : mode;
}

double ReduceLROnPlateauScheduler::Step(double metric, double lr)
{
    if (!initialized) {
        bestMetric = metric;
        currentLR = lr;
        initialized = true;
        return lr;
    }
    const bool improved = (Mode == "min") ? metric < bestMetric - Threshold : metric > bestMetric + Threshold;
    if (improved) {
        bestMetric = metric;
        badEpochs = 0;
    } else {
        badEpochs++;
        if (badEpochs >= Patience) {
            currentLR *= Factor;
            badEpochs = 0;
        }
    }
    return currentLR;
}

double ReduceLROnPlateauScheduler::GetLR(int, int, double baseLR) { return initialized ? currentLR : baseLR; }

}  // namespace training
}  // namespace gometal
