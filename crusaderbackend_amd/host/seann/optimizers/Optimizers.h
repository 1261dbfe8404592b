// seann optimizers: the Optimizer interface, the Momentum optimizer and the OptimizerInfo factories that hand one
// optimizer to every trainable parameter (seann/optimizers/Optimizers.cuh:24-37,52-69,171-195; Optimizers.cu:16-26).
// Only momentum (and plain SGD as its beta = 0 case) is built; AdaGrad / AdaDelta / Adam are not.
#pragma once
#include "../../seblas/operations/operations.h"

namespace seann {
using namespace seblas;

struct Optimizer {
    float LEARNING_RATE;
    Parameter *A;
    float L2 = 0.0001f;  // weight decay applied to weights only (Optimizers.cuh:28, Optimizers.cu:17-19)
    bool isWeight = false;
    Optimizer(float LEARNING_RATE, Parameter *A) : LEARNING_RATE(LEARNING_RATE), A(A) {}
    virtual ~Optimizer() = default;
    virtual void apply() = 0;       // per-sample update
    virtual void batchApply() = 0;  // per-batch update
    virtual void zeroGrad() = 0;
};

// m = beta*m + (1-beta)*g;  w = w*(1 - L2 if weight) - lr*m;  g = 0 — decay and step in one kernel launch.
struct Momentum : public Optimizer {
    float BETA = 0.9f;
    Tensor *m;
    Momentum(float LEARNING_RATE, Parameter *A) : Optimizer(LEARNING_RATE, A) { m = Tensor::create(A->dA->dims); }
    Momentum(float LEARNING_RATE, Parameter *A, float BETA) : Momentum(LEARNING_RATE, A) { this->BETA = BETA; }
    void apply() override { momentumApplyDecay(A->A, A->dA, m, LEARNING_RATE, BETA, isWeight ? L2 : 0.0f); }
    void batchApply() override {}
    void zeroGrad() override { m->constFill(0); }
};

struct OptimizerInfo {
    virtual ~OptimizerInfo() = default;
    virtual Optimizer *create(Parameter *A) = 0;
};

struct OPTIMIZER_MOMENTUM : public OptimizerInfo {
    float LEARNING_RATE;
    float BETA = 0.9f;
    OPTIMIZER_MOMENTUM(float LEARNING_RATE, float BETA) : LEARNING_RATE(LEARNING_RATE), BETA(BETA) {}
    explicit OPTIMIZER_MOMENTUM(float LEARNING_RATE) : LEARNING_RATE(LEARNING_RATE) {}
    Optimizer *create(Parameter *A) override { return new Momentum(LEARNING_RATE, A, BETA); }
};
}  // namespace seann
