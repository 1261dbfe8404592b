// seann::NetParam — a trainable Parameter (weights or biases) as the conv/linear operands hold it
// (seann/containers/NetParam.cuh:20-116). The reference pairs it with an Optimizer; optimizers are outside
// this build, so `opt` is an opaque pointer that the operands pass through untouched, and the gradient
// zeroing the reference's optimizers perform after every apply (seblas/operations/cuOptim.cu:65-71) is
// available as zeroGrad().
#pragma once
#include "../../seblas/tensor/Parameter.h"

namespace seann {
using namespace seblas;

struct Optimizer;      // not part of this build
struct OptimizerInfo;  // not part of this build

class NetParam {
public:
    Parameter *A = nullptr;
    Optimizer *opt = nullptr;
    bool isWeight = false;

    template <typename... Args>
    explicit NetParam(OptimizerInfo *, Args &&...args) { A = Parameter::create(std::forward<Args>(args)...); }
    NetParam(Parameter *A, Optimizer *opt) : A(A), opt(opt) {}

    NetParam *setWeight() {
        isWeight = true;
        return this;
    }
    Tensor *data() const { return A->A; }
    Tensor *grad() const { return A->dA; }
    void zeroGrad() const { A->dA->constFill(0); }
};
}  // namespace seann
