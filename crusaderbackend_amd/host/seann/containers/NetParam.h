// seann::NetParam — a trainable Parameter (weights or biases) paired with its optimizer, as the operands hold it
// (seann/containers/NetParam.cuh:20-56). `info` may be null (no optimizer: update() is then a no-op), which is how
// the operands are used when only forward / gradients are wanted. The encode / decode members move the tensor between
// device memory and a model file (NetParam.cuh:45-102) with one device copy per tensor instead of one per 400 values.
#pragma once
#include <fstream>

#include "../optimizers/Optimizers.h"

namespace seann {
using namespace seblas;

class NetParam {
public:
    Parameter *A = nullptr;
    Optimizer *opt = nullptr;
    bool isWeight = false;

    template <typename... Args>
    explicit NetParam(OptimizerInfo *info, Args &&...args) {
        A = Parameter::create(std::forward<Args>(args)...);
        if (info) opt = info->create(A);
    }
    NetParam(Parameter *A, Optimizer *opt) : A(A), opt(opt) {}
    NetParam(Parameter *A, OptimizerInfo *info) : A(A) { opt = info ? info->create(A) : nullptr; }

    NetParam *setWeight() {
        isWeight = true;
        if (opt) opt->isWeight = true;
        return this;
    }
    void setWeightDecay(float weightDecay) const {
        if (opt) opt->L2 = weightDecay;
    }
    void update() const {
        if (opt) opt->apply();
    }
    void batchUpdate() const {
        if (opt) opt->batchApply();
    }
    uint32 encodeNetParamInfo(std::fstream *fout, uint64 offset) const;  // dims n, c, h, w: 16 bytes
    uint32 encodeNetParamData(std::fstream *fout, uint64 offset) const;  // raw float32 values
    static NetParam *decodeNetParamInfo(std::fstream *fin, uint64 &offset, OptimizerInfo *info);
    static NetParam *decodeNetParamData(std::fstream *fin, uint64 &offset, NetParam *param);
    Tensor *data() const { return A->A; }
    Tensor *grad() const { return A->dA; }
    void zeroGrad() const { A->dA->constFill(0); }
};
}  // namespace seann
