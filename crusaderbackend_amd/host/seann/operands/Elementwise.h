// The operands of a CIFAR-style network besides convolution and dense layers: ReLU, MaxPool2D, BatchNorm, Softmax — each
// a thin call into the seblas operator of the same name, with the reference's members and gradient bookkeeping (the reserve gradient a shortcut
// may have deposited in Y->dAReserve is folded into Y->dA first and cleared afterwards).
// seann/operands/seblas/activate/ReLU.{cuh,cu}, pooling/MaxPool2D.{cuh,cu}, Softmax.{cuh,cu}.
#pragma once
#include <stdexcept>

#include "OperandBase.h"

#define OPR_SEBLAS_RELU 0xa002
#define OPR_SEBLAS_MAXPOOL2D 0xb003
#define OPR_SEBLAS_SOFTMAX 0x0005
#define OPR_SEBLAS_BATCHNORM 0x0003

namespace seann {

class ParamFreeOperand : public OperandBase {
public:
    void paramGrads() override {}
    void randFillNetParams() override {}
    void zeroGrads() override {}

};

class ReLU : public ParamFreeOperand {
public:
    uint32 INPUT_SIZE{};
    uint32 PARALELL_SIZE{};
    std::string info() override { return "ReLU          { " + std::to_string(INPUT_SIZE / PARALELL_SIZE) + " }"; }
    void initNetParams(OptimizerInfo *, shape4 inShape) override {  // ReLU.cuh:27-32
        INPUT_SIZE = inShape.size;
        PARALELL_SIZE = inShape.n;
        X = Parameter::declare(inShape);
        Y = Parameter::create(inShape);
    }
    OperandBase *absorbedBy = nullptr;  // set by Sequential::streamline(): the predecessor computes this operand's passes
    void forward() override {             // ReLU.cu:8-10
        if (!absorbedBy) relu(X->A, Y->A);
    }
    void xGrads() override {  // ReLU.cu:13-17
        foldReserve();
        if (!absorbedBy) reluGradFast(X->A, Y->dA, X->dA);
    }
    uint32 OPERAND_ID() override { return OPR_SEBLAS_RELU; }
};

class MaxPool2D : public ParamFreeOperand {
public:
    Tensor *record{};
    uint32 strideH, strideW, rangeH, rangeW;
    MaxPool2D(uint32 strideH, uint32 strideW, uint32 rangeH, uint32 rangeW)
        : strideH(strideH), strideW(strideW), rangeH(rangeH), rangeW(rangeW) {}
    std::string info() override { return "MaxPool2D     { " + X->A->dims.toString() + ", " + Y->A->dims.toString() + " }"; }
    void initNetParams(OptimizerInfo *, shape4 inShape) override {  // MaxPool2D.cuh:42-51
        X = Parameter::declare(inShape);
        Y = Parameter::create(inShape.n, inShape.c, inShape.h / strideH, inShape.w / strideW);
        record = Tensor::create(inShape.n, inShape.c, ((inShape.h - (rangeH - strideH)) / strideH) * rangeH,
                                ((inShape.w - (rangeW - strideW)) / strideW) * rangeW);
    }
    void forward() override { maxPool(X->A, Y->A, record, strideH, strideW, rangeH, rangeW); }  // MaxPool2D.cu:12-14
    void xGrads() override {                                                                     // MaxPool2D.cu:16-20
        foldReserve();
        maxPoolBack(X->dA, Y->dA, record, strideH, strideW, rangeH, rangeW);
    }
    uint32 OPERAND_ID() override { return OPR_SEBLAS_MAXPOOL2D; }
    uint32 encodeInfo(std::fstream *fout, uint64 offset) override;  // strides, ranges (MaxPool2D.cu:22-29)
    uint32 getInfoEncodingSize() override { return sizeof(uint32) * 4; }
};

// Batch normalisation with per-feature statistics and trainable beta / gamma of one sample's shape
// (seann/operands/seblas/BatchNorm.{cuh,cu}). paramGrads gives gamma the gradient of gamma and beta the gradient of beta
// (the reference passes the two tensors to batchNormParamGrads in swapped order, BatchNorm.cu:24).
class BatchNorm : public OperandBase {
public:
    NetParam *beta{};
    NetParam *gamma{};
    Tensor *mean{};
    Tensor *variance{};
    Tensor *xHatP{};
    bool paramGradsDone = false;
    OperandBase *fusedRelu = nullptr;  // the ReLU behind this operand whose passes it computes (absorbReLU)
    // Set by Sequential::streamline() when an identity shortcut closes between this operand and the absorbed ReLU: the
    // shortcut's value is added before the ReLU, and the masked gradient is copied to the shortcut's reserve gradient.
    Tensor *shortcutValue = nullptr, *shortcutGrad = nullptr;
    Tensor *gradPartA = nullptr, *gradPartB = nullptr;  // takeGradientInParts
    bool absorbReLU(OperandBase *relu) override {
        fusedRelu = relu;
        return true;
    }
    bool takeGradientInParts(Tensor *a, Tensor *b) override {
        if (!fusedRelu) return false;
        gradPartA = a, gradPartB = b;
        return true;
    }
    std::string info() override { return "BatchNorm"; }
    void initNetParams(OptimizerInfo *info, shape4 inShape) override {  // BatchNorm.cuh:27-37
        shape4 paramShape = {1, inShape.c, inShape.h, inShape.w};
        beta = new NetParam(info, paramShape);
        gamma = new NetParam(info, paramShape);
        mean = Tensor::create(paramShape);
        variance = Tensor::create(paramShape);
        xHatP = Tensor::create(inShape);
        X = Parameter::declare(inShape);
        Y = Parameter::create(inShape);
    }
    void randFillNetParams() override {  // BatchNorm.cu:8-11
        beta->data()->constFill(0.0f);
        gamma->data()->constFill(1.0f);
    }
    void forward() override {
        paramGradsDone = false;
        if (fusedRelu) {  // Y and xHat are not needed: the ReLU's output is this operand's result, xGrads recomputes from X
            batchNormRelu(X->A, beta->data(), gamma->data(), mean, variance, fusedRelu->Y->A, shortcutValue);
            return;
        }
        batchNorm(X->A, beta->data(), gamma->data(), mean, variance, Y->A, xHatP);
    }
    // xGrads also produces the parameter gradients (they fall out of the same per-feature sums); the paramGrads call
    // that follows it in Sequential::backward then has nothing left to do. Called on its own, paramGrads computes them.
    void xGrads() override {  // BatchNorm.cu:17-21
        foldReserve();
        if (fusedRelu)
            batchNormReluGradAll(gradPartA ? gradPartA : fusedRelu->Y->dA, fusedRelu->Y->A, gamma->data(), X->A, X->dA, gamma->grad(),
                                 beta->grad(), gradPartB, shortcutGrad);
        else
            batchNormGradAll(Y->dA, gamma->data(), X->A, X->dA, gamma->grad(), beta->grad());
        paramGradsDone = true;
    }
    void paramGrads() override {
        if (!paramGradsDone && fusedRelu) throw std::logic_error("BatchNorm: with an absorbed ReLU, paramGrads follows xGrads");
        if (!paramGradsDone) batchNormParamGrads(Y->dA, xHatP, gamma->grad(), beta->grad());
        paramGradsDone = false;
    }
    void updateParams() override {
        beta->update();
        gamma->update();
    }
    void batchUpdateParams() override {
        beta->batchUpdate();
        gamma->batchUpdate();
    }
    void zeroGrads() override {
        beta->zeroGrad();
        gamma->zeroGrad();
    }
    void collectNetParams(std::vector<NetParam *> &out) override {
        out.push_back(beta);
        out.push_back(gamma);
    }
    uint32 OPERAND_ID() override { return OPR_SEBLAS_BATCHNORM; }
    uint32 encodeNetParams(std::fstream *fout, uint64 offset) override;  // beta, then gamma (BatchNorm.cu:50-55)
    uint32 getNetParamsEncodingSize() override {
        return uint32(sizeof(float) * (beta->data()->dims.size + gamma->data()->dims.size));
    }
};

// Output probabilities; the loss function writes Y->dA = Y->A - labels, which is already the gradient with respect to
// the softmax input, so xGrads only passes it on (Softmax.cu:12-18).
class Softmax : public ParamFreeOperand {
public:
    std::string info() override { return "Softmax       { " + std::to_string(Y->A->dims.size / Y->A->dims.n) + " }"; }
    void initNetParams(OptimizerInfo *, shape4 inShape) override {
        X = Parameter::declare(inShape);
        Y = Parameter::create(inShape);
    }
    void forward() override { softmax(X->A, Y->A, nullptr, Y->A->dims.size / Y->A->dims.n); }  // Softmax.cu:8-10
    void xGrads() override {
        foldReserve();
        Y->dA->copyToD2D(X->dA);
    }
    uint32 OPERAND_ID() override { return OPR_SEBLAS_SOFTMAX; }
};
}  // namespace seann
