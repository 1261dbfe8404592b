// seann::Linear — the dense operand calling the seblas path (seann/operands/seblas/Linear.cuh:14-73,
// Linear.cu:8-60). The input is flattened to (N, 1, IN, 1); weights are stored OUT x IN.
#pragma once
#include "OperandBase.h"

#define OPR_SEBLAS_LINEAR 0x0001

namespace seann {

class Linear : public OperandBase {
public:
    NetParam *weights{};
    NetParam *biases{};
    uint32 INPUT_SIZE{};
    uint32 OUTPUT_SIZE;
    OperandBase *fusedRelu = nullptr;  // the ReLU behind this operand whose passes it computes (absorbReLU)

    explicit Linear(uint32 OUTPUT_SIZE) : OUTPUT_SIZE(OUTPUT_SIZE) {}

    std::string info() override {
        return "Linear        { " + std::to_string(INPUT_SIZE) + ", " + std::to_string(OUTPUT_SIZE) + " }";
    }

    void initNetParams(OptimizerInfo *info, shape4 inShape) override;
    void forward() override;
    void paramGrads() override;
    void xGrads() override;
    void randFillNetParams() override;
    void zeroGrads() override;
    void updateParams() override {  // Linear.cu:25-28
        weights->update();
        biases->update();
    }
    void batchUpdateParams() override {
        weights->batchUpdate();
        biases->batchUpdate();
    }
    void collectNetParams(std::vector<NetParam *> &out) override {
        out.push_back(weights);
        out.push_back(biases);
    }
    // forward writes max(., 0) straight into the ReLU's output; xGrads masks the ReLU's output gradient by that output
    bool absorbReLU(OperandBase *relu) override {
        fusedRelu = relu;
        return true;
    }
    uint32 OPERAND_ID() override { return OPR_SEBLAS_LINEAR; }
    // info: OUTPUT_SIZE; params: weights, then biases (Linear.cu:62-75)
    uint32 encodeInfo(std::fstream *fout, uint64 offset) override;
    uint32 encodeNetParams(std::fstream *fout, uint64 offset) override;
    uint32 getInfoEncodingSize() override { return sizeof(uint32); }
    uint32 getNetParamsEncodingSize() override {
        return uint32(sizeof(float) * (weights->data()->dims.size + biases->data()->dims.size));
    }
};
}  // namespace seann
