// seann::Conv2D — the convolution operand calling the seblas path, with the reference's members, constructor
// and method set (seann/operands/seblas/Conv2D.cuh:14-100, Conv2D.cu:8-57).
#pragma once
#include "OperandBase.h"

#define OPR_SEBLAS_CONV2D 0x0002

namespace seann {

class Conv2D : public OperandBase {
public:
    shape4 filterShape;
    NetParam *filter{};
    NetParam *bias = nullptr;
    uint32 strideH, strideW, padH, padW;
    bool WITH_BIAS = false;
    bool gradsFused = false;      // xGrads computes the filter gradient too (fuseGrads())
    bool filterGradDone = false;  // ... and has done so since the last forward / paramGrads
    Tensor *gradSlices = nullptr;  // deferSliceSum(): xGrads leaves the filter gradient here as partial sums
    OperandBase *fusedRelu = nullptr;  // the ReLU behind this operand whose passes it computes (absorbReLU)

    Conv2D(shape4 filterShape, uint32 strideH, uint32 strideW, uint32 padH, uint32 padW, bool WITH_BIAS)
        : filterShape(filterShape), strideH(strideH), strideW(strideW), padH(padH), padW(padW), WITH_BIAS(WITH_BIAS) {}

    std::string info() override {
        return "Conv2D        { filter: " + filter->data()->dims.toString() + ", input feature: " + X->A->dims.toString() + " }";
    }

    // output shape (N, OC, (H + 2p - FH)/s + 1, (W + 2p - FW)/s + 1)  — Conv2D.cuh:40-44
    void initNetParams(OptimizerInfo *info, shape4 inShape) override;
    void forward() override;
    void xGrads() override;
    void paramGrads() override;
    void randFillNetParams() override;
    void zeroGrads() override;
    void updateParams() override {  // Conv2D.cu:31-34
        filter->update();
        if (WITH_BIAS) bias->update();
    }
    void batchUpdateParams() override {
        filter->batchUpdate();
        if (WITH_BIAS) bias->batchUpdate();
    }
    void collectNetParams(std::vector<NetParam *> &out) override {
        out.push_back(filter);
        if (WITH_BIAS) out.push_back(bias);
    }
    void fuseGrads() override { gradsFused = true; }
    // forward writes max(conv, 0) straight into the ReLU's output; xGrads masks the ReLU's output gradient by that output
    // (positive exactly where the convolution's own result was) before it runs the convolution's gradients
    bool absorbReLU(OperandBase *relu) override {
        fusedRelu = relu;
        return true;
    }
    void deferSliceSum(std::vector<seblas::SliceSumItem> &items) override;
    uint32 OPERAND_ID() override { return OPR_SEBLAS_CONV2D; }
    // info: filter dims, strides, paddings, has-bias flag (36 bytes); params: filter, then bias (Conv2D.cu:59-80)
    uint32 encodeInfo(std::fstream *fout, uint64 offset) override;
    uint32 encodeNetParams(std::fstream *fout, uint64 offset) override;
    uint32 getInfoEncodingSize() override { return sizeof(uint32) * 9; }
    uint32 getNetParamsEncodingSize() override {
        return uint32((filter->data()->dims.size + (WITH_BIAS ? bias->data()->dims.size : 0)) * sizeof(float));
    }
};
}  // namespace seann
