// seann::ShortcutEndpoint — the pair of markers that delimit a residual connection in a Sequential
// (seann/operands/controlling/ShortcutEndpoint.{cuh,cu}). The opening endpoint (isContainer = false) forwards its input
// unchanged; the closing endpoint (isContainer = true, same uuid) adds to the main path either the opening endpoint's
// output (identity shortcut) or the output of its own branch operands applied to it (projection shortcut). Backward, the
// closing endpoint hands its output gradient to the branch (or, for the identity, to the opening endpoint's reserve
// gradient), and the opening endpoint folds that reserve into the gradient it passes further back.
#pragma once
#include <initializer_list>
#include <vector>

#include "OperandBase.h"

#define OPR_CTRL_SHORTCUTENDPOINT_BEG 0xf002
#define OPR_CTRL_SHORTCUTENDPOINT_END 0xf003

namespace seann {

class ShortcutEndpoint : public OperandBase {
public:
    bool isContainer;
    ShortcutEndpoint *other{};
    std::vector<OperandBase *> branchOperands;
    uint32 operandCount = 0;
    uint32 uuid;
    OperandBase *fusedRelu = nullptr;  // closing endpoint: the ReLU behind it whose passes it computes (absorbReLU)
    Tensor *gradPartA = nullptr, *gradPartB = nullptr;  // takeGradientInParts
    // Set by Sequential::streamline(): this endpoint's passes are computed by a neighbour — a closing identity endpoint's by
    // the batch normalisation in front of it, an opening endpoint's gradient sum by the operand that absorbed the ReLU in
    // front of it — and forward / xGrads do nothing.
    bool idleForward = false, idleGrad = false;
    bool absorbReLU(OperandBase *relu) override {
        if (!isContainer) return false;
        fusedRelu = relu;
        return true;
    }
    bool takeGradientInParts(Tensor *a, Tensor *b) override {
        if (!isContainer || !fusedRelu) return false;
        gradPartA = a, gradPartB = b;
        return true;
    }

    ShortcutEndpoint(bool isContainer, uint32 uuid, std::initializer_list<OperandBase *> operands)
        : isContainer(isContainer), uuid(uuid) {
        if (isContainer) branchOperands.assign(operands.begin(), operands.end());
        operandCount = uint32(branchOperands.size());
    }
    ShortcutEndpoint(bool isContainer, uint32 uuid, const std::vector<OperandBase *> &operands) : isContainer(isContainer), uuid(uuid) {
        if (isContainer) branchOperands = operands;
        operandCount = uint32(branchOperands.size());
    }
    ShortcutEndpoint(bool isContainer, uint32 uuid, OperandBase **operands, uint32 operandCount)
        : ShortcutEndpoint(isContainer, uuid, std::vector<OperandBase *>(operands, operands + operandCount)) {}

    // Set once the branch operands own their tensors (a model file's decoder creates and fills them before the chain is
    // bound); postWaiveInit then binds them without creating them again.
    bool branchInitialised = false;

    void initNetParams(OptimizerInfo *info, shape4 inShape) override;
    void postWaiveInit(OptimizerInfo *info) override;
    void forward() override;
    void xGrads() override;
    void paramGrads() override;
    void updateParams() override;
    void batchUpdateParams() override;
    void randFillNetParams() override;
    void zeroGrads() override;
    void collectNetParams(std::vector<NetParam *> &out) override {
        for (OperandBase *op : branchOperands) op->collectNetParams(out);
    }
    void pruneReserveFolds() override {
        OperandBase::pruneReserveFolds();
        for (OperandBase *op : branchOperands) op->pruneReserveFolds();
    }
    void fuseGrads() override {
        for (OperandBase *op : branchOperands) op->fuseGrads();
    }
    void deferSliceSum(std::vector<seblas::SliceSumItem> &items) override {
        for (OperandBase *op : branchOperands) op->deferSliceSum(items);
    }
    std::string info() override { return "ShortcutEndpoint { " + std::to_string(operandCount) + " }"; }
    uint32 OPERAND_ID() override { return isContainer ? OPR_CTRL_SHORTCUTENDPOINT_END : OPR_CTRL_SHORTCUTENDPOINT_BEG; }
    // info: uuid, branch operand count, then for a closing endpoint the branch's type ids and infos; params: the branch's
    // (ShortcutEndpoint.cu:151-177)
    uint32 encodeInfo(std::fstream *fout, uint64 offset) override;
    uint32 encodeNetParams(std::fstream *fout, uint64 offset) override;
    uint32 getInfoEncodingSize() override;
    uint32 getNetParamsEncodingSize() override;
};
}  // namespace seann
