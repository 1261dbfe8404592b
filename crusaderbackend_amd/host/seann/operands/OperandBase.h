// seann::OperandBase — the operand plugin interface of the reference (seann/operands/OperandBase.cuh:16-108):
// forward / xGrads / paramGrads, parameter initialisation, optimizer application and graph wiring. Checkpoint
// encoding is outside this build.
#pragma once
#include <string>

#include "../../seblas/operations/operations.h"
#include "../containers/NetParam.h"

namespace seann {

class OperandBase {
public:
    Parameter *X = nullptr;  // input: a shadow of the previous operand's output
    Parameter *Y = nullptr;  // output
    OperandBase *prev = nullptr;
    OperandBase *next = nullptr;
    uint32 operandID = 0;

    virtual ~OperandBase() = default;

    virtual void forward() = 0;     // X -> Y
    virtual void paramGrads() = 0;  // gradients of weights / biases
    virtual void xGrads() = 0;      // gradient of the input
    virtual void updateParams() {}
    virtual void batchUpdateParams() {}
    virtual void initNetParams(OptimizerInfo *info, shape4 inShape) = 0;
    virtual void randFillNetParams() = 0;
    virtual void postWaiveInit(OptimizerInfo *) {}  // second construction pass, after the chain is bound
    virtual void inferenceForward() { forward(); }
    virtual void zeroGrads() = 0;
    virtual std::string info() = 0;
    virtual uint32 OPERAND_ID() { return 0x0000; }

    void bindPrev(OperandBase *p) { prev = p; }
    void bindNext(OperandBase *n) { next = n; }
    void bindInput(Parameter *prevY) const { X->inherit(prevY); }
    OperandBase *tracePrev() const { return prev; }
    OperandBase *traceNext() const { return next; }
    OperandBase *tracePrev(uint32 ago) { return ago == 0 ? this : prev->tracePrev(ago - 1); }
    OperandBase *traceNext(uint32 dist) { return dist == 0 ? this : next->traceNext(dist - 1); }
};
}  // namespace seann
