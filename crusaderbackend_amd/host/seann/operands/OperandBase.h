// seann::OperandBase — the operand plugin interface of the reference (seann/operands/OperandBase.cuh:16-108):
// forward / xGrads / paramGrads, parameter initialisation, optimizer application, graph wiring and the operand's records
// in a model file.
#pragma once
#include <fstream>
#include <string>
#include <vector>

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
    // Operands that deposit a gradient in this operand's Y->dAReserve (shortcut endpoints) count themselves here;
    // pruneReserveFolds() switches the fold off where nobody does. Until it is called every operand folds, as in the reference.
    uint32 reserveWriters = 0;
    bool foldReserveEnabled = true;

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

    // Model-file records (OperandBase.cuh:102-108): the construction arguments ("info") and the trainable tensors
    // ("net params") written at byte `offset` of the stream; each returns the number of bytes it wrote. Operands without
    // arguments or parameters write nothing.
    virtual uint32 encodeInfo(std::fstream *, uint64) { return 0; }
    virtual uint32 encodeNetParams(std::fstream *, uint64) { return 0; }
    virtual uint32 getInfoEncodingSize() { return 0; }
    virtual uint32 getNetParamsEncodingSize() { return 0; }

    virtual void collectNetParams(std::vector<NetParam *> &) {}  // every trainable parameter, for a fused update
    virtual void pruneReserveFolds() { foldReserveEnabled = reserveWriters > 0; }
    // Lets xGrads also produce the parameter gradients where one launch can compute both; the paramGrads call that follows
    // it in Sequential::backward then finds them done. Only for callers that always pair the two calls (Sequential does).
    virtual void fuseGrads() {}
    // Lets xGrads leave the parameter gradient as partial sums and adds what completes them to `items`; the caller sums all
    // items in one launch after the last xGrads of a backward pass (Sequential::backward does, once streamline() was
    // called). An operand that has added an item must from then on be driven that way.
    virtual void deferSliceSum(std::vector<seblas::SliceSumItem> &) {}
    // Asked of an operand whose successor in the chain is a ReLU: take over that ReLU's work (write its output in the same
    // pass as your own, apply its gradient rule in your xGrads) and return true, or return false. The ReLU is then told
    // to do nothing. Only Sequential::streamline() asks.
    virtual bool absorbReLU(OperandBase *) { return false; }
    // Asked of an operand that has absorbed a ReLU behind which a residual connection opens: from now on the gradient with
    // respect to that ReLU's output arrives in two parts (the opening endpoint's main-path and shortcut gradients), which
    // the operand adds on the fly; the opening endpoint then has nothing left to do in xGrads. False = not supported.
    virtual bool takeGradientInParts(Tensor *, Tensor *) { return false; }

    // Y->dA += Y->dAReserve and the reserve is cleared, in one pass (the reference clears it after the gradient call, which
    // never reads it): the first thing every xGrads does
    void foldReserve() const {
        if (foldReserveEnabled) Y->dA->addAndClear(Y->dAReserve);
    }

    void bindPrev(OperandBase *p) { prev = p; }
    void bindNext(OperandBase *n) { next = n; }
    void bindInput(Parameter *prevY) const { X->inherit(prevY); }
    OperandBase *tracePrev() const { return prev; }
    OperandBase *traceNext() const { return next; }
    OperandBase *tracePrev(uint32 ago) { return ago == 0 ? this : prev->tracePrev(ago - 1); }
    OperandBase *traceNext(uint32 dist) { return dist == 0 ? this : next->traceNext(dist - 1); }
};
}  // namespace seann
