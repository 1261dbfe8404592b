// Conv2D and Linear operands: thin glue over the seblas operator API, in the reference's calling order.
#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstring>
#include <stdexcept>

#include "../../../../include/crusader_hip.h"
#include "../../seblas/assist/HipAssert.h"
#include "../containers/Sequential.h"
#include "Conv2D.h"
#include "Elementwise.h"
#include "Linear.h"
#include "ShortcutEndpoint.h"

namespace seann {

// ---- Conv2D (seann/operands/seblas/Conv2D.cu) ----------------------------------------------------------
void Conv2D::initNetParams(OptimizerInfo *info, shape4 inShape) {
    filter = (new NetParam(info, filterShape))->setWeight();
    if (WITH_BIAS) bias = new NetParam(info, filterShape.n, 1);
    X = Parameter::declare(inShape);
    shape4 outShape = {X->A->dims.n, filterShape.n, (inShape.h + 2 * padH - filterShape.h) / strideH + 1,
                       (inShape.w + 2 * padW - filterShape.w) / strideW + 1};
    Y = Parameter::create(outShape);
}

void Conv2D::forward() {  // Conv2D.cu:8-16
    filterGradDone = false;
    conv(filter->data(), X->A, fusedRelu ? fusedRelu->Y->A : Y->A, int(strideH), int(strideW), int(padH), int(padW),
         WITH_BIAS ? bias->data() : nullptr, fusedRelu != nullptr);
}

void Conv2D::xGrads() {  // Conv2D.cu:18-22
    foldReserve();
    if (fusedRelu) reluGradFast(fusedRelu->Y->A, fusedRelu->Y->dA, Y->dA);
    if (gradSlices) {  // both gradients in one call, the filter gradient as partial sums that the caller completes
        convBackwardSliced(filter->data(), Y->dA, X->A, X->dA, gradSlices, int(strideH), int(strideW), int(padH), int(padW));
        filterGradDone = true;
        return;
    }
    if (gradsFused) {  // both gradients in one call; paramGrads then only adds the bias gradient
        convBackward(filter->data(), Y->dA, X->A, X->dA, filter->grad(), int(strideH), int(strideW), int(padH), int(padW));
        filterGradDone = true;
        return;
    }
    convDerive(filter->data(), Y->dA, X->dA, int(strideH), int(strideW), int(padH), int(padW));
}

void Conv2D::paramGrads() {  // Conv2D.cu:24-29; the bias gradient is the per-channel sum of dY
    if (!filterGradDone) convError(Y->dA, X->A, filter->grad(), int(strideH), int(strideW), int(padH), int(padW));
    filterGradDone = false;
    if (WITH_BIAS) {
        const shape4 &d = Y->dA->dims;
        throwOnStatus(crb_conv_bias_grad(Y->dA->elements, bias->grad()->elements, d.n, d.c, d.h * d.w, nullptr), __FILE__,
                      __LINE__);
        if (isBlocking() && hipStreamSynchronize(nullptr) != hipSuccess) assertHip(__FILE__, __LINE__);
    }
}

void Conv2D::deferSliceSum(std::vector<seblas::SliceSumItem> &items) {
    if (gradSlices) return;
    const uint32 n = convBackwardSlices(filter->data(), Y->dA, X->dA, int(strideH), int(strideW), int(padH), int(padW));
    if (!n) return;  // no sliced form for this shape: xGrads keeps summing on its own
    gradSlices = Tensor::create(shape4(1, convBackwardSliceFloats(filter->data(), Y->dA, X->dA, int(strideH), int(strideW), int(padH), int(padW))));
    items.push_back(seblas::SliceSumItem{gradSlices->elements, filter->grad()->elements, filter->grad()->dims.size, n});
}

void Conv2D::randFillNetParams() {  // Conv2D.cu:45-50: N(0, sqrt(2/K)), K = IC*FH*FW; bias N(0, sqrt(2/OC))
    uint32 K = filter->data()->dims.size / filter->data()->dims.n;
    filter->data()->randNormal(0, float(std::sqrt(2.0 / float(K))), 0x5eb1a5u + operandID);
    if (WITH_BIAS) bias->data()->randNormal(0, float(std::sqrt(2.0 / float(filter->data()->dims.n))), 0xb1a5u + operandID);
}

void Conv2D::zeroGrads() {
    filter->zeroGrad();
    if (WITH_BIAS) bias->zeroGrad();
}

// ---- Linear (seann/operands/seblas/Linear.cu) ----------------------------------------------------------
void Linear::initNetParams(OptimizerInfo *info, shape4 inShape) {  // Linear.cu:8-14
    INPUT_SIZE = inShape.size / inShape.n;
    X = Parameter::declare(inShape.n, 1, INPUT_SIZE, 1);
    Y = Parameter::create(inShape.n, 1, OUTPUT_SIZE, 1);
    weights = (new NetParam(info, OUTPUT_SIZE, INPUT_SIZE))->setWeight();
    biases = new NetParam(info, OUTPUT_SIZE, 1);
}

void Linear::forward() {  // Linear.cu:17-19
    linear(X->A, weights->data(), biases->data(), fusedRelu ? fusedRelu->Y->A : Y->A, fusedRelu != nullptr);
}

void Linear::paramGrads() { linearParamGrad(Y->dA, X->A, weights->grad(), biases->grad()); }  // :21-23

void Linear::xGrads() {  // Linear.cu:35-40
    foldReserve();
    if (fusedRelu) reluGradFast(fusedRelu->Y->A, fusedRelu->Y->dA, Y->dA);
    linearXGrad(Y->dA, weights->data(), X->dA);
}

void Linear::randFillNetParams() {  // Linear.cu:42-46
    uint32 K = weights->data()->dims.w;
    weights->data()->randNormal(0, float(std::sqrt(2.0 / float(K))), 0x11ea5u + operandID);
    biases->data()->randNormal(0, float(std::sqrt(2.0 / float(biases->data()->dims.size))), 0xb1a5e5u + operandID);
}

void Linear::zeroGrads() {
    weights->zeroGrad();
    biases->zeroGrad();
}

// ---- ShortcutEndpoint (seann/operands/controlling/ShortcutEndpoint.cu) ---------------------------------------------------
void ShortcutEndpoint::initNetParams(OptimizerInfo *, shape4 inShape) {  // :8-11
    X = Parameter::declare(inShape);
    Y = Parameter::create(inShape);
}

void ShortcutEndpoint::postWaiveInit(OptimizerInfo *inf) {  // :13-55
    if (isContainer) {
        OperandBase *tracer = tracePrev();
        while (tracer && (tracer->OPERAND_ID() != OPR_CTRL_SHORTCUTENDPOINT_BEG || static_cast<ShortcutEndpoint *>(tracer)->uuid != uuid))
            tracer = tracer->tracePrev();
        if (!tracer) throw std::invalid_argument("ShortcutEndpoint: no opening endpoint with this uuid");
        other = static_cast<ShortcutEndpoint *>(tracer);
        other->reserveWriters++;  // identity: this endpoint's xGrads copies into it; projection: the branch's input gradient is it
        if (operandCount > 0) {
            if (!branchInitialised) {
                branchOperands[0]->initNetParams(inf, other->Y->A->dims);
                for (uint32 i = 1; i < operandCount; i++) branchOperands[i]->initNetParams(inf, branchOperands[i - 1]->Y->A->dims);
                branchInitialised = true;
            } else if (!(branchOperands[0]->X->A->dims == other->Y->A->dims)) {
                throw std::invalid_argument("ShortcutEndpoint: branch was created for another input shape");
            }
            if (!(branchOperands[operandCount - 1]->Y->A->dims == Y->A->dims))
                throw std::invalid_argument("ShortcutEndpoint: branch output shape differs from the main path");
            branchOperands[0]->bindPrev(other);
            branchOperands[0]->bindInput(other->Y);
            branchOperands[0]->X->dA = other->Y->dAReserve;  // the branch's input gradient lands in the reserve
            for (uint32 i = 1; i < operandCount; i++) {
                branchOperands[i]->bindPrev(branchOperands[i - 1]);
                branchOperands[i]->bindInput(branchOperands[i - 1]->Y);
            }
            for (uint32 i = 0; i < operandCount; i++) branchOperands[i]->postWaiveInit(inf);
        }
    } else {
        OperandBase *tracer = traceNext();
        while (tracer && (tracer->OPERAND_ID() != OPR_CTRL_SHORTCUTENDPOINT_END || static_cast<ShortcutEndpoint *>(tracer)->uuid != uuid))
            tracer = tracer->traceNext();
        if (!tracer) throw std::invalid_argument("ShortcutEndpoint: no closing endpoint with this uuid");
        other = static_cast<ShortcutEndpoint *>(tracer);
    }
}

static void launched(int status, const char *file, int line) {
    throwOnStatus(status, file, line);
    if (isBlocking() && hipStreamSynchronize(nullptr) != hipSuccess) assertHip(file, line);
}

void ShortcutEndpoint::forward() {  // :57-74: Y = X for the opening endpoint, Y = X + shortcut for the closing one
    const uint32 n = X->A->dims.size;
    if (idleForward) return;
    if (!isContainer) {
        if (Y->A->elements != X->A->elements) X->A->copyToD2D(Y->A);  // aliased by Sequential::streamline()
        return;
    }
    for (uint32 i = 0; i < operandCount; i++) branchOperands[i]->forward();
    Tensor *shortcut = operandCount > 0 ? branchOperands[operandCount - 1]->Y->A : other->Y->A;
    if (fusedRelu) {  // the sum goes straight through the ReLU into that operand's output
        addRelu(X->A, shortcut, fusedRelu->Y->A);
        return;
    }
    launched(crb_tensor_add(Y->A->elements, X->A->elements, shortcut->elements, n, nullptr), __FILE__, __LINE__);
}

void ShortcutEndpoint::xGrads() {  // :76-99
    const uint32 n = X->A->dims.size;
    if (idleGrad) return;
    if (isContainer && fusedRelu) {
        // the gradient behind the absorbed ReLU, masked by its output, goes to the main path and to the shortcut at once
        Tensor *second = operandCount > 0 ? branchOperands[operandCount - 1]->Y->dA : other->Y->dAReserve;
        reluGradTwice(fusedRelu->Y->A, gradPartA ? gradPartA : fusedRelu->Y->dA, X->dA, second, gradPartB);
        for (int i = int(operandCount) - 1; i >= 0; i--) branchOperands[i]->xGrads();
        return;
    }
    if (isContainer) {
        if (operandCount > 0) {
            // projection: the branch gets a copy of the gradient, as does the main path
            launched(crb_tensor_copy2(X->dA->elements, branchOperands[operandCount - 1]->Y->dA->elements, Y->dA->elements, n, nullptr),
                     __FILE__, __LINE__);
            for (int i = int(operandCount) - 1; i >= 0; i--) branchOperands[i]->xGrads();
        } else {
            // identity: the opening endpoint's reserve gets a copy of the gradient, as does the main path
            launched(crb_tensor_copy2(X->dA->elements, other->Y->dAReserve->elements, Y->dA->elements, n, nullptr), __FILE__, __LINE__);
        }
    } else if (foldReserveEnabled) {
        launched(crb_tensor_add_clear_copy(X->dA->elements, Y->dA->elements, Y->dAReserve->elements, n, nullptr), __FILE__, __LINE__);
    } else {
        Y->dA->copyToD2D(X->dA);
    }
}

void ShortcutEndpoint::paramGrads() {
    for (OperandBase *op : branchOperands) op->paramGrads();
}
void ShortcutEndpoint::updateParams() {
    for (OperandBase *op : branchOperands) op->updateParams();
}
void ShortcutEndpoint::batchUpdateParams() {
    for (OperandBase *op : branchOperands) op->batchUpdateParams();
}
void ShortcutEndpoint::randFillNetParams() {
    for (OperandBase *op : branchOperands) op->randFillNetParams();
}
void ShortcutEndpoint::zeroGrads() {
    for (OperandBase *op : branchOperands) op->zeroGrads();
}

// ---- Sequential (seann/containers/Sequential.cu:10-103) -----------------------------------------------------------------
void Sequential::waive() const {
    for (uint32 i = 1; i < OPERAND_COUNT; i++) {
        operands[i]->bindPrev(operands[i - 1]);
        operands[i]->bindInput(operands[i - 1]->Y);
    }
    for (uint32 i = 0; i + 1 < OPERAND_COUNT; i++) operands[i]->bindNext(operands[i + 1]);
}

void Sequential::construct(OptimizerInfo *info) {
    if (OPERAND_COUNT == 0) throw std::invalid_argument("Sequential: no operands");
    for (uint32 i = 0; i < OPERAND_COUNT; i++) {
        operands[i]->initNetParams(info, i == 0 ? netX->A->dims : operands[i - 1]->Y->A->dims);
        operands[i]->operandID = i;
    }
    operands[0]->X->inherit(netX);
    netY = Parameter::declare(operands[OPERAND_COUNT - 1]->Y->A->dims)->inherit(operands[OPERAND_COUNT - 1]->Y);
    waive();
    for (uint32 i = 0; i < OPERAND_COUNT; i++) operands[i]->postWaiveInit(info);
}

void Sequential::randInit() const {
    for (OperandBase *op : operands) op->randFillNetParams();
}

Tensor *Sequential::forward() const {
    for (OperandBase *op : operands) op->forward();
    return netY->A;
}

Tensor *Sequential::forward(Tensor *X) const {
    X->copyToD2D(netX->A);
    return forward();
}

Tensor *Sequential::inferenceForward() const {
    for (OperandBase *op : operands) op->inferenceForward();
    return netY->A;
}

Tensor *Sequential::inferenceForward(Tensor *X) const {
    X->copyToD2D(netX->A);
    return inferenceForward();
}

Tensor *Sequential::backward(Tensor *label) const {
    if (!loss) throw std::invalid_argument("Sequential::backward: no loss function set");
    loss(netY, label);
    for (int i = int(OPERAND_COUNT) - 1; i >= 0; i--) {
        operands[i]->xGrads();
        operands[i]->paramGrads();
    }
    if (!sliceItems.empty()) sumSlicesMulti(sliceItems.data(), uint32(sliceItems.size()));
    return netX->dA;
}

void Sequential::learn() const {
    for (OperandBase *op : operands) op->updateParams();
}

void Sequential::learnBatch() const {
    for (OperandBase *op : operands) op->batchUpdateParams();
}

void Sequential::zeroGrads() const {
    for (OperandBase *op : operands) op->zeroGrads();
}

void Sequential::pruneReserveFolds() const {
    for (OperandBase *op : operands) op->pruneReserveFolds();
}

void Sequential::streamline() const {
    pruneReserveFolds();
    for (OperandBase *op : operands) op->fuseGrads();  // backward() always calls xGrads and paramGrads as a pair
    sliceItems.clear();
    for (OperandBase *op : operands) op->deferSliceSum(sliceItems);  // ... and sums all convolutions' slices at its end
    // a ReLU behind a batch normalisation or a closing shortcut endpoint is computed by that operand, in its passes
    for (uint32 i = 0; i + 1 < OPERAND_COUNT; i++) {
        if (operands[i + 1]->OPERAND_ID() != OPR_SEBLAS_RELU) continue;
        auto *r = static_cast<ReLU *>(operands[i + 1]);
        if (!r->absorbedBy && operands[i]->absorbReLU(r)) r->absorbedBy = operands[i];
    }
    // batch normalisation, closing identity endpoint, ReLU: the normalisation also adds the shortcut's value and hands the
    // shortcut its gradient, and the endpoint is idle
    for (uint32 i = 0; i + 2 < OPERAND_COUNT; i++) {
        auto *bn = dynamic_cast<BatchNorm *>(operands[i]);
        if (!bn || bn->fusedRelu || operands[i + 1]->OPERAND_ID() != OPR_CTRL_SHORTCUTENDPOINT_END) continue;
        auto *end = static_cast<ShortcutEndpoint *>(operands[i + 1]);
        if (end->operandCount > 0 || !end->fusedRelu || end->fusedRelu != operands[i + 2] || end->idleForward) continue;
        auto *r = static_cast<ReLU *>(operands[i + 2]);
        bn->fusedRelu = r, bn->shortcutValue = end->other->Y->A, bn->shortcutGrad = end->other->Y->dAReserve;
        r->absorbedBy = bn;
        end->fusedRelu = nullptr, end->idleForward = end->idleGrad = true;
    }
    // absorbed ReLU, opening endpoint: the operand that absorbed the ReLU adds the endpoint's two gradients itself
    for (uint32 i = 0; i + 1 < OPERAND_COUNT; i++) {
        if (operands[i]->OPERAND_ID() != OPR_SEBLAS_RELU || operands[i + 1]->OPERAND_ID() != OPR_CTRL_SHORTCUTENDPOINT_BEG) continue;
        auto *r = static_cast<ReLU *>(operands[i]);
        auto *beg = static_cast<ShortcutEndpoint *>(operands[i + 1]);
        if (!r->absorbedBy || beg->idleGrad || !beg->foldReserveEnabled) continue;
        if (r->absorbedBy->takeGradientInParts(beg->Y->dA, beg->Y->dAReserve)) beg->idleGrad = true;
    }
    if (hipDeviceSynchronize() != hipSuccess) assertHip(__FILE__, __LINE__);  // buffers are released below: nothing may be in flight
    for (uint32 i = 0; i + 1 < OPERAND_COUNT; i++) {
        OperandBase *op = operands[i];
        if (op->OPERAND_ID() != OPR_CTRL_SHORTCUTENDPOINT_BEG) continue;
        if (op->Y->A->elements == op->X->A->elements) continue;
        // The opening endpoint only passes its input on: its output value takes over the input's storage. Every tensor that
        // was bound to the old output buffer holds a copy of its address (Tensor::attach copies the pointer), so the
        // consumers are re-attached before anything can run: the next operand of the chain and, for a projection
        // shortcut, the first operand of the closing endpoint's branch.
        auto *beg = static_cast<ShortcutEndpoint *>(op);
        op->Y->A->destroy();
        op->Y->A->attach(op->X->A);
        operands[i + 1]->X->A->attach(op->Y->A);
        if (beg->other && beg->other->operandCount > 0) beg->other->branchOperands[0]->X->A->attach(op->Y->A);
    }
    // no operand may be left reading a buffer other than its producer's
    for (uint32 i = 1; i < OPERAND_COUNT; i++) {
        if (operands[i]->X->A->elements != operands[i - 1]->Y->A->elements)
            throw std::runtime_error("Sequential::streamline: an operand's input is not its predecessor's output");
        if (operands[i]->OPERAND_ID() == OPR_CTRL_SHORTCUTENDPOINT_END) {
            auto *end = static_cast<ShortcutEndpoint *>(operands[i]);
            if (end->operandCount > 0 && end->branchOperands[0]->X->A->elements != end->other->Y->A->elements)
                throw std::runtime_error("Sequential::streamline: a shortcut branch's input is not the opening endpoint's output");
        }
    }
}

// All parameters in one kernel launch. The device table of (weights, gradient, momentum, rates) is built on the first
// call and rebuilt when a rate changed; any optimizer other than Momentum makes this fall back to learn().
void Sequential::learnFused() {
    std::vector<NetParam *> params;
    for (OperandBase *op : operands) op->collectNetParams(params);
    std::vector<crb_momentum_item> items;
    uint32 maxCount = 0;
    for (NetParam *p : params) {
        auto *m = dynamic_cast<Momentum *>(p->opt);
        if (!m) {
            learn();
            return;
        }
        // a row of the launch grid covers one item with at most 64 workgroups: large tensors are entered in pieces so
        // that they spread over the chip like the many small ones
        const uint32 count = p->data()->dims.size, piece = 1u << 18;
        for (uint32 at = 0; at < count; at += piece) {
            const uint32 n = count - at < piece ? count - at : piece;
            items.push_back({p->data()->elements + at, p->grad()->elements + at, m->m->elements + at, n, m->LEARNING_RATE, m->BETA,
                             m->isWeight ? 1.0f - m->L2 : 1.0f});
            maxCount = n > maxCount ? n : maxCount;
        }
    }
    if (items.empty()) return;
    const size_t bytes = items.size() * sizeof(crb_momentum_item);
    if (fusedHost.size() != bytes || std::memcmp(fusedHost.data(), items.data(), bytes) != 0) {
        if (fusedTable && fusedHost.size() != bytes) {
            (void)hipFree(fusedTable);
            fusedTable = nullptr;
        }
        if (!fusedTable && hipMalloc(&fusedTable, bytes) != hipSuccess) assertHip(__FILE__, __LINE__);
        if (hipMemcpy(fusedTable, items.data(), bytes, hipMemcpyHostToDevice) != hipSuccess) assertHip(__FILE__, __LINE__);
        fusedHost.assign(reinterpret_cast<const char *>(items.data()), reinterpret_cast<const char *>(items.data()) + bytes);
    }
    throwOnStatus(crb_momentum_apply_multi(static_cast<const crb_momentum_item *>(fusedTable), uint32(items.size()), maxCount, nullptr),
                  __FILE__, __LINE__);
    if (isBlocking() && hipStreamSynchronize(nullptr) != hipSuccess) assertHip(__FILE__, __LINE__);
}

}  // namespace seann
