// Conv2D and Linear operands: thin glue over the seblas operator API, in the reference's calling order.
#include <hip/hip_runtime_api.h>

#include <cmath>

#include "../../../../include/crusader_hip.h"
#include "../../seblas/assist/HipAssert.h"
#include "Conv2D.h"
#include "Linear.h"

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
    conv(filter->data(), X->A, Y->A, int(strideH), int(strideW), int(padH), int(padW), WITH_BIAS ? bias->data() : nullptr);
}

void Conv2D::xGrads() {  // Conv2D.cu:18-22
    *Y->dA + Y->dAReserve;
    convDerive(filter->data(), Y->dA, X->dA, int(strideH), int(strideW), int(padH), int(padW));
    Y->dAReserve->constFill(0);
}

void Conv2D::paramGrads() {  // Conv2D.cu:24-29; the bias gradient is the per-channel sum of dY
    convError(Y->dA, X->A, filter->grad(), int(strideH), int(strideW), int(padH), int(padW));
    if (WITH_BIAS) {
        const shape4 &d = Y->dA->dims;
        throwOnStatus(crb_conv_bias_grad(Y->dA->elements, bias->grad()->elements, d.n, d.c, d.h * d.w, nullptr), __FILE__,
                      __LINE__);
        if (hipStreamSynchronize(nullptr) != hipSuccess) assertHip(__FILE__, __LINE__);
    }
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

void Linear::forward() { linear(X->A, weights->data(), biases->data(), Y->A); }  // Linear.cu:17-19

void Linear::paramGrads() { linearParamGrad(Y->dA, X->A, weights->grad(), biases->grad()); }  // :21-23

void Linear::xGrads() {  // Linear.cu:35-40
    *Y->dA + Y->dAReserve;
    linearXGrad(Y->dA, weights->data(), X->dA);
    Y->dAReserve->constFill(0);
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

}  // namespace seann
