// seblas operator API over the C ABI: shape checks as in the reference, launch on the default stream,
// block until done, translate status codes to exceptions. See operations.h.
#include "operations.h"

#include <hip/hip_runtime_api.h>

#include <stdexcept>

#include "../../../../include/crusader_hip.h"
#include "../assist/HipAssert.h"

namespace seblas {

static void require(bool ok, const char *what) {
    if (!ok) throw std::invalid_argument(what);
}

// every reference op ends with cudaDeviceSynchronize(); assertCuda(...)
static void finish(int status, const char *file, int line) {
    throwOnStatus(status, file, line);
    if (isBlocking() && hipStreamSynchronize(nullptr) != hipSuccess) assertHip(file, line);
    assertHip(file, line);
}

Tensor *sgemm(Tensor *A, Tensor *B, Tensor *C) {
    require(A->dims.w == B->dims.h, "sgemm: A.w != B.h");       // cuGEMM.cu:1650
    require(A->dims.h == C->dims.h, "sgemm: A.h != C.h");       // :1651
    require(B->dims.w == C->dims.w, "sgemm: B.w != C.w");       // :1652
    finish(crb_sgemm_nn(A->elements, B->elements, C->elements, A->dims.h, B->dims.w, A->dims.w, B->dims.n, nullptr),
           __FILE__, __LINE__);
    return C;
}

Tensor *sgemmTN(Tensor *A, Tensor *B, Tensor *C) {
    require(A->dims.h == B->dims.h, "sgemmTN: A.h != B.h");                                // :1668
    require(A->dims.w == C->dims.h && B->dims.w == C->dims.w, "sgemmTN: C shape mismatch");  // :1669
    finish(crb_sgemm_tn(A->elements, B->elements, C->elements, A->dims.w, B->dims.w, A->dims.h, B->dims.n, nullptr),
           __FILE__, __LINE__);
    return C;
}

Tensor *sgemmNT(Tensor *A, Tensor *B, Tensor *C) {
    require(A->dims.w == B->dims.w, "sgemmNT: A.w != B.w");                                // :1686
    require(A->dims.h == C->dims.h && B->dims.h == C->dims.w, "sgemmNT: C shape mismatch");  // :1687
    finish(crb_sgemm_nt(A->elements, B->elements, C->elements, A->dims.h, B->dims.h, A->dims.w, nullptr), __FILE__,
           __LINE__);
    return C;
}

Tensor *sgemmNTA(Tensor *A, Tensor *B, Tensor *C) {
    require(A->dims.w == B->dims.w, "sgemmNTA: A.w != B.w");                                // :1702
    require(A->dims.h == C->dims.h && B->dims.h == C->dims.w, "sgemmNTA: C shape mismatch");  // :1703
    finish(crb_sgemm_nta(A->elements, B->elements, C->elements, A->dims.h, B->dims.h, A->dims.w, A->dims.n, nullptr),
           __FILE__, __LINE__);
    return C;
}

Tensor *linear(Tensor *X, Tensor *W, Tensor *B, Tensor *Y, bool relu) {
    const uint32 M = Y->dims.h;                                  // cuLinear.cu:1053
    const uint32 N = Y->dims.n * Y->dims.w;                      // :1054
    require(W->dims.w == X->dims.h, "linear: W.w != X.h");       // :1056
    require(B->dims.h == M, "linear: B.h != Y.h");               // :1057
    require(Y->dims.w == 1 && B->dims.w == 1 && X->dims.w == 1, "linear: X, B, Y must have w == 1");  // :1058
    require(X->dims.n == Y->dims.n, "linear: batch mismatch");   // :1059
    require(W->dims.h == M, "linear: W.h != Y.h");
    finish(crb_linear_fwd(X->elements, W->elements, B->elements, Y->elements, N, W->dims.w, M, relu ? CRB_FLAG_RELU : 0u, nullptr), __FILE__,
           __LINE__);
    return Y;
}

Tensor *linearXGrad(Tensor *dY, Tensor *W, Tensor *dX) {
    const uint32 N = dX->dims.n * dX->dims.w;                                // :1077
    require(W->dims.h == dY->dims.h, "linearXGrad: W.h != dY.h");            // :1079
    require(dX->dims.n == dY->dims.n, "linearXGrad: batch mismatch");        // :1080
    require(dX->dims.w == 1 && dY->dims.w == 1, "linearXGrad: w must be 1");  // :1081
    require(W->dims.w == dX->dims.h, "linearXGrad: W.w != dX.h");            // :1082
    finish(crb_linear_dgrad(dY->elements, W->elements, dX->elements, N, W->dims.w, W->dims.h, nullptr), __FILE__,
           __LINE__);
    return dX;
}

Tensor *linearParamGrad(Tensor *dY, Tensor *X, Tensor *dW, Tensor *dB) {
    const uint32 M = dW->dims.h, N = dW->dims.w;                          // :1099-1100
    require(X->dims.h == N, "linearParamGrad: X.h != dW.w");             // :1102
    require(dY->dims.h == M, "linearParamGrad: dY.h != dW.h");           // :1103
    require(X->dims.n == dY->dims.n, "linearParamGrad: batch mismatch");  // :1104
    require(dB->dims.size == M, "linearParamGrad: dB size != dW.h");
    finish(crb_linear_wgrad(dY->elements, X->elements, dW->elements, dB->elements, X->dims.n, N, M, nullptr), __FILE__,
           __LINE__);
    return dW;
}

// Geometry + the four relations of assertConv (cuConv.cu:731-755); h/w relations are checked by the C ABI with
// the reference's messages, channel/batch relations here.
static crb_conv_geom geom(Tensor *filters, Tensor *features, Tensor *featureOut, int sH, int sW, int pH, int pW) {
    require(sH > 0 && sW > 0 && pH >= 0 && pW >= 0, "assertConv: stride must be positive and padding non-negative");
    if (featureOut->dims.c != filters->dims.n || features->dims.c != filters->dims.c)
        throw std::invalid_argument("assertConv: channels relationship did not satisfy");
    if (featureOut->dims.n != features->dims.n) throw std::invalid_argument("assertConv: batch relationship did not satisfy");
    crb_conv_geom g;
    g.N = features->dims.n;
    g.IC = features->dims.c, g.IH = features->dims.h, g.IW = features->dims.w;
    g.OC = filters->dims.n, g.FH = filters->dims.h, g.FW = filters->dims.w;
    g.OH = featureOut->dims.h, g.OW = featureOut->dims.w;
    g.sH = uint32(sH), g.sW = uint32(sW), g.pH = uint32(pH), g.pW = uint32(pW);
    return g;
}

Tensor *conv(Tensor *A, Tensor *B, Tensor *C, int strideH, int strideW, int padH, int padW, Tensor *biases, bool relu) {
    crb_conv_geom g = geom(A, B, C, strideH, strideW, padH, padW);
    if (biases) require(biases->dims.size == g.OC, "conv: biases must hold OC elements");
    finish(crb_conv_fwd(A->elements, B->elements, C->elements, biases ? biases->elements : nullptr, &g, relu ? CRB_FLAG_RELU : 0u, nullptr),
           __FILE__, __LINE__);
    return C;
}

Tensor *convDerive(Tensor *A, Tensor *B, Tensor *C, int strideH, int strideW, int padH, int padW) {
    crb_conv_geom g = geom(A, C, B, strideH, strideW, padH, padW);  // assertConv(A, C, B, ...) cuConv.cu:775
    finish(crb_conv_dgrad(A->elements, B->elements, C->elements, &g, nullptr), __FILE__, __LINE__);
    return C;
}

Tensor *convError(Tensor *A, Tensor *B, Tensor *C, int strideH, int strideW, int padH, int padW) {
    crb_conv_geom g = geom(C, B, A, strideH, strideW, padH, padW);  // assertConv(C, B, A, ...) cuConv.cu:794
    finish(crb_conv_wgrad(A->elements, B->elements, C->elements, &g, nullptr, 0, nullptr), __FILE__, __LINE__);
    return A;  // the reference returns its first argument (cuConv.cu:805)
}

void convBackward(Tensor *filter, Tensor *dY, Tensor *X, Tensor *dX, Tensor *dFilter, int strideH, int strideW, int padH, int padW) {
    crb_conv_geom g = geom(filter, dX, dY, strideH, strideW, padH, padW);
    require(X->dims == dX->dims && dFilter->dims == filter->dims, "convBackward: gradient shapes differ from their tensors");
    finish(crb_conv_bwd(filter->elements, dY->elements, X->elements, dX->elements, dFilter->elements, &g, nullptr, 0, nullptr),
           __FILE__, __LINE__);
}

uint32 convBackwardSlices(Tensor *filter, Tensor *dY, Tensor *dX, int strideH, int strideW, int padH, int padW) {
    crb_conv_geom g = geom(filter, dX, dY, strideH, strideW, padH, padW);
    return crb_conv_bwd_slices(&g);
}

uint32 convBackwardSliceFloats(Tensor *filter, Tensor *dY, Tensor *dX, int strideH, int strideW, int padH, int padW) {
    crb_conv_geom g = geom(filter, dX, dY, strideH, strideW, padH, padW);
    return uint32(crb_conv_wgrad_workspace_bytes(&g) / sizeof(float));
}

void convBackwardSliced(Tensor *filter, Tensor *dY, Tensor *X, Tensor *dX, Tensor *slices, int strideH, int strideW, int padH, int padW) {
    crb_conv_geom g = geom(filter, dX, dY, strideH, strideW, padH, padW);
    require(X->dims == dX->dims, "convBackwardSliced: gradient shape differs from its tensor");
    finish(crb_conv_bwd_sliced(filter->elements, dY->elements, X->elements, dX->elements, &g, slices->elements,
                               size_t(slices->dims.size) * sizeof(float), nullptr),
           __FILE__, __LINE__);
}

void sumSlicesMulti(const SliceSumItem *items, uint32 count) {
    static_assert(sizeof(SliceSumItem) == sizeof(crb_slice_sum_item), "item layout");
    finish(crb_sum_slices_multi(reinterpret_cast<const crb_slice_sum_item *>(items), count, nullptr), __FILE__, __LINE__);
}

Tensor *convBias(Tensor *Y, Tensor *biases) {
    require(biases->dims.size == Y->dims.c, "convBias: bias size != channels");  // cuConv.cu:809
    finish(crb_conv_bias(Y->elements, biases->elements, Y->dims.n, Y->dims.c, Y->dims.h * Y->dims.w, nullptr), __FILE__,
           __LINE__);
    return Y;
}

// ---- elementwise / reduction operators ---------------------------------------------------------------------------------

Tensor *relu(Tensor *X, Tensor *Y) {
    require(X->dims.size == Y->dims.size, "relu: element counts differ");
    finish(crb_relu_fwd(X->elements, Y->elements, X->dims.size, nullptr), __FILE__, __LINE__);  // cuActivation.cu:268-280
    return Y;
}

Tensor *reluGradFast(Tensor *X, Tensor *dY, Tensor *dX) {
    require(X->dims.size == dY->dims.size && X->dims.size == dX->dims.size, "reluGradFast: element counts differ");
    finish(crb_relu_bwd(X->elements, dY->elements, dX->elements, X->dims.size, nullptr), __FILE__, __LINE__);  // :296-308
    return dX;
}

static void requirePool(const char *what, Tensor *X, Tensor *Y, Tensor *record, uint32 sH, uint32 sW, uint32 rH, uint32 rW) {
    require(sH && sW && rH && rW, what);
    require(X->dims.h >= rH - sH && X->dims.w >= rW - sW, what);
    require((X->dims.h - (rH - sH)) / sH == Y->dims.h, what);  // cuPool.cu:136
    require((X->dims.w - (rW - sW)) / sW == Y->dims.w, what);  // :137
    require(X->dims.n == Y->dims.n && X->dims.c == Y->dims.c, what);
    require(record->dims.size == uint64_t(X->dims.n) * X->dims.c * Y->dims.h * rH * Y->dims.w * rW, what);  // MaxPool2D.cuh:47-51
}

void maxPool(Tensor *X, Tensor *Y, Tensor *record, uint32 strideH, uint32 strideW, uint32 rangeH, uint32 rangeW) {
    requirePool("maxPool: shapes do not satisfy the pooling relationship", X, Y, record, strideH, strideW, rangeH, rangeW);
    finish(crb_maxpool_fwd(X->elements, Y->elements, record->elements, X->dims.n * X->dims.c, X->dims.h, X->dims.w, strideH,
                           strideW, rangeH, rangeW, nullptr),
           __FILE__, __LINE__);
}

void maxPoolBack(Tensor *dX, Tensor *dY, Tensor *record, uint32 strideH, uint32 strideW, uint32 rangeH, uint32 rangeW) {
    requirePool("maxPoolBack: shapes do not satisfy the pooling relationship", dX, dY, record, strideH, strideW, rangeH, rangeW);
    finish(crb_maxpool_bwd(dX->elements, dY->elements, record->elements, dX->dims.n * dX->dims.c, dX->dims.h, dX->dims.w,
                           strideH, strideW, rangeH, rangeW, nullptr),
           __FILE__, __LINE__);
}

Tensor *softmax(Tensor *A, Tensor *out, Tensor *buffer, uint32 step) {
    (void)buffer;
    require(step != 0 && A->dims.size % step == 0, "softmax: size is not a multiple of step");  // cuReduce.cu:297
    require(out->dims.size == A->dims.size, "softmax: element counts differ");                   // :298
    finish(crb_softmax(A->elements, out->elements, A->dims.size / step, step, nullptr), __FILE__, __LINE__);
    return out;
}

void crossEntropyLoss(Parameter *Y, Tensor *labels) {
    require(Y->A->dims.size == labels->dims.size, "crossEntropyLoss: element counts differ");
    finish(crb_cross_entropy_grad(Y->A->elements, labels->elements, Y->dA->elements, Y->A->dims.size, nullptr), __FILE__,
           __LINE__);  // cuLoss.cu:231-234
}

float crossEntropyCalc(Parameter *Y, Tensor *labels, Tensor *buf) {
    const uint32 n = Y->A->dims.size;
    require(n == labels->dims.size, "crossEntropyCalc: element counts differ");
    const uint32 need = crb_cross_entropy_scratch_floats(n);
    require(buf != nullptr && buf->dims.size >= need + 1, "crossEntropyCalc: buf too small");
    float *out = buf->elements + (buf->dims.size - 1);  // partial sums at the front, the total in the last element
    finish(crb_cross_entropy_loss(Y->A->elements, labels->elements, buf->elements, buf->dims.size - 1, out, n, nullptr),
           __FILE__, __LINE__);
    float loss = 0.f;
    if (hipMemcpy(&loss, out, sizeof(float), hipMemcpyDeviceToHost) != hipSuccess) assertHip(__FILE__, __LINE__);
    return loss;
}

Tensor *batchNorm(Tensor *X, Tensor *beta, Tensor *gamma, Tensor *mean, Tensor *var, Tensor *Y, Tensor *xHat) {
    require(X->dims.n == Y->dims.n && X->dims.size == Y->dims.size, "batchNorm: X and Y differ");  // cuBatchNorm.cu:162-163
    const uint32 F = X->dims.size / X->dims.n;
    require(xHat->dims.size == X->dims.size, "batchNorm: xHat size");
    require(beta->dims.size == F && gamma->dims.size == F && mean->dims.size == F && var->dims.size == F,
            "batchNorm: beta / gamma / mean / var must hold one value per feature");
    finish(crb_batchnorm_fwd(X->elements, beta->elements, gamma->elements, mean->elements, var->elements, Y->elements,
                             xHat->elements, X->dims.n, F, nullptr),
           __FILE__, __LINE__);
    return Y;
}

Tensor *batchNormGrad(Tensor *dY, Tensor *gamma, Tensor *X, Tensor *dX) {
    require(dY->dims.n == X->dims.n && dY->dims.size == X->dims.size, "batchNormGrad: dY and X differ");  // :177-178
    require(dX->dims.size == X->dims.size, "batchNormGrad: dX size");
    const uint32 F = X->dims.size / X->dims.n;
    require(gamma->dims.size == F, "batchNormGrad: gamma must hold one value per feature");
    finish(crb_batchnorm_bwd(dY->elements, gamma->elements, X->elements, dX->elements, nullptr, nullptr, X->dims.n, F, nullptr),
           __FILE__, __LINE__);
    return dX;
}

Tensor *batchNormGradAll(Tensor *dY, Tensor *gamma, Tensor *X, Tensor *dX, Tensor *dGamma, Tensor *dBeta) {
    require(dY->dims.n == X->dims.n && dY->dims.size == X->dims.size, "batchNormGradAll: dY and X differ");
    require(dX->dims.size == X->dims.size, "batchNormGradAll: dX size");
    const uint32 F = X->dims.size / X->dims.n;
    require(gamma->dims.size == F && dGamma->dims.size == F && dBeta->dims.size == F, "batchNormGradAll: one value per feature");
    finish(crb_batchnorm_bwd(dY->elements, gamma->elements, X->elements, dX->elements, dGamma->elements, dBeta->elements,
                             X->dims.n, F, nullptr),
           __FILE__, __LINE__);
    return dX;
}

Tensor *batchNormRelu(Tensor *X, Tensor *beta, Tensor *gamma, Tensor *mean, Tensor *var, Tensor *reluOut, Tensor *addend) {
    require(X->dims.n == reluOut->dims.n && X->dims.size == reluOut->dims.size, "batchNormRelu: X and the output differ");
    const uint32 F = X->dims.size / X->dims.n;
    require(beta->dims.size == F && gamma->dims.size == F && mean->dims.size == F && var->dims.size == F,
            "batchNormRelu: beta / gamma / mean / var must hold one value per feature");
    require(!addend || addend->dims.size == X->dims.size, "batchNormRelu: addend size");
    finish(crb_batchnorm_relu_fwd(X->elements, beta->elements, gamma->elements, mean->elements, var->elements, nullptr, nullptr,
                                  addend ? addend->elements : nullptr, reluOut->elements, X->dims.n, F, nullptr),
           __FILE__, __LINE__);
    return reluOut;
}

Tensor *batchNormReluGradAll(Tensor *dReluOut, Tensor *reluOut, Tensor *gamma, Tensor *X, Tensor *dX, Tensor *dGamma, Tensor *dBeta,
                             Tensor *dReluOut2, Tensor *maskedCopy) {
    require(dReluOut->dims.size == X->dims.size && reluOut->dims.size == X->dims.size && dX->dims.size == X->dims.size,
            "batchNormReluGradAll: tensor sizes differ");
    const uint32 F = X->dims.size / X->dims.n;
    require(gamma->dims.size == F && dGamma->dims.size == F && dBeta->dims.size == F, "batchNormReluGradAll: one value per feature");
    require((!dReluOut2 || dReluOut2->dims.size == X->dims.size) && (!maskedCopy || maskedCopy->dims.size == X->dims.size),
            "batchNormReluGradAll: optional tensor sizes differ");
    finish(crb_batchnorm_relu_bwd(dReluOut->elements, dReluOut2 ? dReluOut2->elements : nullptr, reluOut->elements, gamma->elements,
                                  X->elements, dX->elements, dGamma->elements, dBeta->elements, maskedCopy ? maskedCopy->elements : nullptr,
                                  X->dims.n, F, nullptr),
           __FILE__, __LINE__);
    return dX;
}

Tensor *addRelu(Tensor *A, Tensor *B, Tensor *out) {
    require(A->dims.size == B->dims.size && A->dims.size == out->dims.size, "addRelu: element counts differ");
    finish(crb_tensor_add_relu(out->elements, A->elements, B->elements, out->dims.size, nullptr), __FILE__, __LINE__);
    return out;
}

void reluGradTwice(Tensor *out, Tensor *dOut, Tensor *d1, Tensor *d2, Tensor *dOut2) {
    require(out->dims.size == dOut->dims.size && out->dims.size == d1->dims.size && out->dims.size == d2->dims.size,
            "reluGradTwice: element counts differ");
    require(!dOut2 || dOut2->dims.size == out->dims.size, "reluGradTwice: second gradient part size");
    finish(crb_tensor_relu_grad_copy2(d1->elements, d2->elements, out->elements, dOut->elements, dOut2 ? dOut2->elements : nullptr,
                                      out->dims.size, nullptr),
           __FILE__, __LINE__);
}

void batchNormParamGrads(Tensor *dY, Tensor *xHat, Tensor *dGamma, Tensor *dBeta) {
    require(dY->dims.n == xHat->dims.n && dY->dims.size == xHat->dims.size, "batchNormParamGrads: dY and xHat differ");  // :191-192
    const uint32 F = dY->dims.size / dY->dims.n;
    require(dGamma->dims.size == F && dBeta->dims.size == F, "batchNormParamGrads: one value per feature");
    finish(crb_batchnorm_param_grads(dY->elements, xHat->elements, dGamma->elements, dBeta->elements, dY->dims.n, F, nullptr),
           __FILE__, __LINE__);
}

void momentumApply(Tensor *X, Tensor *Xgrad, Tensor *V, float LEARNING_RATE, float MOMENTUM) {
    momentumApplyDecay(X, Xgrad, V, LEARNING_RATE, MOMENTUM, 0.0f);
}

void momentumApplyDecay(Tensor *X, Tensor *Xgrad, Tensor *V, float LEARNING_RATE, float MOMENTUM, float L2) {
    require(X->dims.size == Xgrad->dims.size && X->dims.size == V->dims.size, "momentumApply: element counts differ");
    finish(crb_momentum_apply(X->elements, Xgrad->elements, V->elements, X->dims.size, LEARNING_RATE, MOMENTUM, 1.0f - L2,
                              nullptr),
           __FILE__, __LINE__);  // cuOptim.cu:259-272
}

}  // namespace seblas
