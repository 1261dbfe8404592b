// The seblas free-function operator API of the GEMM / linear / convolution path, with the reference's
// signatures, argument meaning, return-pointer quirks, blocking behaviour and error behaviour
// (seblas/operations/cuGEMM.cuh:12-21, cuConv.cuh:20-42, cuLinear.cuh:14-18). Each function validates shapes
// the way the reference does, calls the C ABI in include/crusader_hip.h on the default stream, synchronises
// (the reference ends every op with cudaDeviceSynchronize) and throws on failure.
//
// Shape violations: the reference uses assert() for GEMM/linear (abort in debug builds, unchecked in release)
// and std::invalid_argument for conv; here both throw std::invalid_argument. Device errors throw
// std::runtime_error.
#pragma once
#include "../tensor/Parameter.h"
#include "../tensor/Tensor.h"

namespace seblas {
// cuGEMM.cu:1649-1714
Tensor *sgemm(Tensor *A, Tensor *B, Tensor *C);     // C[n] = A * B[n]
Tensor *sgemmTN(Tensor *A, Tensor *B, Tensor *C);   // C[n] = A^T * B[n]
Tensor *sgemmNT(Tensor *A, Tensor *B, Tensor *C);   // C = A * B^T
Tensor *sgemmNTA(Tensor *A, Tensor *B, Tensor *C);  // C += sum_n A[n] * B[n]^T

// cuLinear.cu:1052-1113
Tensor *linear(Tensor *X, Tensor *W, Tensor *B, Tensor *Y, bool relu = false);  // relu: max(., 0) applied in the same pass (not in the reference)
Tensor *linearXGrad(Tensor *dY, Tensor *W, Tensor *dX);
Tensor *linearParamGrad(Tensor *dY, Tensor *X, Tensor *dW, Tensor *dB);  // returns dW

// cuConv.cu:757-818. A: filters OC x IC x FH x FW.
Tensor *conv(Tensor *A, Tensor *B, Tensor *C, int strideH, int strideW, int padH, int padW, Tensor *biases, bool relu = false);
Tensor *convDerive(Tensor *A, Tensor *B, Tensor *C, int strideH, int strideW, int padH, int padW);
// A: errors N x OC x OH x OW, B: inputs N x IC x IH x IW, C: filter grads (accumulated). Returns A, as the
// reference does (cuConv.cu:805).
Tensor *convError(Tensor *A, Tensor *B, Tensor *C, int strideH, int strideW, int padH, int padW);
// convDerive(filter, dY, dX, ...) and convError(dY, X, dFilter, ...) in one call: the two gradients of a layer are independent
// and, for the layer shapes of CIFAR residual networks, run as one kernel launch. Same results as the two calls. No
// counterpart in the reference.
void convBackward(Tensor *filter, Tensor *dY, Tensor *X, Tensor *dX, Tensor *dFilter, int strideH, int strideW, int padH, int padW);
// The same with the filter gradient's last step postponed: convBackwardSliced writes dX and leaves the filter gradient of
// this call as convBackwardSlices(...) partial sums in `slices` (a device tensor of convBackwardSliceFloats(...) floats
// that the caller keeps until the sum); sumSlicesMulti then completes any number of such gradients in one launch
// (grad += sum of its slices; same bits as convBackward). convBackwardSlices returns 0 where there is no sliced form.
struct SliceSumItem {  // layout of crb_slice_sum_item
    const float *slices;
    float *dst;
    uint32 count, n_slices;
};
uint32 convBackwardSlices(Tensor *filter, Tensor *dY, Tensor *dX, int strideH, int strideW, int padH, int padW);
uint32 convBackwardSliceFloats(Tensor *filter, Tensor *dY, Tensor *dX, int strideH, int strideW, int padH, int padW);
void convBackwardSliced(Tensor *filter, Tensor *dY, Tensor *X, Tensor *dX, Tensor *slices, int strideH, int strideW, int padH, int padW);
void sumSlicesMulti(const SliceSumItem *items, uint32 count);
Tensor *convBias(Tensor *Y, Tensor *biases);

// ---- the elementwise / reduction operators a training step runs between those calls -------------------------------
// cuActivation.cuh:13,18
Tensor *relu(Tensor *X, Tensor *Y);
Tensor *reluGradFast(Tensor *X, Tensor *dY, Tensor *dX);
// cuPool.cuh:13-17. Non-overlapping windows only (stride == range); see include/crusader_hip.h.
void maxPool(Tensor *X, Tensor *Y, Tensor *record, uint32 strideH, uint32 strideW, uint32 rangeH, uint32 rangeW);
void maxPoolBack(Tensor *dX, Tensor *dY, Tensor *record, uint32 strideH, uint32 strideW, uint32 rangeH, uint32 rangeW);
// cuReduce.cuh:44. `buffer` is accepted for signature compatibility and never used (may be null).
Tensor *softmax(Tensor *A, Tensor *out, Tensor *buffer, uint32 step);
// cuLoss.cuh:18,20. crossEntropyLoss: Y->dA = Y->A - labels. crossEntropyCalc: sum of -log(Y->A + 1e-10)*label; `buf`
// is device scratch (the reference passes a tensor of Y's size; its last element receives the sum before the copy back).
void crossEntropyLoss(Parameter *Y, Tensor *labels);
float crossEntropyCalc(Parameter *Y, Tensor *labels, Tensor *buf);
// cuBatchNorm.cuh: per-feature batch normalisation (a feature = one (c,h,w) position; statistics over n). beta, gamma,
// mean, var have the shape of one sample. batchNormParamGrads overwrites dGamma / dBeta. Any batch size (the reference
// asserts n <= 96).
Tensor *batchNorm(Tensor *X, Tensor *beta, Tensor *gamma, Tensor *mean, Tensor *var, Tensor *Y, Tensor *xHat);
Tensor *batchNormGrad(Tensor *dY, Tensor *gamma, Tensor *X, Tensor *dX);
void batchNormParamGrads(Tensor *dY, Tensor *xHat, Tensor *dGamma, Tensor *dBeta);
// batchNormGrad and batchNormParamGrads in one pass over the data (no counterpart in the reference; same results up to
// the rounding of xHat, which is recomputed instead of read back).
Tensor *batchNormGradAll(Tensor *dY, Tensor *gamma, Tensor *X, Tensor *dX, Tensor *dGamma, Tensor *dBeta);
// Normalisation and the ReLU behind it in one pass each way (same results as the two operators one after the other; no
// counterpart in the reference). Forward writes reluOut = relu(batchNorm(X)), mean and var; backward takes the gradient
// with respect to reluOut and yields dX, dGamma, dBeta.
// addend (or null): the other summand of a residual connection that closes between the normalisation and the ReLU.
// dReluOut2 (or null): second part of the gradient (a residual connection opens right behind the ReLU: its main-path
// and shortcut gradients are added here instead of in a pass of their own). maskedCopy (or null) receives the gradient as
// it reaches the normalisation, for the shortcut of the connection that closes in front of the ReLU.
Tensor *batchNormRelu(Tensor *X, Tensor *beta, Tensor *gamma, Tensor *mean, Tensor *var, Tensor *reluOut, Tensor *addend = nullptr);
Tensor *batchNormReluGradAll(Tensor *dReluOut, Tensor *reluOut, Tensor *gamma, Tensor *X, Tensor *dX, Tensor *dGamma, Tensor *dBeta,
                             Tensor *dReluOut2 = nullptr, Tensor *maskedCopy = nullptr);
// out = relu(A + B), and the ReLU's gradient (dOut where out > 0, else 0) written to two tensors at once: the closing
// shortcut endpoint with the ReLU behind it.
Tensor *addRelu(Tensor *A, Tensor *B, Tensor *out);
void reluGradTwice(Tensor *out, Tensor *dOut, Tensor *d1, Tensor *d2, Tensor *dOut2 = nullptr);  // dOut2: second part of the gradient
// cuOptim.cuh:16. V is the momentum buffer; Xgrad is cleared by the step.
void momentumApply(Tensor *X, Tensor *Xgrad, Tensor *V, float LEARNING_RATE, float MOMENTUM);
// Optimizers.cu:16-22 in one pass: X *= (1 - L2) then momentumApply. No separate counterpart in the reference.
void momentumApplyDecay(Tensor *X, Tensor *Xgrad, Tensor *V, float LEARNING_RATE, float MOMENTUM, float L2);
}  // namespace seblas
