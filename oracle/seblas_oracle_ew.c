/*
 * seblas_oracle_ew.c — CPU fp32 restatement of the elementwise / reduction operators that surround the
 * GEMM and convolution path in a training step: ReLU, max pooling, softmax, cross-entropy, the in-place
 * tensor arithmetic, the momentum update and per-feature batch normalisation.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE (same rule as seblas_oracle.c): only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg may load it.
 *
 * Each function follows the reference's intended arithmetic in plain scalar loops and cites the lines it
 * restates (paths relative to the reference tree). The reference cannot be built here and holds no golden
 * vectors; each function is pinned in tests/test_oracle_elementwise.py by independent checks:
 *   relu / reluGradFast   numpy maximum / where; the gradient is the derivative of the forward (finite differences
 *                         away from 0)
 *   maxPool / maxPoolBack torch-CPU max_pool2d and its autograd on tie-free inputs; tie rule (first maximum in
 *                         row-major window order) by a hand-written 4x4 case; record has exactly one 1 per window
 *   softmax               numpy float64 exp/sum; rows sum to 1/(1 + 1e-10/s); invariance to a per-row shift
 *   crossEntropy*         numpy float64 -sum(label*log(y + 1e-10)); gradient = softmax - label is the derivative of
 *                         the loss through the softmax (finite differences)
 *   tensor add/sub/scale/fill   numpy
 *   momentumApply         closed form after k steps with a constant gradient; numpy float64 recurrence
 *   batchNorm*            torch-CPU batch_norm (training mode) and its autograd in float64; xHat has zero mean and unit
 *                         variance per feature; finite differences
 * No function here is "parity unpinned".
 */
#include <math.h>
#include <stdint.h>
#include <stddef.h>

typedef uint32_t u32;

/* relu: Y = max(X, 0) (seblas/operations/cuActivation.cu:14-19 reluD, :28-39 relu4D, host :268-280). */
void oracle_relu(const float *X, float *Y, u32 n) {
    for (u32 i = 0; i < n; ++i) Y[i] = X[i] > 0.0f ? X[i] : 0.0f;
}

/* reluGradFast: dX = X > 0 ? dY : 0 (cuActivation.cu:54-59 reluDGradFast, :61-76 relu4DGradFast, host :296-308). */
void oracle_reluGradFast(const float *X, const float *dY, float *dX, u32 n) {
    for (u32 i = 0; i < n; ++i) dX[i] = X[i] > 0.0f ? dY[i] : 0.0f;
}

/* maxPool with non-overlapping windows (range == stride, the only case the reference's indexing addresses
 * correctly: cuPool.cu:8-40 multiplies the Y plane offset by strideH*strideW to reach the X plane).
 * X: planes x IH x IW, Y: planes x OH x OW with OH = IH / rH, OW = IW / rW (host asserts :135-137).
 * Y = window maximum starting from -1e15 with a strict '>' in row-major window order (:20-35), so the FIRST maximum
 * wins; record (same extent as the pooled region of X: planes x OH*rH x OW*rW) gets 1 at that element (:37-38).
 * The reference leaves the other record entries untouched (they are 0 by construction: created zeroed, and the
 * backward pass clears the entry it used, :68-69); here every window entry is written, 1 or 0. */
void oracle_maxPool(const float *X, float *Y, float *record, u32 planes, u32 IH, u32 IW, u32 rH, u32 rW) {
    const u32 OH = IH / rH, OW = IW / rW;
    const u32 RH = OH * rH, RW = OW * rW;
    for (u32 p = 0; p < planes; ++p)
        for (u32 oh = 0; oh < OH; ++oh)
            for (u32 ow = 0; ow < OW; ++ow) {
                float best = -1e15f;
                u32 bi = 0, bj = 0;
                for (u32 i = 0; i < rH; ++i)
                    for (u32 j = 0; j < rW; ++j) {
                        const float v = X[((size_t)p * IH + oh * rH + i) * IW + ow * rW + j];
                        if (v > best) best = v, bi = i, bj = j;
                    }
                for (u32 i = 0; i < rH; ++i)
                    for (u32 j = 0; j < rW; ++j)
                        record[((size_t)p * RH + oh * rH + i) * RW + ow * rW + j] = (i == bi && j == bj) ? 1.0f : 0.0f;
                Y[((size_t)p * OH + oh) * OW + ow] = best;
            }
}

/* maxPoolBack: the window element whose record is the first maximum (the 1 written by the forward pass; element
 * (0,0) when the window holds no 1) receives dY, and its record entry is cleared (cuPool.cu:42-70).
 * The reference writes only that element of dX; here the rest of the window is written as 0 (what a freshly created
 * gradient tensor holds), and dX elements outside the pooled region (IH % rH rows, IW % rW columns) are set to 0. */
void oracle_maxPoolBack(float *dX, const float *dY, float *record, u32 planes, u32 IH, u32 IW, u32 rH, u32 rW) {
    const u32 OH = IH / rH, OW = IW / rW;
    const u32 RH = OH * rH, RW = OW * rW;
    for (size_t i = 0; i < (size_t)planes * IH * IW; ++i) dX[i] = 0.0f;
    for (u32 p = 0; p < planes; ++p)
        for (u32 oh = 0; oh < OH; ++oh)
            for (u32 ow = 0; ow < OW; ++ow) {
                float best = -1e15f;
                u32 bi = 0, bj = 0;
                for (u32 i = 0; i < rH; ++i)
                    for (u32 j = 0; j < rW; ++j) {
                        const float v = record[((size_t)p * RH + oh * rH + i) * RW + ow * rW + j];
                        if (v > best) best = v, bi = i, bj = j;
                    }
                dX[((size_t)p * IH + oh * rH + bi) * IW + ow * rW + bj] = dY[((size_t)p * OH + oh) * OW + ow];
                record[((size_t)p * RH + oh * rH + bi) * RW + ow * rW + bj] = 0.0f;
            }
}

/* softmax over consecutive groups of `step` elements: out = exp(a - max) / (sum exp(a - max) + 1e-10)
 * (cuReduce.cu:98-146 softmaxD1024: row maximum, exp(val - max), row sum, val / (sum + 1e-10); host :296-315;
 * the looped variant for step > 1024, :320-357, computes the same quantities). Float exp, float running sum
 * in ascending order. */
void oracle_softmax(const float *A, float *out, u32 rows, u32 step) {
    for (u32 r = 0; r < rows; ++r) {
        const float *a = A + (size_t)r * step;
        float *o = out + (size_t)r * step;
        float mx = -1e15f;
        for (u32 i = 0; i < step; ++i) mx = a[i] > mx ? a[i] : mx;
        float sum = 0.0f;
        for (u32 i = 0; i < step; ++i) {
            o[i] = expf(a[i] - mx);
            sum += o[i];
        }
        const float den = sum + 1e-10f;
        for (u32 i = 0; i < step; ++i) o[i] = o[i] / den;
    }
}

/* crossEntropyLoss: dY = Y - labels (cuLoss.cu:231-234: copy A to dA, then dA -= labels) — the gradient of the
 * cross-entropy of a softmax output with respect to the softmax input. */
void oracle_crossEntropyLoss(const float *Y, const float *labels, float *dY, u32 n) {
    for (u32 i = 0; i < n; ++i) dY[i] = Y[i] - labels[i];
}

/* crossEntropyCalc: sum over all elements of -log(Y + 1e-10) * label (cuLoss.cu:31-37 crossEntropyPrepare, :220-228:
 * the per-element terms are summed by reduce(buf, buf)). Terms in float, accumulated in double so the oracle's own
 * rounding does not depend on the element count. */
float oracle_crossEntropyCalc(const float *Y, const float *labels, u32 n) {
    double s = 0.0;
    for (u32 i = 0; i < n; ++i) s += (double)(-logf(Y[i] + 1e-10f) * labels[i]);
    return (float)s;
}

/* In-place tensor arithmetic (seblas/tensor/Tensor.cu:462-483 operator+(Tensor*), :485-506 operator-(Tensor*),
 * operator*(float) :596-617 used as `*A * (1 - L2)` in seann/optimizers/Optimizers.cu:10,18, :638-657 constFill). */
void oracle_tensorAdd(float *A, const float *B, u32 n) {
    for (u32 i = 0; i < n; ++i) A[i] = A[i] + B[i];
}
void oracle_tensorSub(float *A, const float *B, u32 n) {
    for (u32 i = 0; i < n; ++i) A[i] = A[i] - B[i];
}
void oracle_tensorScale(float *A, float s, u32 n) {
    for (u32 i = 0; i < n; ++i) A[i] = A[i] * s;
}
void oracle_constFill(float *A, float v, u32 n) {
    for (u32 i = 0; i < n; ++i) A[i] = v;
}

/* Momentum step with the weight decay the optimizer applies first (Optimizers.cu:16-22: `A *= (1 - L2)` for weights,
 * then momentumApply; cuOptim.cu:38-46 momentumApplyD, :48-73 momentumApply4D, host :259-272):
 *   x = x * decay;  m = beta*m + (1 - beta)*g;  x -= lr*m;  g = 0.
 * decay = 1 - L2 for weights, 1 for biases. Each product and sum is rounded to float separately (volatile keeps the
 * compiler from fusing), matching two separate kernels for decay and update. */
void oracle_momentumApply(float *X, float *G, float *M, u32 n, float lr, float beta, float decay) {
    for (u32 i = 0; i < n; ++i) {
        volatile float x = X[i] * decay;
        volatile float a = beta * M[i];
        volatile float b = (1.0f - beta) * G[i];
        volatile float m = a + b;
        volatile float step = lr * m;
        X[i] = x - step;
        M[i] = m;
        G[i] = 0.0f;
    }
}

/* ---- batch normalisation over the batch dimension, per feature -----------------------------------------------------
 * A "feature" is one (c, h, w) position: X is viewed as N x F with F = C*H*W, and every column is normalised with its
 * own statistics over the N samples (seblas/operations/cuBatchNorm.cu:13-61: one thread per feature index, loop over
 * depth = sample). beta, gamma, mean, var hold F values. Pinned in tests/test_oracle_elementwise.py by torch-CPU
 * batch_norm (training mode, eps 1e-8) on the N x F view in float64, its autograd for all three gradients, the
 * zero-mean / unit-variance property of xHat, and finite differences. */

/* batchNorm (cuBatchNorm.cu:13-61, host :150-164): mean = sum/N, var = sum (x-mean)^2 / N (biased),
 * xHat = (x - mean) / sqrt(var + 1e-8), Y = xHat*gamma + beta; mean, var and xHat are stored. The reference asserts
 * N <= 96 (its shared-memory staging, :9,164); that limit does not exist here. */
void oracle_batchNorm(const float *X, const float *beta, const float *gamma, float *mean, float *var, float *Y,
                      float *xHat, u32 N, u32 F) {
    for (u32 f = 0; f < F; ++f) {
        float m = 0.0f, v = 0.0f;
        for (u32 n = 0; n < N; ++n) m += X[(size_t)n * F + f];
        m /= (float)N;
        for (u32 n = 0; n < N; ++n) {
            const float d = X[(size_t)n * F + f] - m;
            v += d * d;
        }
        v /= (float)N;
        const float inv = 1.0f / sqrtf(v + 1e-8f);
        for (u32 n = 0; n < N; ++n) {
            const float xh = (X[(size_t)n * F + f] - m) * inv;
            xHat[(size_t)n * F + f] = xh;
            Y[(size_t)n * F + f] = xh * gamma[f] + beta[f];
        }
        mean[f] = m;
        var[f] = v;
    }
}

/* batchNormGrad (cuBatchNorm.cu:63-125, host :167-178): statistics are recomputed from X, then with dxHat = dY*gamma
 *   dVar  = sum dxHat*(x-mean) * -0.5*(var+1e-8)^(-3/2)
 *   dMean = sum dxHat * -1/sqrt(var+1e-8)  +  dVar * sum(-2(x-mean)) / N
 *   dX    = dxHat/sqrt(var+1e-8) + dVar*2(x-mean)/N + dMean/N. */
void oracle_batchNormGrad(const float *dY, const float *gamma, const float *X, float *dX, u32 N, u32 F) {
    for (u32 f = 0; f < F; ++f) {
        float m = 0.0f, v = 0.0f;
        for (u32 n = 0; n < N; ++n) m += X[(size_t)n * F + f];
        m /= (float)N;
        for (u32 n = 0; n < N; ++n) {
            const float d = X[(size_t)n * F + f] - m;
            v += d * d;
        }
        v /= (float)N;
        const float inv = 1.0f / sqrtf(v + 1e-8f);
        const float g = gamma[f];
        float dVar = 0.0f, dMean = 0.0f, temp = 0.0f;
        for (u32 n = 0; n < N; ++n) {
            const float d = X[(size_t)n * F + f] - m;
            const float dxh = dY[(size_t)n * F + f] * g;
            dVar += dxh * d * -0.5f * inv * inv * inv;
            dMean += dxh * -inv;
            temp += -2.0f * d;
        }
        dMean += dVar * temp / (float)N;
        for (u32 n = 0; n < N; ++n) {
            const float d = X[(size_t)n * F + f] - m;
            const float dxh = dY[(size_t)n * F + f] * g;
            dX[(size_t)n * F + f] = dxh * inv + dVar * d * 2.0f / (float)N + dMean / (float)N;
        }
    }
}

/* batchNormParamGrads (cuBatchNorm.cu:127-147, host :180-191): dBeta = sum dY, dGamma = sum dY*xHat; both OVERWRITE.
 * (The BatchNorm operand of the reference passes the two output tensors in swapped order,
 * seann/operands/seblas/BatchNorm.cu:24 against cuBatchNorm.cu:180, so its beta receives dGamma and its gamma dBeta;
 * that slip is not reproduced: here dGamma is the gradient of gamma.) */
void oracle_batchNormParamGrads(const float *dY, const float *xHat, float *dGamma, float *dBeta, u32 N, u32 F) {
    for (u32 f = 0; f < F; ++f) {
        float db = 0.0f, dg = 0.0f;
        for (u32 n = 0; n < N; ++n) {
            const float dy = dY[(size_t)n * F + f];
            db += dy;
            dg += dy * xHat[(size_t)n * F + f];
        }
        dBeta[f] = db;
        dGamma[f] = dg;
    }
}
