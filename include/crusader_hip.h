/*
 * crusader_hip.h — C ABI of the MI355X (gfx950) implementation of the seblas fp32 GEMM /
 * linear / convolution hot path.
 *
 * Conventions
 *   - Every pointer is a DEVICE pointer to row-major fp32 (tensors are NCHW), owned by the caller.
 *     The library never frees caller memory and never retains a pointer after the call returns.
 *   - Dimensions are passed by value as uint32_t. Any dimension >= 1 is accepted; element counts of
 *     a single operand must stay below 2^31.
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream). Calls only enqueue work;
 *     they do not synchronise. The reference's blocking behaviour (cudaDeviceSynchronize after every
 *     op, e.g. seblas/operations/cuGEMM.cu:1661) is restored by the C++ seblas wrappers, which
 *     synchronise the stream after the call.
 *   - Return value: CRB_OK (0) or a negative crb_status. The reference signals the same conditions
 *     with assert()/std::invalid_argument (shape) and std::runtime_error (device error,
 *     seblas/assist/CudaAssert.cu:8-15); the C++ wrappers translate. crb_last_error_string() gives
 *     the message of the calling thread's most recent failure.
 *   - "overwrite" entry points write every element of their output; "accumulate" entry points
 *     read-modify-write it (C += ...), exactly once per element, deterministically.
 */
#ifndef CRUSADER_HIP_H
#define CRUSADER_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum crb_status {
    CRB_OK = 0,
    CRB_EINVAL_SHAPE = -1, /* a shape relation the reference asserts does not hold, or a zero dim */
    CRB_ENULL = -2,        /* a required pointer is NULL */
    CRB_EHIP = -3,         /* a HIP runtime call or kernel launch failed */
    CRB_EWORKSPACE = -4    /* caller-provided workspace is too small */
} crb_status;

/* Flags for crb_conv_fwd / crb_linear_fwd. Default 0 reproduces the reference (bias only). */
#define CRB_FLAG_NONE 0u
#define CRB_FLAG_RELU 1u /* extra, not in the reference: clamp the output at 0 in the epilogue */

/* Library / device ------------------------------------------------------------------------- */

/* Version of this ABI (major*1000 + minor). */
int crb_abi_version(void);

/* Message for the most recent non-OK status returned to the calling thread ("" if none). */
const char *crb_last_error_string(void);

/* Releases the library's lazily grown split-K scratch arenas (call it only when no library kernel is in
 * flight and no recorded graph that used the arenas will be replayed). The library keeps one arena per
 * (device, stream), so calls queued on different streams never share scratch and may overlap; calls on
 * one stream run in order and reuse that stream's arena. An arena grows with hipMalloc on first use or
 * when a call needs more; a block it has outgrown stays allocated until this call, because work in
 * flight or a recorded graph may still name it. Growth is refused (CRB_EWORKSPACE) while the stream is
 * being captured. Callers that must not allocate bind their own block (crb_bind_workspace) or pass a
 * workspace where an entry point takes one. */
void crb_release_workspace(void);

/* Binds a caller-owned block of device memory (256-byte aligned) to `stream` of the current device as the split scratch
 * of every entry point that takes no workspace argument of its own (the GEMM and dense-layer families, the general
 * convolution forward / data-gradient path, crb_conv_bias_grad, and the convolution entry points when their workspace
 * argument is NULL). While a block is bound, calls on that stream never allocate: a call that needs more than the block
 * holds returns CRB_EWORKSPACE. The *_workspace_bytes queries below tell what a call needs. workspace == NULL unbinds
 * (the library arena serves the stream again). The block must stay valid until the work queued on the stream that uses
 * it has finished; the library never frees it. No counterpart in the reference, whose operators never need scratch
 * (seblas/operations/cuGEMM.cu:1649-1714 launches one kernel per call). For callers that record the calls into a HIP
 * graph or must not allocate on their hot path. One stream must not be driven by several host threads at once. */
int crb_bind_workspace(void *workspace, size_t workspace_bytes, void *stream);

/* GEMM family ------------------------------------------------------------------------------ */

/* Bytes of split scratch a call of the GEMM or dense-layer family needs (0: none) when its result is M x N per batch
 * entry and its contraction has length K: crb_sgemm_nn / crb_sgemm_tn (M, N, K, batch); crb_sgemm_nt (M, N, K, 1);
 * crb_sgemm_nta (M, N, K * batch, 1); crb_linear_fwd (batch, OUT, IN, 1); crb_linear_dgrad (batch, IN, OUT, 1);
 * crb_linear_wgrad (OUT, IN, batch, 1). The scratch comes from the block bound with crb_bind_workspace, else from the
 * library arena. */
size_t crb_gemm_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t batch);

/* Replaces seblas::sgemm (seblas/operations/cuGEMM.cu:1649-1664; kernels :34-210, :791-999).
 * For nd in [0,batch): C[nd] (MxN) = A (MxK) * B[nd] (KxN). A is shared across the batch
 * (batch = B.n in the reference). Overwrite. */
int crb_sgemm_nn(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                 void *stream);

/* Replaces seblas::sgemmTN (cuGEMM.cu:1667-1682; kernels :229-409, :1016-1217).
 * For nd in [0,batch): C[nd] (MxN) = A^T * B[nd], A stored K x M. Overwrite. */
int crb_sgemm_tn(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                 void *stream);

/* Replaces seblas::sgemmNT (cuGEMM.cu:1685-1699; kernels :427-595, :1222-1429).
 * C (MxN) = A (MxK) * B^T, B stored N x K. No batch. Overwrite. */
int crb_sgemm_nt(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, void *stream);

/* Replaces seblas::sgemmNTA (cuGEMM.cu:1701-1714; kernels :600-773, :1434-1647).
 * C (MxN) += sum_{nd<batch} A[nd] (MxK) * B[nd]^T (B[nd] stored N x K). Accumulate. */
int crb_sgemm_nta(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                  void *stream);

/* Dense-layer family ------------------------------------------------------------------------ */

/* Replaces seblas::linear (seblas/operations/cuLinear.cu:1052-1072; kernels :33-206, :224-439).
 * Y (batch x OUT) = X (batch x IN) * W^T (W stored OUT x IN) + bias (OUT). bias must not be NULL
 * (the reference dereferences it unconditionally). Overwrite. flags: CRB_FLAG_*. */
int crb_linear_fwd(const float *X, const float *W, const float *bias, float *Y, uint32_t batch, uint32_t IN,
                   uint32_t OUT, uint32_t flags, void *stream);

/* Replaces seblas::linearXGrad (cuLinear.cu:1075-1095; kernels :457-631, :649-854).
 * dX (batch x IN) = dY (batch x OUT) * W (OUT x IN). Overwrite. */
int crb_linear_dgrad(const float *dY, const float *W, float *dX, uint32_t batch, uint32_t IN, uint32_t OUT,
                     void *stream);

/* Replaces seblas::linearParamGrad (cuLinear.cu:1098-1113; kernel :872-1049).
 * dW (OUT x IN) += dY^T * X; dB (OUT) += column sums of dY (each element updated exactly once;
 * dB may be NULL to skip it). Accumulate. */
int crb_linear_wgrad(const float *dY, const float *X, float *dW, float *dB, uint32_t batch, uint32_t IN,
                     uint32_t OUT, void *stream);

/* Convolution family ------------------------------------------------------------------------ */

/* Geometry shared by the three convolution passes. OH/OW are the output-feature extents the caller's
 * tensors have; they must satisfy the relation the reference's assertConv checks
 * (cuConv.cu:731-755): OH == (IH - FH + 2*pH)/sH + 1 and likewise for OW (integer division). */
typedef struct crb_conv_geom {
    uint32_t N;          /* batch */
    uint32_t IC, IH, IW; /* input features  N x IC x IH x IW */
    uint32_t OC, FH, FW; /* filters         OC x IC x FH x FW */
    uint32_t OH, OW;     /* output features N x OC x OH x OW */
    uint32_t sH, sW;     /* strides (>= 1) */
    uint32_t pH, pW;     /* zero padding */
} crb_conv_geom;

/* Replaces seblas::conv (seblas/operations/cuConv.cu:757-770; kernel :32-243).
 * Y[n,oc,oh,ow] = sum_{ic,fh,fw} W[oc,ic,fh,fw] * X[n,ic,oh*sH-pH+fh,ow*sW-pW+fw] (+ bias[oc]);
 * taps outside the image contribute 0; bias may be NULL. Overwrite. flags: CRB_FLAG_*. */
int crb_conv_fwd(const float *W, const float *X, float *Y, const float *bias_or_null, const crb_conv_geom *g,
                 uint32_t flags, void *stream);

/* Replaces seblas::convDerive (cuConv.cu:774-790; kernel :262-483).
 * dX[n,ic,y,x] = sum over (oc,fh,fw) with y+pH-fh = oh*sH, x+pW-fw = ow*sW, 0<=oh<OH, 0<=ow<OW of
 * W[oc,ic,fh,fw] * dY[n,oc,oh,ow]. Overwrite. */
int crb_conv_dgrad(const float *W, const float *dY, float *dX, const crb_conv_geom *g, void *stream);

/* Bytes of split scratch crb_conv_fwd / crb_conv_dgrad need for this geometry (0 for every shape with a kernel of its
 * own; the general implicit-GEMM path cuts short-and-wide contractions). operands_aligned16: whether the activation
 * tensors are 16-byte aligned (hipMalloc'd ones are); other alignments take the general path. Served from the block
 * bound with crb_bind_workspace, else from the library arena. */
size_t crb_conv_fwd_workspace_bytes(const crb_conv_geom *g, int operands_aligned16);
size_t crb_conv_dgrad_workspace_bytes(const crb_conv_geom *g, int operands_aligned16);

/* Bytes of scratch crb_conv_wgrad needs for this geometry with 16-byte aligned tensors (0 if none). */
size_t crb_conv_wgrad_workspace_bytes(const crb_conv_geom *g);

/* Replaces seblas::convError (cuConv.cu:793-806; kernel :488-707).
 * dW[oc,ic,fh,fw] += sum_{n,oh,ow} dY[n,oc,oh,ow] * X[n,ic,oh*sH-pH+fh,ow*sW-pW+fw]. Accumulate.
 * The reduction over n*OH*OW is split across workgroups and combined in a fixed order (no atomics),
 * so results are bit-reproducible. `workspace` may be NULL: the library then uses the block bound to
 * the stream (crb_bind_workspace) or its own lazily grown arena (which may call hipMalloc on first
 * use / growth, and refuses to during a stream capture); otherwise it must be 16-byte aligned
 * and hold at least crb_conv_wgrad_workspace_bytes(g) bytes (CRB_EWORKSPACE if not). */
int crb_conv_wgrad(const float *dY, const float *X, float *dW, const crb_conv_geom *g, void *workspace,
                   size_t workspace_bytes, void *stream);

/* crb_conv_wgrad for callers that cannot allocate and have no workspace to pass: code under HIP graph capture, tight
 * serving or training loops, harnesses that forbid hipMalloc. No counterpart in the reference. Same result as
 * crb_conv_wgrad (bit for bit); the split scratch is a buffer of CRB_NOALLOC_SCRATCH_BYTES built into the library (device
 * memory each GPU the library runs on holds until the process ends), so the call allocates nothing. Geometries whose
 * crb_conv_wgrad_workspace_bytes exceed that size return CRB_EWORKSPACE. Every call on a GPU uses that GPU's one buffer:
 * calls on one stream run in order and are safe; calls that overlap on different streams of one GPU race. */
#define CRB_NOALLOC_SCRATCH_BYTES (8u << 20)
int crb_conv_wgrad_noalloc(const float *dY, const float *X, float *dW, const crb_conv_geom *g, void *stream);

/* Replaces seblas::convBias (cuConv.cu:808-818; kernel :709-729). Y[n,c,:,:] += bias[c], in place. */
int crb_conv_bias(float *Y, const float *bias, uint32_t N, uint32_t C, uint32_t HW, void *stream);

/* Both gradients of a convolution layer in one call: dX as crb_conv_dgrad writes it and dW as crb_conv_wgrad accumulates
 * it (same workspace rule: crb_conv_wgrad_workspace_bytes(g) bytes, or NULL for the library arena). Replaces the pair of
 * calls Conv2D::xGrads / Conv2D::paramGrads make back to back (seann/operands/seblas/Conv2D.cu:18-29: convDerive, then
 * convError): the two are independent, and for the 3x3 layer shapes of CIFAR residual networks (stride 1, and the 16 -> 32
 * stride-2 transition) and the growth-12 layers of dense networks (48 -> 12) they run as one launch that shares the chip;
 * other shapes run the two calls one after the other. Results are identical to the separate calls.
 * dX must not overlap X or dY. */
int crb_conv_bwd(const float *W, const float *dY, const float *X, float *dX, float *dW, const crb_conv_geom *g, void *workspace,
                 size_t workspace_bytes, void *stream);

/* The backward call with the weight gradient's last step postponed, for callers that need dW only when the optimizer
 * runs (no counterpart in the reference). crb_conv_bwd_sliced writes dX as crb_conv_bwd does and leaves the weight
 * gradient of this call as crb_conv_bwd_slices(g) partial sums ("slices", each OC*IC*FH*FW floats, one after the other)
 * in `workspace` (caller-owned, crb_conv_wgrad_workspace_bytes(g) bytes, 16-byte aligned, not shared with another pending
 * call). Geometries with a sliced form: 3x3 / pad 1 layers on the direct kernels, 1x1 / stride 1 layers on the
 * pixel-contraction kernel (at most 64 output channels, at least 16 input channels, whole 64-pixel runs), 1x1 / stride 2
 * shortcuts. crb_conv_bwd_slices returns 0 for geometries without one: use crb_conv_bwd for those.
 * crb_sum_slices_multi then completes any number of such gradients in one launch: for every item,
 * dst[i] += sum over z of slices[z*count + i]; `items` is host memory. The summation order per element is the one
 * crb_conv_wgrad / crb_conv_bwd use internally, so the results are bit-identical to theirs. */
typedef struct crb_slice_sum_item {
    const float *slices;
    float *dst;
    uint32_t count, n_slices;
} crb_slice_sum_item;
uint32_t crb_conv_bwd_slices(const crb_conv_geom *g);
int crb_conv_bwd_sliced(const float *W, const float *dY, const float *X, float *dX, const crb_conv_geom *g, void *workspace,
                        size_t workspace_bytes, void *stream);
int crb_sum_slices_multi(const crb_slice_sum_item *items, uint32_t n_items, void *stream);

/* Bias gradient of a conv operand: dB[c] += sum_{n,h,w} dY[n,c,h,w], each element updated exactly once.
 * Stands in for the channelReduce call of Conv2D::paramGrads (seann/operands/seblas/Conv2D.cu:26-28), whose
 * size assertion (seblas/operations/cuReduce.cu:237) cannot hold for a C-element bias; this computes the
 * per-channel sum that call is meant to produce. Accumulate. */
int crb_conv_bias_grad(const float *dY, float *dB, uint32_t N, uint32_t C, uint32_t HW, void *stream);
/* Bytes of scratch crb_conv_bias_grad needs (partial column sums; from the bound workspace or the library arena). */
size_t crb_conv_bias_grad_workspace_bytes(uint32_t N, uint32_t C, uint32_t HW);

/* Tensor helpers the conv / linear operands use around the hot path ---------------------------- */

/* Replaces the device branch of seblas::Tensor::operator+(Tensor*) (seblas/tensor/Tensor.cu:118-132,
 * 462-483): a[i] += b[i] for i < count, in place. Used by Conv2D::xGrads / Linear::xGrads to fold the
 * reserve gradient into dA (seann/operands/seblas/Conv2D.cu:19). */
int crb_tensor_add_inplace(float *a, const float *b, uint32_t count, void *stream);

/* Replaces the device branch of seblas::Tensor::constFill (Tensor.cu:294-304, 638-657): a[i] = value. */
int crb_tensor_fill(float *a, float value, uint32_t count, void *stream);

/* Device-to-device copy on `stream`: dst[i] = src[i]. Stands in for the cudaMemcpy(..., cudaMemcpyDeviceToDevice) of
 * seblas::Tensor::copyToD2D (seblas/tensor/Tensor.cu:435-440) and of the shortcut operand
 * (seann/operands/controlling/ShortcutEndpoint.cu:59-60,80-81,96-97) without stalling the host. */
int crb_tensor_copy(float *dst, const float *src, uint32_t count, void *stream);

/* a[i] += b[i]; b[i] = 0. The pair every operand's xGrads performs around its gradient call — `*Y->dA + Y->dAReserve`
 * ... `Y->dAReserve->constFill(0)` (e.g. seann/operands/seblas/Conv2D.cu:19,21) — in one pass. The two must not alias. */
int crb_tensor_add_clear(float *a, float *b, uint32_t count, void *stream);

/* The closing shortcut endpoint with the ReLU that follows it (no counterpart in the reference: ShortcutEndpoint.cu:57-99
 * and ReLU.cu:8-17 are separate operands). crb_tensor_add_relu: dst = max(a + b, 0). crb_tensor_relu_grad_copy2:
 * dst1 = dst2 = (relu_out > 0 ? dY (+ dY2 when given) : 0), the ReLU's gradient delivered to the main path and to the
 * shortcut at once. */
int crb_tensor_add_relu(float *dst, const float *a, const float *b, uint32_t count, void *stream);
int crb_tensor_relu_grad_copy2(float *dst1, float *dst2, const float *relu_out, const float *dY, const float *dY2_or_null, uint32_t count,
                               void *stream);

/* Fused forms of the copies and adds the shortcut operand performs (seann/operands/controlling/ShortcutEndpoint.cu):
 *   crb_tensor_add:             dst = a + b           (forward of the closing endpoint, :59-73: copy then add; dst may be a)
 *   crb_tensor_add_clear_copy:  a += b; b = 0; dst = a (backward of the opening endpoint, :92-97: fold the reserve, copy on)
 *   crb_tensor_copy2:           dst1 = src; dst2 = src (backward of an identity closing endpoint, :88-89,96-97: two copies) */
int crb_tensor_add(float *dst, const float *a, const float *b, uint32_t count, void *stream);
int crb_tensor_add_clear_copy(float *dst, float *a, float *b, uint32_t count, void *stream);
int crb_tensor_copy2(float *dst1, float *dst2, const float *src, uint32_t count, void *stream);

/* Replaces the device branch of seblas::Tensor::operator-(Tensor*) (Tensor.cu:485-506): a[i] -= b[i], in place. */
int crb_tensor_sub_inplace(float *a, const float *b, uint32_t count, void *stream);

/* Replaces the device branch of seblas::Tensor::operator*(float) (Tensor.cu:596-617): a[i] *= factor, in place.
 * The optimizers use it for L2 weight decay, `*A->A * (1 - L2)` (seann/optimizers/Optimizers.cu:10,18). */
int crb_tensor_scale_inplace(float *a, float factor, uint32_t count, void *stream);

/* Elementwise and reduction operators of a training step (the callers around the GEMM / conv path) ----------- */

/* Replaces seblas::relu (seblas/operations/cuActivation.cu:268-280; kernels :14-19, :28-39): Y = max(X, 0). */
int crb_relu_fwd(const float *X, float *Y, uint32_t count, void *stream);

/* Replaces seblas::reluGradFast (cuActivation.cu:296-308; kernels :54-59, :61-76): dX = X > 0 ? dY : 0. */
int crb_relu_bwd(const float *X, const float *dY, float *dX, uint32_t count, void *stream);

/* Replaces seblas::maxPool (seblas/operations/cuPool.cu:135-143; kernel :8-40). X: planes x IH x IW (planes = n*c),
 * Y: planes x IH/rH x IW/rW, record: planes x (IH/rH)*rH x (IW/rW)*rW. Y = window maximum (first maximum in row-major
 * window order, start value -1e15); record = 1 at that element, 0 elsewhere in the window (the reference writes
 * only the 1 and relies on the rest being 0). Only stride == range (non-overlapping windows), the one case the
 * reference's plane-offset arithmetic addresses correctly; anything else returns CRB_EINVAL_SHAPE. */
int crb_maxpool_fwd(const float *X, float *Y, float *record, uint32_t planes, uint32_t IH, uint32_t IW, uint32_t sH,
                    uint32_t sW, uint32_t rH, uint32_t rW, void *stream);

/* Replaces seblas::maxPoolBack (cuPool.cu:145-151; kernel :42-70): per window, the element holding the first maximum
 * of `record` receives dY and that record entry is cleared. Every other element of dX is written as 0 (the reference
 * leaves them untouched, i.e. at the 0 the gradient tensor was created with). */
int crb_maxpool_bwd(float *dX, const float *dY, float *record, uint32_t planes, uint32_t IH, uint32_t IW, uint32_t sH,
                    uint32_t sW, uint32_t rH, uint32_t rW, void *stream);

/* Replaces seblas::softmax (seblas/operations/cuReduce.cu:296-357; kernel :98-146): for each of `rows` consecutive
 * groups of `step` elements, out = exp(a - max) / (sum exp(a - max) + 1e-10). Any step; no buffer needed. */
int crb_softmax(const float *A, float *out, uint32_t rows, uint32_t step, void *stream);

/* Replaces seblas::crossEntropyLoss (seblas/operations/cuLoss.cu:231-234): dY = Y - labels. */
int crb_cross_entropy_grad(const float *Y, const float *labels, float *dY, uint32_t count, void *stream);

/* Replaces seblas::crossEntropyCalc (cuLoss.cu:220-228; kernel :31-37): *loss_out (device) = sum over all elements of
 * -log(Y + 1e-10) * label, summed in a fixed order. `scratch` must hold crb_cross_entropy_scratch_floats(count)
 * floats (the reference's `buf`, which has Y's size, always does); it may be null when that is 1. */
uint32_t crb_cross_entropy_scratch_floats(uint32_t count);
int crb_cross_entropy_loss(const float *Y, const float *labels, float *scratch, uint32_t scratch_floats, float *loss_out,
                           uint32_t count, void *stream);

/* Replaces seann::Momentum::apply (seann/optimizers/Optimizers.cu:16-22) = weight decay `A *= decay` followed by
 * seblas::momentumApply (seblas/operations/cuOptim.cu:259-272; kernels :38-46, :48-73), in one pass:
 *   x = x*decay;  m = beta*m + (1-beta)*g;  x -= lr*m;  g = 0.   decay = 1 - L2 for weights, 1 otherwise. */
int crb_momentum_apply(float *X, float *G, float *M, uint32_t count, float lr, float beta, float decay, void *stream);

/* The same step for a whole table of parameter tensors in ONE launch (a network has hundreds of small ones and a launch
 * per tensor is then launch-bound). `items_on_device` is a device array of n_items entries, built and kept by the caller;
 * max_count = the largest `count` in it. No counterpart in the reference, which launches per parameter
 * (seann/containers/Sequential.cu:93-97 -> updateParams -> Optimizer::apply). Arithmetic identical to crb_momentum_apply. */
typedef struct crb_momentum_item {
    float *X, *G, *M;
    uint32_t count;
    float lr, beta, decay;
} crb_momentum_item;
int crb_momentum_apply_multi(const crb_momentum_item *items_on_device, uint32_t n_items, uint32_t max_count, void *stream);

/* Batch normalisation with per-feature statistics: X is N x F, F = c*h*w, and each of the F positions is normalised
 * over the N samples (biased variance, eps 1e-8); beta, gamma, mean, var hold F floats.
 * Replaces seblas::batchNorm (seblas/operations/cuBatchNorm.cu:150-164; kernel :13-61): Y = xHat*gamma + beta, and
 * mean, var, xHat are stored. The reference's N <= 96 limit (:9,164) does not apply. */
int crb_batchnorm_fwd(const float *X, const float *beta, const float *gamma, float *mean, float *var, float *Y, float *xHat,
                      uint32_t N, uint32_t F, void *stream);

/* Replaces seblas::batchNormGrad (cuBatchNorm.cu:167-178; kernel :63-125): dX from dY, gamma and X (statistics are
 * recomputed from X, as in the reference). When dGamma / dBeta are given (both or neither) the parameter gradients are
 * written too — they are by-products of the same sums (dBeta = sum dY, dGamma = sum dY*xHat) — which saves the separate
 * crb_batchnorm_param_grads pass. */
int crb_batchnorm_bwd(const float *dY, const float *gamma, const float *X, float *dX, float *dGamma_or_null, float *dBeta_or_null,
                      uint32_t N, uint32_t F, void *stream);

/* Batch normalisation with the ReLU that follows it, in one pass each way (no counterpart in the reference, where
 * BatchNorm, ShortcutEndpoint and ReLU are separate operands: seann/operands/seblas/BatchNorm.cu:13-21,
 * controlling/ShortcutEndpoint.cu:57-99, activate/ReLU.cu:8-17).
 * Forward: what crb_batchnorm_fwd computes, plus reluOut = max(Y + addend, 0); addend (or NULL) is the other summand of a
 * residual connection that closes between the normalisation and the ReLU; Y and xHat are written only when given.
 * Backward: dY (+ dY2 when given: the gradient arrives in two parts, as it does when a residual connection opens right
 * behind the ReLU) is the gradient with respect to reluOut; the gradient reaching the normalisation is that sum where
 * reluOut > 0 and 0 elsewhere (reluGradFast's rule, since reluOut > 0 exactly where the ReLU's input is), then
 * crb_batchnorm_bwd. dYmasked, when given, receives that masked gradient (what the closing residual connection hands to
 * its shortcut). Results are bit-identical to the separate calls. */
int crb_batchnorm_relu_fwd(const float *X, const float *beta, const float *gamma, float *mean, float *var, float *Y_or_null,
                           float *xHat_or_null, const float *addend_or_null, float *reluOut, uint32_t N, uint32_t F, void *stream);
int crb_batchnorm_relu_bwd(const float *dY, const float *dY2_or_null, const float *reluOut, const float *gamma, const float *X, float *dX,
                           float *dGamma_or_null, float *dBeta_or_null, float *dYmasked_or_null, uint32_t N, uint32_t F, void *stream);

/* Replaces seblas::batchNormParamGrads (cuBatchNorm.cu:180-191; kernel :127-147): dBeta = sum_n dY, dGamma = sum_n dY*xHat.
 * Both are overwritten, not accumulated. */
int crb_batchnorm_param_grads(const float *dY, const float *xHat, float *dGamma, float *dBeta, uint32_t N, uint32_t F,
                              void *stream);

/* Dataset bytes to network input. src holds `images` images of `channels` planes of H x W byte pixels, as they lie in a
 * dataset file; dst receives the same images as floats, normalised per image:
 *   CRB_NORM_NONE          dst = (float) src                                  (seio/data/DataLoader.cu:34-36)
 *   CRB_NORM_UNIFORM       (x - min) / (max - min) * (p1 - p0) + p0, p0 = desiredMin, p1 = desiredMax, with the extrema
 *                          of channel k taken over channels 0..k of the image, as UniformNorm::apply computes them
 *                          (seio/data/DataTransform.cu:29-44)
 *   CRB_NORM_DISTRIBUTION  (x - mean) * p1 / sqrt(var + 1e-8) + p0, p0 = desiredMean, p1 = desiredVar, per channel,
 *                          biased variance (DistribNorm::apply, DataTransform.cu:7-27)
 * aug_on_device, when not null, holds one record per image (device memory): with CRB_AUG_MIRROR the image is mirrored
 * along its width (the effect RandFlipW::apply is written for, seio/data/DataAugmentor.cu:64-104); with CRB_AUG_SHIFT the
 * output pixel (h, w) is the (mirrored) pixel (h + dh, w + dw) where 0 < h + dh < H and 0 < w + dw < W and 0 elsewhere
 * (RandCorp::apply, DataAugmentor.cu:26-62, comparisons as written there). Normalisation statistics are those of the
 * whole stored image, as in the reference, where the transforms run before the augmentations (Dataset.cu:65-72).
 * Replaces the per-image host loops of Dataset::genBatch (seio/data/Dataset.cu:63-85) and the float upload that follows
 * them: the batch is uploaded as bytes and converted here. channels <= 64. */
enum { CRB_NORM_NONE = 0, CRB_NORM_UNIFORM = 1, CRB_NORM_DISTRIBUTION = 2 };
enum { CRB_AUG_MIRROR = 1, CRB_AUG_SHIFT = 2 };
typedef struct crb_image_aug {
    int32_t dh, dw;
    uint32_t flags;
} crb_image_aug;
int crb_images_from_bytes(const uint8_t *src, float *dst, uint32_t images, uint32_t channels, uint32_t H, uint32_t W, int norm,
                          float p0, float p1, const crb_image_aug *aug_on_device, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* CRUSADER_HIP_H */
