// Internal entry points of the GEMM translation unit used by the convolution dispatcher (1x1 convolutions are
// batched GEMMs on the native NCHW layout).
#pragma once
#include "crb_common.h"

namespace crb {
// For nd < batch: C[nd] (M x N) = A (M x K) * B[nd] (K x N) (+ row_bias[m]) (ReLU if flags has EPI_RELU).
int gemm_nn_rowbias(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, u32 batch, const float *row_bias, u32 flags,
                    hipStream_t s, const char *what);
// For nd < batch: C[nd] (M x N) = A^T * B[nd], A stored K x M.
int gemm_tn_batched(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, u32 batch, hipStream_t s, const char *what);
// 3x3 / pad 1 / stride 1 convolution on 2x2 images (every input pixel reaches every output pixel through one tap):
// dense products over (channel, pixel) pairs. All tensors 16-byte aligned. dW is accumulated.
int conv2x2_fwd(const float *W, const float *X, float *Y, const float *bias, u32 N, u32 IC, u32 OC, u32 flags, hipStream_t s,
                const char *what);
int conv2x2_dgrad(const float *W, const float *dY, float *dX, u32 N, u32 IC, u32 OC, hipStream_t s, const char *what);
// G: scratch of OC*4 x IC*4 floats.
// Scratch bytes the GEMM family asks for on a dense M x N result per batch entry with contraction length K (0: none).
// one_launch_form = false: the caller goes to the tiled engine directly and never takes the one-launch small-product kernel
// (the 2x2-image convolutions), so the split plan of the tiles applies whatever the size.
size_t gemm_scratch_bytes(u32 M, u32 N, u32 K, u32 zdim, bool one_launch_form = true);
int conv2x2_wgrad(const float *dY, const float *X, float *dW, float *G, u32 N, u32 IC, u32 OC, hipStream_t s, const char *what);
}  // namespace crb
