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
}  // namespace crb
