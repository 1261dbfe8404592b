// Elementwise helpers the operands call around the hot path: in-place add, add-and-clear, copy and constant fill.
// Pure streaming kernels (HBM-bound): 16-byte accesses when the buffer is 16-byte aligned, grid-stride loop.
#include "igemm_engine.h"

namespace crb {

__global__ void __launch_bounds__(256) add_inplace_kernel(float *__restrict__ a, const float *__restrict__ b, u32 count,
                                                          u32 vec) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const u32 nq = count / 4;
        v4f *a4 = reinterpret_cast<v4f *>(a);
        const v4f *b4 = reinterpret_cast<const v4f *>(b);
        for (u32 q = i; q < nq; q += stride) a4[q] = a4[q] + b4[q];
        for (u32 r = nq * 4 + i; r < count; r += stride) a[r] += b[r];
    } else {
        for (; i < count; i += stride) a[i] += b[i];
    }
}

__global__ void __launch_bounds__(256) fill_kernel(float *__restrict__ a, float value, u32 count, u32 vec) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const u32 nq = count / 4;
        v4f *a4 = reinterpret_cast<v4f *>(a);
        const v4f v = {value, value, value, value};
        for (u32 q = i; q < nq; q += stride) a4[q] = v;
        for (u32 r = nq * 4 + i; r < count; r += stride) a[r] = value;
    } else {
        for (; i < count; i += stride) a[i] = value;
    }
}

// a[i] += b[i]; b[i] = 0 — folds a side gradient into the main one and clears it, in one pass.
__global__ void __launch_bounds__(256) add_clear_kernel(float *__restrict__ a, float *__restrict__ b, u32 count, u32 vec) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const u32 nq = count / 4;
        v4f *a4 = reinterpret_cast<v4f *>(a), *b4 = reinterpret_cast<v4f *>(b);
        const v4f z = {0.f, 0.f, 0.f, 0.f};
        for (u32 q = i; q < nq; q += stride) {
            a4[q] = a4[q] + b4[q];
            b4[q] = z;
        }
        for (u32 r = nq * 4 + i; r < count; r += stride) a[r] += b[r], b[r] = 0.f;
    } else {
        for (; i < count; i += stride) a[i] += b[i], b[i] = 0.f;
    }
}

__global__ void __launch_bounds__(256) copy_kernel(float *__restrict__ dst, const float *__restrict__ src, u32 count, u32 vec) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const u32 nq = count / 4;
        for (u32 q = i; q < nq; q += stride) reinterpret_cast<v4f *>(dst)[q] = reinterpret_cast<const v4f *>(src)[q];
        for (u32 r = nq * 4 + i; r < count; r += stride) dst[r] = src[r];
    } else {
        for (; i < count; i += stride) dst[i] = src[i];
    }
}

// Three-operand streaming forms used by the residual-connection operand. MODE 0: d = a + b. MODE 1: a += b; b = 0; d = a.
// MODE 2: d = a; b = a (one source, two destinations). MODE 3: d = max(a + b, 0).
__device__ __forceinline__ float relu_of(float v) { return v > 0.f ? v : 0.f; }
__device__ __forceinline__ v4f relu_of(v4f v) { return v4f{relu_of(v.x), relu_of(v.y), relu_of(v.z), relu_of(v.w)}; }

template <int MODE>
__global__ void __launch_bounds__(256) tri_kernel(float *d, float *a, float *b, u32 count, u32 vec) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    auto one = [&](auto *pd, auto *pa, auto *pb, u32 k, auto zero) {
        if (MODE == 0) {
            pd[k] = pa[k] + pb[k];
        } else if (MODE == 1) {
            const auto v = pa[k] + pb[k];
            pa[k] = v, pb[k] = zero, pd[k] = v;
        } else if (MODE == 2) {
            const auto v = pa[k];
            pd[k] = v, pb[k] = v;
        } else {
            pd[k] = relu_of(pa[k] + pb[k]);
        }
    };
    if (vec) {
        const u32 nq = count / 4;
        const v4f z4 = {0.f, 0.f, 0.f, 0.f};
        for (u32 q = i; q < nq; q += stride) one(reinterpret_cast<v4f *>(d), reinterpret_cast<v4f *>(a), reinterpret_cast<v4f *>(b), q, z4);
        for (u32 r = nq * 4 + i; r < count; r += stride) one(d, a, b, r, 0.f);
    } else {
        for (; i < count; i += stride) one(d, a, b, i, 0.f);
    }
}

// d1 = d2 = (mask > 0 ? src (+ src2) : 0): the gradient behind a ReLU whose output is `mask`, delivered to two consumers;
// with src2 the gradient arrives in two parts that are added first.
template <bool SUM2>
__global__ void __launch_bounds__(256) relu_grad_copy2_kernel(float *d1, float *d2, const float *mask, const float *src, const float *src2,
                                                              u32 count, u32 vec) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    auto pick = [](float m, float v) { return m > 0.f ? v : 0.f; };
    if (vec) {
        const u32 nq = count / 4;
        for (u32 q = i; q < nq; q += stride) {
            const v4f m = reinterpret_cast<const v4f *>(mask)[q];
            v4f v = reinterpret_cast<const v4f *>(src)[q];
            if (SUM2) v = v + reinterpret_cast<const v4f *>(src2)[q];
            const v4f r = {pick(m.x, v.x), pick(m.y, v.y), pick(m.z, v.z), pick(m.w, v.w)};
            reinterpret_cast<v4f *>(d1)[q] = r, reinterpret_cast<v4f *>(d2)[q] = r;
        }
        for (u32 k = nq * 4 + i; k < count; k += stride) d1[k] = d2[k] = pick(mask[k], SUM2 ? src[k] + src2[k] : src[k]);
    } else {
        for (; i < count; i += stride) d1[i] = d2[i] = pick(mask[i], SUM2 ? src[i] + src2[i] : src[i]);
    }
}

static u32 stream_grid(u32 count) {
    u32 blocks = ceil_div(ceil_div(count, 4), 256);
    return blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
}

template <int MODE>
static int launch_tri(float *d, float *a, float *b, uint32_t count, void *stream, const char *what) {
    if (!d || !a || !b) return fail(CRB_ENULL, "%s: null operand", what);
    if (!count) return fail(CRB_EINVAL_SHAPE, "%s: zero size", what);
    const u32 vec = ((reinterpret_cast<uintptr_t>(d) | reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
    hipLaunchKernelGGL((tri_kernel<MODE>), dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), d, a, b, count, vec);
    return check_launch(what);
}

}  // namespace crb

using namespace crb;

extern "C" {

int crb_tensor_add_inplace(float *a, const float *b, uint32_t count, void *stream) {
    if (!a || !b) return fail(CRB_ENULL, "crb_tensor_add_inplace: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_add_inplace: zero size");
    const u32 vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
    hipLaunchKernelGGL(add_inplace_kernel, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), a, b, count, vec);
    return check_launch("crb_tensor_add_inplace");
}

int crb_tensor_add_clear(float *a, float *b, uint32_t count, void *stream) {
    if (!a || !b) return fail(CRB_ENULL, "crb_tensor_add_clear: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_add_clear: zero size");
    if (a == b) return fail(CRB_EINVAL_SHAPE, "crb_tensor_add_clear: operands alias");
    const u32 vec = ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b)) & 15u) == 0;
    hipLaunchKernelGGL(add_clear_kernel, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), a, b, count, vec);
    return check_launch("crb_tensor_add_clear");
}

int crb_tensor_copy(float *dst, const float *src, uint32_t count, void *stream) {
    if (!dst || !src) return fail(CRB_ENULL, "crb_tensor_copy: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_copy: zero size");
    if (dst == src) return CRB_OK;
    const u32 vec = ((reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(src)) & 15u) == 0;
    hipLaunchKernelGGL(copy_kernel, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), dst, src, count, vec);
    return check_launch("crb_tensor_copy");
}

int crb_tensor_add(float *dst, const float *a, const float *b, uint32_t count, void *stream) {
    return launch_tri<0>(dst, const_cast<float *>(a), const_cast<float *>(b), count, stream, "crb_tensor_add");
}

int crb_tensor_add_relu(float *dst, const float *a, const float *b, uint32_t count, void *stream) {
    return launch_tri<3>(dst, const_cast<float *>(a), const_cast<float *>(b), count, stream, "crb_tensor_add_relu");
}

int crb_tensor_relu_grad_copy2(float *dst1, float *dst2, const float *relu_out, const float *dY, const float *dY2_or_null, uint32_t count,
                               void *stream) {
    if (!dst1 || !dst2 || !relu_out || !dY) return fail(CRB_ENULL, "crb_tensor_relu_grad_copy2: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_relu_grad_copy2: zero size");
    const u32 vec = ((reinterpret_cast<uintptr_t>(dst1) | reinterpret_cast<uintptr_t>(dst2) | reinterpret_cast<uintptr_t>(relu_out) |
                      reinterpret_cast<uintptr_t>(dY) | reinterpret_cast<uintptr_t>(dY2_or_null)) & 15u) == 0;
    if (dY2_or_null)
        hipLaunchKernelGGL(relu_grad_copy2_kernel<true>, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), dst1, dst2, relu_out, dY,
                           dY2_or_null, count, vec);
    else
        hipLaunchKernelGGL(relu_grad_copy2_kernel<false>, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), dst1, dst2, relu_out, dY,
                           dY2_or_null, count, vec);
    return check_launch("crb_tensor_relu_grad_copy2");
}

int crb_tensor_add_clear_copy(float *dst, float *a, float *b, uint32_t count, void *stream) {
    if (a == b || dst == b) return fail(CRB_EINVAL_SHAPE, "crb_tensor_add_clear_copy: operands alias");
    return launch_tri<1>(dst, a, b, count, stream, "crb_tensor_add_clear_copy");
}

int crb_tensor_copy2(float *dst1, float *dst2, const float *src, uint32_t count, void *stream) {
    return launch_tri<2>(dst1, const_cast<float *>(src), dst2, count, stream, "crb_tensor_copy2");
}

int crb_tensor_fill(float *a, float value, uint32_t count, void *stream) {
    if (!a) return fail(CRB_ENULL, "crb_tensor_fill: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_fill: zero size");
    const u32 vec = (reinterpret_cast<uintptr_t>(a) & 15u) == 0;
    hipLaunchKernelGGL(fill_kernel, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), a, value, count, vec);
    return check_launch("crb_tensor_fill");
}

}  // extern "C"
