// Elementwise and small reduction operators that sit between the GEMM / convolution calls of a training step:
// ReLU and its gradient, max pooling (non-overlapping windows) and its gradient, row softmax, cross-entropy value and
// gradient, in-place subtract / scale, the momentum update with weight decay, and per-feature batch normalisation.
// All are HBM-bound streaming kernels: 16-byte accesses where alignment allows, grid-stride loops, and reductions
// with a fixed association (bit-reproducible, no atomics).
#include <type_traits>
#include "igemm_engine.h"

namespace crb {

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static u32 stream_grid(u32 count) {
    u32 blocks = ceil_div(ceil_div(count, 4), 256);
    return blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
}

// out[i] = f(in0[i], in1[i]) over `count` floats; quads when `vec`, scalars for the tail / unaligned buffers.
// (no __restrict__: the in-place forms pass the same buffer as input and output)
template <class F>
__global__ void __launch_bounds__(256) map2_kernel(const float *a, const float *b, float *o,
                                                   u32 count, u32 vec, F f) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const u32 nq = count / 4;
        for (u32 q = i; q < nq; q += stride) {
            const v4f x = reinterpret_cast<const v4f *>(a)[q];
            const v4f y = b ? reinterpret_cast<const v4f *>(b)[q] : v4f{0.f, 0.f, 0.f, 0.f};
            reinterpret_cast<v4f *>(o)[q] = v4f{f(x.x, y.x), f(x.y, y.y), f(x.z, y.z), f(x.w, y.w)};
        }
        for (u32 r = nq * 4 + i; r < count; r += stride) o[r] = f(a[r], b ? b[r] : 0.f);
    } else {
        for (; i < count; i += stride) o[i] = f(a[i], b ? b[i] : 0.f);
    }
}

struct ReluF {
    __device__ float operator()(float x, float) const { return x > 0.f ? x : 0.f; }
};
struct ReluGradF {  // (x, dy) -> dx
    __device__ float operator()(float x, float dy) const { return x > 0.f ? dy : 0.f; }
};
struct SubF {
    __device__ float operator()(float a, float b) const { return a - b; }
};
struct ScaleF {
    float s;
    __device__ float operator()(float a, float) const { return a * s; }
};

template <class F>
static int launch_map2(const float *a, const float *b, float *o, u32 count, F f, hipStream_t s, const char *what) {
    const u32 vec = aligned16(a) && aligned16(o) && (!b || aligned16(b));
    hipLaunchKernelGGL((map2_kernel<F>), dim3(stream_grid(count)), dim3(256), 0, s, a, b, o, count, vec, f);
    return check_launch(what);
}

// ---- max pooling, windows rH x rW, stride = window ------------------------------------------------------------------
// One thread per window. X plane IH x IW; record plane RH x RW = (OH*rH) x (OW*rW). The first maximum in row-major
// window order wins (strict '>', start value -1e15).
__global__ void __launch_bounds__(256) maxpool_fwd_kernel(const float *__restrict__ X, float *__restrict__ Y, float *__restrict__ rec,
                                                          u32 windows, u32 IH, u32 IW, u32 rH, u32 rW, FastDiv ow_div,
                                                          FastDiv oh_div) {
    const u32 w = blockIdx.x * 256 + threadIdx.x;
    if (w >= windows) return;
    u32 t, ow, p, oh;
    ow_div.divmod(w, t, ow);
    oh_div.divmod(t, p, oh);
    const u32 OH = oh_div.d, OW = ow_div.d;
    const float *x = X + (size_t(p) * IH + oh * rH) * IW + ow * rW;
    float best = -1e15f;
    u32 bi = 0, bj = 0;
    for (u32 i = 0; i < rH; ++i)
        for (u32 j = 0; j < rW; ++j) {
            const float v = x[i * IW + j];
            if (v > best) best = v, bi = i, bj = j;
        }
    float *r = rec + (size_t(p) * OH * rH + oh * rH) * (OW * rW) + ow * rW;
    for (u32 i = 0; i < rH; ++i)
        for (u32 j = 0; j < rW; ++j) r[i * (OW * rW) + j] = (i == bi && j == bj) ? 1.f : 0.f;
    Y[w] = best;
}

// 2x2 windows on rows of even length with 16-byte aligned planes: one thread per pair of horizontally adjacent
// windows, i.e. one quad of each of the two input rows.
__global__ void __launch_bounds__(256) maxpool2x2_fwd_kernel(const float *__restrict__ X, float *__restrict__ Y,
                                                             float *__restrict__ rec, u32 pairs, u32 IW, FastDiv qdiv) {
    const u32 e = blockIdx.x * 256 + threadIdx.x;  // (plane*OH + oh, quad)
    if (e >= pairs) return;
    u32 row, q;
    qdiv.divmod(e, row, q);
    const float *x = X + size_t(row) * 2 * IW + 4 * q;
    const v4f a = *reinterpret_cast<const v4f *>(x), b = *reinterpret_cast<const v4f *>(x + IW);
    v4f ra = {0.f, 0.f, 0.f, 0.f}, rb = ra;
    float y[2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const float v00 = h ? a.z : a.x, v01 = h ? a.w : a.y, v10 = h ? b.z : b.x, v11 = h ? b.w : b.y;
        float best = -1e15f;
        int k = 0;
        if (v00 > best) best = v00, k = 0;
        if (v01 > best) best = v01, k = 1;
        if (v10 > best) best = v10, k = 2;
        if (v11 > best) best = v11, k = 3;
        y[h] = best;
        if (h == 0) ra.x = k == 0, ra.y = k == 1, rb.x = k == 2, rb.y = k == 3;
        else ra.z = k == 0, ra.w = k == 1, rb.z = k == 2, rb.w = k == 3;
    }
    float *r = rec + size_t(row) * 2 * IW + 4 * q;  // record has the extent of X here (IH, IW even)
    *reinterpret_cast<v4f *>(r) = ra;
    *reinterpret_cast<v4f *>(r + IW) = rb;
    *reinterpret_cast<v2f *>(Y + size_t(row) * (IW / 2) + 2 * q) = v2f{y[0], y[1]};
}

// One thread per window: the first maximum of the record window receives dY, the rest of the window 0; the used
// record entry is cleared.
__global__ void __launch_bounds__(256) maxpool_bwd_kernel(float *__restrict__ dX, const float *__restrict__ dY, float *__restrict__ rec,
                                                          u32 windows, u32 IH, u32 IW, u32 rH, u32 rW, FastDiv ow_div,
                                                          FastDiv oh_div) {
    const u32 w = blockIdx.x * 256 + threadIdx.x;
    if (w >= windows) return;
    u32 t, ow, p, oh;
    ow_div.divmod(w, t, ow);
    oh_div.divmod(t, p, oh);
    const u32 OH = oh_div.d, OW = ow_div.d;
    float *r = rec + (size_t(p) * OH * rH + oh * rH) * (OW * rW) + ow * rW;
    float best = -1e15f;
    u32 bi = 0, bj = 0;
    for (u32 i = 0; i < rH; ++i)
        for (u32 j = 0; j < rW; ++j) {
            const float v = r[i * (OW * rW) + j];
            if (v > best) best = v, bi = i, bj = j;
        }
    const float g = dY[w];
    float *x = dX + (size_t(p) * IH + oh * rH) * IW + ow * rW;
    for (u32 i = 0; i < rH; ++i)
        for (u32 j = 0; j < rW; ++j) x[i * IW + j] = (i == bi && j == bj) ? g : 0.f;
    r[bi * (OW * rW) + bj] = 0.f;
}

__global__ void __launch_bounds__(256) maxpool2x2_bwd_kernel(float *__restrict__ dX, const float *__restrict__ dY,
                                                             float *__restrict__ rec, u32 pairs, u32 IW, FastDiv qdiv) {
    const u32 e = blockIdx.x * 256 + threadIdx.x;
    if (e >= pairs) return;
    u32 row, q;
    qdiv.divmod(e, row, q);
    float *r = rec + size_t(row) * 2 * IW + 4 * q;
    v4f ra = *reinterpret_cast<const v4f *>(r), rb = *reinterpret_cast<const v4f *>(r + IW);
    const v2f g = *reinterpret_cast<const v2f *>(dY + size_t(row) * (IW / 2) + 2 * q);
    v4f xa = {0.f, 0.f, 0.f, 0.f}, xb = xa;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const float v00 = h ? ra.z : ra.x, v01 = h ? ra.w : ra.y, v10 = h ? rb.z : rb.x, v11 = h ? rb.w : rb.y;
        float best = -1e15f;
        int k = 0;
        if (v00 > best) best = v00, k = 0;
        if (v01 > best) best = v01, k = 1;
        if (v10 > best) best = v10, k = 2;
        if (v11 > best) best = v11, k = 3;
        const float gv = h ? g.y : g.x;
        if (h == 0) {
            xa.x = k == 0 ? gv : 0.f, xa.y = k == 1 ? gv : 0.f, xb.x = k == 2 ? gv : 0.f, xb.y = k == 3 ? gv : 0.f;
            if (k == 0) ra.x = 0.f; else if (k == 1) ra.y = 0.f; else if (k == 2) rb.x = 0.f; else rb.y = 0.f;
        } else {
            xa.z = k == 0 ? gv : 0.f, xa.w = k == 1 ? gv : 0.f, xb.z = k == 2 ? gv : 0.f, xb.w = k == 3 ? gv : 0.f;
            if (k == 0) ra.z = 0.f; else if (k == 1) ra.w = 0.f; else if (k == 2) rb.z = 0.f; else rb.w = 0.f;
        }
    }
    float *x = dX + size_t(row) * 2 * IW + 4 * q;
    *reinterpret_cast<v4f *>(x) = xa;
    *reinterpret_cast<v4f *>(x + IW) = xb;
    *reinterpret_cast<v4f *>(r) = ra;
    *reinterpret_cast<v4f *>(r + IW) = rb;
}

// ---- block-wide reductions with a fixed association (256 threads) ------------------------------------------------------
template <bool MAX>
__device__ __forceinline__ float block_reduce(float v, float *sh) {
    const u32 t = threadIdx.x;
    sh[t] = v;
    __syncthreads();
#pragma unroll
    for (u32 s = 128; s > 0; s >>= 1) {
        if (t < s) sh[t] = MAX ? (sh[t] > sh[t + s] ? sh[t] : sh[t + s]) : sh[t] + sh[t + s];
        __syncthreads();
    }
    const float r = sh[0];
    __syncthreads();
    return r;
}

// Row softmax: out = exp(a - max) / (sum exp(a - max) + 1e-10). One workgroup per row (any row length).
__global__ void __launch_bounds__(256) softmax_rows_kernel(const float *__restrict__ A, float *__restrict__ out, u32 step) {
    __shared__ float sh[256];
    const float *a = A + size_t(blockIdx.x) * step;
    float *o = out + size_t(blockIdx.x) * step;
    float mx = -1e15f;
    for (u32 i = threadIdx.x; i < step; i += 256) mx = a[i] > mx ? a[i] : mx;
    mx = block_reduce<true>(mx, sh);
    float sum = 0.f;
    for (u32 i = threadIdx.x; i < step; i += 256) {
        const float e = expf(a[i] - mx);
        o[i] = e;
        sum += e;
    }
    sum = block_reduce<false>(sum, sh);
    const float den = sum + 1e-10f;
    for (u32 i = threadIdx.x; i < step; i += 256) o[i] = o[i] / den;
}

// Short rows (step <= 64): one wave per row, 4 rows per workgroup, lanes reduced with cross-lane shuffles in a
// fixed butterfly order.
__global__ void __launch_bounds__(256) softmax_short_kernel(const float *__restrict__ A, float *__restrict__ out, u32 rows, u32 step) {
    const u32 row = blockIdx.x * 4 + threadIdx.x / 64, lane = threadIdx.x % 64;
    if (row >= rows) return;
    const bool on = lane < step;
    const float v = on ? A[size_t(row) * step + lane] : -1e15f;
    float mx = v;
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) {
        const float other = __shfl_xor(mx, m, 64);
        mx = other > mx ? other : mx;
    }
    const float e = on ? expf(v - mx) : 0.f;
    float sum = e;
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) sum += __shfl_xor(sum, m, 64);
    if (on) out[size_t(row) * step + lane] = e / (sum + 1e-10f);
}

// ---- cross-entropy value: sum of -log(y + 1e-10) * label --------------------------------------------------------------
// Stage 1: workgroup b sums elements b*chunk .. (b+1)*chunk - 1 (thread-strided, then the fixed tree) into part[b].
// Stage 2 (or the only stage when one workgroup covers everything): sums part[] the same way into *loss.
__global__ void __launch_bounds__(256) ce_partial_kernel(const float *__restrict__ Y, const float *__restrict__ L,
                                                         float *__restrict__ part, u32 count, u32 chunk) {
    __shared__ float sh[256];
    const u32 lo = blockIdx.x * chunk, hi = lo + chunk < count ? lo + chunk : count;
    float s = 0.f;
    for (u32 i = lo + threadIdx.x; i < hi; i += 256) s += -logf(Y[i] + 1e-10f) * L[i];
    s = block_reduce<false>(s, sh);
    if (threadIdx.x == 0) part[blockIdx.x] = s;
}

__global__ void __launch_bounds__(256) sum_small_kernel(const float *__restrict__ part, float *__restrict__ out, u32 n) {
    __shared__ float sh[256];
    float s = 0.f;
    for (u32 i = threadIdx.x; i < n; i += 256) s += part[i];
    s = block_reduce<false>(s, sh);
    if (threadIdx.x == 0) out[0] = s;
}

// ---- momentum step with weight decay -------------------------------------------------------------------------------------
// x = x*decay; m = beta*m + (1-beta)*g; x -= lr*m; g = 0. Every product and sum is rounded on its own (no fused
// multiply-add), as when decay and update run as separate kernels.
__device__ __forceinline__ void momentum1(float &x, float &g, float &m, float lr, float beta, float omb, float decay) {
#pragma clang fp contract(off)
    const float xd = x * decay;
    const float mn = beta * m + omb * g;
    x = xd - lr * mn;
    m = mn;
    g = 0.f;
}

__global__ void __launch_bounds__(256) momentum_kernel(float *__restrict__ X, float *__restrict__ G, float *__restrict__ M, u32 count,
                                                       u32 vec, float lr, float beta, float omb, float decay) {
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    if (vec) {
        const u32 nq = count / 4;
        for (u32 q = i; q < nq; q += stride) {
            const v4f xv = reinterpret_cast<v4f *>(X)[q], gv = reinterpret_cast<v4f *>(G)[q], mv = reinterpret_cast<v4f *>(M)[q];
            float x[4] = {xv.x, xv.y, xv.z, xv.w}, g[4] = {gv.x, gv.y, gv.z, gv.w}, m[4] = {mv.x, mv.y, mv.z, mv.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) momentum1(x[k], g[k], m[k], lr, beta, omb, decay);
            reinterpret_cast<v4f *>(X)[q] = v4f{x[0], x[1], x[2], x[3]};
            reinterpret_cast<v4f *>(G)[q] = v4f{g[0], g[1], g[2], g[3]};
            reinterpret_cast<v4f *>(M)[q] = v4f{m[0], m[1], m[2], m[3]};
        }
        for (u32 r = nq * 4 + i; r < count; r += stride) momentum1(X[r], G[r], M[r], lr, beta, omb, decay);
    } else {
        for (; i < count; i += stride) momentum1(X[i], G[i], M[i], lr, beta, omb, decay);
    }
}

// ---- batch normalisation per feature over the batch -------------------------------------------------------------------
// X viewed as N x F. A workgroup owns FL consecutive features and splits the samples over G = 256 / FL lane groups: group
// g takes samples g, g+G, ...; per-feature sums are combined through LDS in group order (fixed association). FL is 64
// (256-byte row segments) when that already yields enough workgroups for the chip, else 32 or 16, which also shortens
// each thread's sample loop. A thread keeps up to kBnCache of its samples in registers (N <= G * kBnCache: every tensor is
// then read from memory once, with all loads of a sweep in flight together); beyond that it re-reads them.
constexpr int kBnCache = 16;

template <int FL>
struct BnGeom {
    static constexpr u32 G = 256 / FL;
    u32 fl, g, f;
    bool on;
    __device__ __forceinline__ BnGeom(u32 F) : fl(threadIdx.x % FL), g(threadIdx.x / FL), f(blockIdx.x * FL + fl), on(f < F) {}
    // sum of v over the G lane groups of feature fl, in group order
    __device__ __forceinline__ float reduce(float v, float (*red)[FL]) const {
        __syncthreads();  // the previous use of `red` is over
        red[g][fl] = v;
        __syncthreads();
        float r = red[0][fl];
#pragma unroll
        for (u32 k = 1; k < G; ++k) r += red[k][fl];
        return r;
    }
    // four sums at once (one round through LDS instead of four), each in the same group order as `reduce`
    __device__ __forceinline__ void reduce4(float &a, float &b, float &c, float &d, v4f (*red4)[FL]) const {
        __syncthreads();
        red4[g][fl] = v4f{a, b, c, d};
        __syncthreads();
        v4f r = red4[0][fl];
#pragma unroll
        for (u32 k = 1; k < G; ++k) {
            const v4f o = red4[k][fl];
            r.x += o.x, r.y += o.y, r.z += o.z, r.w += o.w;
        }
        a = r.x, b = r.y, c = r.z, d = r.w;
    }
};

template <int FL>
__global__ void __launch_bounds__(256) batchnorm_fwd_kernel(const float *__restrict__ X, const float *__restrict__ beta,
                                                            const float *__restrict__ gamma, float *__restrict__ mean,
                                                            float *__restrict__ var, float *__restrict__ Y, float *__restrict__ xHat,
                                                            const float *__restrict__ addend, float *__restrict__ reluOut, u32 N, u32 F) {
    constexpr u32 G = 256 / FL;
    __shared__ float red[G][FL];
    const BnGeom<FL> t(F);
    const bool cached = N <= G * kBnCache;
    const float *x = X + (t.on ? t.f : 0);
    // Cached sweeps load unconditionally (a sample past the batch reads row 0, a feature past the extent column 0) and drop
    // what does not count afterwards: with a branch around every load the compiler puts each load next to its use, and a
    // sweep becomes one memory round trip per sample instead of one in all.
    float xv[kBnCache], av[kBnCache];
    float s = 0.f;
    // scale and shift are requested with the first sweep and pinned behind the first reduction: requested where they are
    // used, they would still be in flight when the store sweep starts, and every conditionally executed store block would
    // wait for them again, and with them for the stores issued before it
    float ga = gamma[t.on ? t.f : 0], be = beta[t.on ? t.f : 0];
    if (cached) {
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) {
            const u32 n = t.g + G * i;
            xv[i] = x[size_t(n < N ? n : 0) * F];
        }
        if (reluOut && addend) {  // the other summand of the residual connection: requested with the first sweep
            const float *ad = addend + (t.on ? t.f : 0);
#pragma unroll
            for (int i = 0; i < kBnCache; ++i) {
                const u32 n = t.g + G * i;
                av[i] = ad[size_t(n < N ? n : 0) * F];
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // no use of a loaded value moves up between the loads
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) xv[i] = (t.on && t.g + G * i < N) ? xv[i] : 0.f;
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) s += xv[i];
    } else if (t.on) {
        for (u32 n = t.g; n < N; n += G) s += x[size_t(n) * F];
    }
    const float m = t.reduce(s, red) / float(N);
    asm volatile("" : "+v"(ga), "+v"(be));
    float q = 0.f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) {
            const float d = xv[i] - m;
            q += (t.g + G * i < N) ? d * d : 0.f;
        }
    } else if (t.on) {
        for (u32 n = t.g; n < N; n += G) {
            const float d = x[size_t(n) * F] - m;
            q += d * d;
        }
    }
    const float v = t.reduce(q, red) / float(N);
    if (!t.on) return;
    const float inv = 1.0f / sqrtf(v + 1e-8f);
    // outputs a caller does not need are not written: Y and xHat may be null; reluOut = max(Y + addend, 0) is optional
    // (addend: the other summand of a residual connection that closes right behind this normalisation, or null)
    auto put = [&](u32 n, float xh, float add, auto has_xhat, auto has_y, auto has_relu) {
        const float y = xh * ga + be;
        if constexpr (has_xhat.value) xHat[size_t(n) * F + t.f] = xh;
        if constexpr (has_y.value) Y[size_t(n) * F + t.f] = y;
        if constexpr (has_relu.value) {
            const float z = addend ? y + add : y;
            reluOut[size_t(n) * F + t.f] = z > 0.f ? z : 0.f;
        }
    };
    // Which outputs exist is decided once, outside the store sweep: with a test in front of every store the compiler's
    // wait in front of the next block also covers the stores just issued (they count like loads), one round trip per sample.
    auto sweep = [&](auto has_xhat, auto has_y, auto has_relu) {
        if (cached) {
#pragma unroll
            for (int i = 0; i < kBnCache; ++i) {
                const u32 n = t.g + G * i;
                if (n < N) put(n, (xv[i] - m) * inv, (has_relu.value && addend) ? av[i] : 0.f, has_xhat, has_y, has_relu);
            }
        } else {
            for (u32 n = t.g; n < N; n += G)
                put(n, (x[size_t(n) * F] - m) * inv, (has_relu.value && addend) ? addend[size_t(n) * F + t.f] : 0.f, has_xhat, has_y, has_relu);
        }
    };
    using T = std::true_type;
    using Fa = std::false_type;
    switch ((xHat ? 1 : 0) | (Y ? 2 : 0) | (reluOut ? 4 : 0)) {
        case 1: sweep(T{}, Fa{}, Fa{}); break;
        case 2: sweep(Fa{}, T{}, Fa{}); break;
        case 3: sweep(T{}, T{}, Fa{}); break;
        case 4: sweep(Fa{}, Fa{}, T{}); break;
        case 5: sweep(T{}, Fa{}, T{}); break;
        case 6: sweep(Fa{}, T{}, T{}); break;
        case 7: sweep(T{}, T{}, T{}); break;
        default: break;
    }
    if (t.g == 0) mean[t.f] = m, var[t.f] = v;
}

template <int FL, bool MASK, bool SUM2>
__global__ void __launch_bounds__(256) batchnorm_bwd_kernel(const float *__restrict__ dY, const float *__restrict__ dY2,
                                                            float *__restrict__ dyOut, const float *__restrict__ gamma,
                                                            const float *__restrict__ X, float *__restrict__ dX,
                                                            float *__restrict__ dGamma, float *__restrict__ dBeta,
                                                            const float *__restrict__ reluOut, u32 N, u32 F) {
    constexpr u32 G = 256 / FL;
    __shared__ float red[G][FL];
    const BnGeom<FL> t(F);
    const bool cached = N <= G * kBnCache;
    const float *x = X + (t.on ? t.f : 0), *dy = dY + (t.on ? t.f : 0);
    // reluOut given: dY is the gradient behind a ReLU whose output is reluOut, so the gradient that reaches this
    // normalisation is dY where reluOut > 0 and 0 elsewhere
    // SUM2: the gradient arrives in two parts that are added first (a residual connection opens right behind the ReLU).
    // dyOut, when given, receives the gradient as it reaches this normalisation (the copy the residual connection that
    // closes in front of the ReLU hands to its shortcut).
    const float *mk = MASK ? reluOut + (t.on ? t.f : 0) : nullptr;
    const float *dy2 = SUM2 ? dY2 + (t.on ? t.f : 0) : nullptr;
    auto grad = [&](u32 n) -> float {
        float e = dy[size_t(n) * F];
        if (SUM2) e = e + dy2[size_t(n) * F];
        if (!MASK) return e;
        return mk[size_t(n) * F] > 0.f ? e : 0.f;
    };
    float xv[kBnCache], dv[kBnCache];
    float s = 0.f;
    float ga = gamma[t.on ? t.f : 0];  // requested with the sweep, pinned behind the first reduction
    if (cached) {
        // every load of the sweep is issued, unconditionally (a sample past the batch reads row 0), before any is used: with
        // a branch around a load the compiler puts it next to its use, one memory round trip per sample
        float ev[SUM2 ? kBnCache : 1], mv[MASK ? kBnCache : 1];
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) {
            const u32 n = t.g + G * i;
            const size_t row = size_t(n < N ? n : 0) * F;
            xv[i] = x[row];
            dv[i] = dy[row];
            if (SUM2) ev[i] = dy2[row];
            if (MASK) mv[i] = mk[row];
        }
        __builtin_amdgcn_sched_barrier(0);  // no use of a loaded value moves up between the loads
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) {
            const bool ok = t.on && t.g + G * i < N;
            if (SUM2) dv[i] = dv[i] + ev[i];
            if (MASK) dv[i] = mv[i] > 0.f ? dv[i] : 0.f;
            xv[i] = ok ? xv[i] : 0.f;
            dv[i] = ok ? dv[i] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) s += xv[i];
    } else if (t.on) {
        for (u32 n = t.g; n < N; n += G) s += x[size_t(n) * F];
    }
    const float m = t.reduce(s, red) / float(N);
    asm volatile("" : "+v"(ga));
    // one sweep for the remaining sums: sum d^2, sum dy*d, sum dy, sum d  (d = x - mean)
    float q = 0.f, sdd = 0.f, sdy = 0.f, sd = 0.f;
    if (cached) {
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) {
            const bool ok = t.g + G * i < N;
            const float d = ok ? xv[i] - m : 0.f;
            q += d * d, sdd += dv[i] * d, sdy += dv[i], sd += d;
        }
    } else if (t.on) {
        for (u32 n = t.g; n < N; n += G) {
            const float d = x[size_t(n) * F] - m, e = grad(n);
            q += d * d, sdd += e * d, sdy += e, sd += d;
        }
    }
    __shared__ __attribute__((aligned(16))) v4f red4[G][FL];
    float Sdd = sdd, Sdy = sdy, Sd = sd;
    t.reduce4(q, Sdd, Sdy, Sd, red4);
    const float v = q / float(N);
    if (!t.on) return;
    const float inv = 1.0f / sqrtf(v + 1e-8f), invN = 1.0f / float(N);
    const float dVar = ga * Sdd * -0.5f * inv * inv * inv;
    const float dMean = ga * Sdy * -inv + dVar * (-2.0f * Sd) * invN;
    // the parameter gradients fall out of the same sums: dBeta = sum dy, dGamma = sum dy*xHat = inv * sum dy*(x - mean)
    if (dGamma && t.g == 0) dGamma[t.f] = Sdd * inv, dBeta[t.f] = Sdy;
    if (cached) {
#pragma unroll
        for (int i = 0; i < kBnCache; ++i) {
            const u32 n = t.g + G * i;
            if (n < N) {
                dX[size_t(n) * F + t.f] = dv[i] * ga * inv + dVar * (xv[i] - m) * 2.0f * invN + dMean * invN;
                if (dyOut) dyOut[size_t(n) * F + t.f] = dv[i];
            }
        }
    } else {
        for (u32 n = t.g; n < N; n += G) {
            const float e = grad(n);
            dX[size_t(n) * F + t.f] = e * ga * inv + dVar * (x[size_t(n) * F] - m) * 2.0f * invN + dMean * invN;
            if (dyOut) dyOut[size_t(n) * F + t.f] = e;
        }
    }
}

template <int FL>
__global__ void __launch_bounds__(256) batchnorm_param_grads_kernel(const float *__restrict__ dY, const float *__restrict__ xHat,
                                                                    float *__restrict__ dGamma, float *__restrict__ dBeta, u32 N, u32 F) {
    constexpr u32 G = 256 / FL;
    __shared__ float red[G][FL];
    const BnGeom<FL> t(F);
    float db = 0.f, dg = 0.f;
    if (t.on) {
        const float *dy = dY + t.f, *xh = xHat + t.f;
        u32 n = t.g;
        for (; n + 3 * G < N; n += 4 * G) {  // four independent samples in flight
            const float e0 = dy[size_t(n) * F], e1 = dy[size_t(n + G) * F], e2 = dy[size_t(n + 2 * G) * F], e3 = dy[size_t(n + 3 * G) * F];
            const float h0 = xh[size_t(n) * F], h1 = xh[size_t(n + G) * F], h2 = xh[size_t(n + 2 * G) * F], h3 = xh[size_t(n + 3 * G) * F];
            db += (e0 + e1) + (e2 + e3);
            dg += (e0 * h0 + e1 * h1) + (e2 * h2 + e3 * h3);
        }
        for (; n < N; n += G) {
            const float e = dy[size_t(n) * F];
            db += e;
            dg += e * xh[size_t(n) * F];
        }
    }
    const float DB = t.reduce(db, red), DG = t.reduce(dg, red);
    if (t.on && t.g == 0) dBeta[t.f] = DB, dGamma[t.f] = DG;
}

// features per workgroup: the widest of 64 / 32 / 16 that still gives at least 512 workgroups (16 if none does)
static u32 bn_features_per_wg(u32 F) { return F >= 64 * 512 ? 64 : (F >= 32 * 512 ? 32 : 16); }

static int check_bn(const char *what, u32 N, u32 F) {
    if (!N || !F) return fail(CRB_EINVAL_SHAPE, "%s: zero dimension", what);
    if (uint64_t(N) * F > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: tensor exceeds 2^31 elements", what);
    return CRB_OK;
}

// The momentum step over a table of parameter tensors in one launch: blockIdx.y selects the item, the blocks of a row
// stride over its elements. Same arithmetic as momentum_kernel.
__global__ void __launch_bounds__(256) momentum_multi_kernel(const crb_momentum_item *__restrict__ items) {
    const crb_momentum_item it = items[blockIdx.y];
    const float omb = 1.0f - it.beta;
    const u32 stride = gridDim.x * 256;
    u32 i = blockIdx.x * 256 + threadIdx.x;
    const bool vec = ((reinterpret_cast<uintptr_t>(it.X) | reinterpret_cast<uintptr_t>(it.G) | reinterpret_cast<uintptr_t>(it.M)) & 15u) == 0;
    if (vec) {
        const u32 nq = it.count / 4;
        for (u32 q = i; q < nq; q += stride) {
            const v4f xv = reinterpret_cast<v4f *>(it.X)[q], gv = reinterpret_cast<v4f *>(it.G)[q], mv = reinterpret_cast<v4f *>(it.M)[q];
            float x[4] = {xv.x, xv.y, xv.z, xv.w}, g[4] = {gv.x, gv.y, gv.z, gv.w}, m[4] = {mv.x, mv.y, mv.z, mv.w};
#pragma unroll
            for (int k = 0; k < 4; ++k) momentum1(x[k], g[k], m[k], it.lr, it.beta, omb, it.decay);
            reinterpret_cast<v4f *>(it.X)[q] = v4f{x[0], x[1], x[2], x[3]};
            reinterpret_cast<v4f *>(it.G)[q] = v4f{g[0], g[1], g[2], g[3]};
            reinterpret_cast<v4f *>(it.M)[q] = v4f{m[0], m[1], m[2], m[3]};
        }
        for (u32 r = nq * 4 + i; r < it.count; r += stride) momentum1(it.X[r], it.G[r], it.M[r], it.lr, it.beta, omb, it.decay);
    } else {
        for (; i < it.count; i += stride) momentum1(it.X[i], it.G[i], it.M[i], it.lr, it.beta, omb, it.decay);
    }
}

static int check_pool(const char *what, u32 planes, u32 IH, u32 IW, u32 sH, u32 sW, u32 rH, u32 rW) {
    if (!planes || !IH || !IW || !sH || !sW || !rH || !rW) return fail(CRB_EINVAL_SHAPE, "%s: zero dimension", what);
    if (sH != rH || sW != rW)
        return fail(CRB_EINVAL_SHAPE, "%s: only non-overlapping windows (stride == range) are supported, got stride %ux%u range %ux%u",
                    what, sH, sW, rH, rW);
    if (IH < rH || IW < rW) return fail(CRB_EINVAL_SHAPE, "%s: window larger than the input", what);
    if (uint64_t(planes) * IH * IW > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: tensor exceeds 2^31 elements", what);
    return CRB_OK;
}

template <bool MASK, bool SUM2>
static void bn_bwd_launch(const float *dY, const float *dY2, float *dyOut, const float *gamma, const float *X, float *dX, float *dGamma,
                          float *dBeta, const float *reluOut, uint32_t N, uint32_t F, hipStream_t s) {
    switch (bn_features_per_wg(F)) {
        case 64: hipLaunchKernelGGL((batchnorm_bwd_kernel<64, MASK, SUM2>), dim3(ceil_div(F, 64)), dim3(256), 0, s, dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F); break;
        case 32: hipLaunchKernelGGL((batchnorm_bwd_kernel<32, MASK, SUM2>), dim3(ceil_div(F, 32)), dim3(256), 0, s, dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F); break;
        default: hipLaunchKernelGGL((batchnorm_bwd_kernel<16, MASK, SUM2>), dim3(ceil_div(F, 16)), dim3(256), 0, s, dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F);
    }
}

}  // namespace crb

using namespace crb;

extern "C" {

int crb_relu_fwd(const float *X, float *Y, uint32_t count, void *stream) {
    if (!X || !Y) return fail(CRB_ENULL, "crb_relu_fwd: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_relu_fwd: zero size");
    return launch_map2(X, nullptr, Y, count, ReluF{}, hipStream_t(stream), "crb_relu_fwd");
}

int crb_relu_bwd(const float *X, const float *dY, float *dX, uint32_t count, void *stream) {
    if (!X || !dY || !dX) return fail(CRB_ENULL, "crb_relu_bwd: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_relu_bwd: zero size");
    return launch_map2(X, dY, dX, count, ReluGradF{}, hipStream_t(stream), "crb_relu_bwd");
}

int crb_maxpool_fwd(const float *X, float *Y, float *record, uint32_t planes, uint32_t IH, uint32_t IW, uint32_t sH, uint32_t sW,
                    uint32_t rH, uint32_t rW, void *stream) {
    if (!X || !Y || !record) return fail(CRB_ENULL, "crb_maxpool_fwd: null operand");
    if (int st = check_pool("crb_maxpool_fwd", planes, IH, IW, sH, sW, rH, rW)) return st;
    const u32 OH = IH / rH, OW = IW / rW;
    hipStream_t s = hipStream_t(stream);
    if (rH == 2 && rW == 2 && IH % 2 == 0 && IW % 4 == 0 && aligned16(X) && aligned16(record) && aligned16(Y)) {
        const u32 pairs = planes * OH * (IW / 4);
        hipLaunchKernelGGL(maxpool2x2_fwd_kernel, dim3(ceil_div(pairs, 256)), dim3(256), 0, s, X, Y, record, pairs, IW, FastDiv(IW / 4));
        return check_launch("crb_maxpool_fwd");
    }
    const u32 windows = planes * OH * OW;
    hipLaunchKernelGGL(maxpool_fwd_kernel, dim3(ceil_div(windows, 256)), dim3(256), 0, s, X, Y, record, windows, IH, IW, rH, rW,
                       FastDiv(OW), FastDiv(OH));
    return check_launch("crb_maxpool_fwd");
}

int crb_maxpool_bwd(float *dX, const float *dY, float *record, uint32_t planes, uint32_t IH, uint32_t IW, uint32_t sH, uint32_t sW,
                    uint32_t rH, uint32_t rW, void *stream) {
    if (!dX || !dY || !record) return fail(CRB_ENULL, "crb_maxpool_bwd: null operand");
    if (int st = check_pool("crb_maxpool_bwd", planes, IH, IW, sH, sW, rH, rW)) return st;
    const u32 OH = IH / rH, OW = IW / rW;
    hipStream_t s = hipStream_t(stream);
    if (rH == 2 && rW == 2 && IH % 2 == 0 && IW % 4 == 0 && aligned16(dX) && aligned16(record) && aligned16(dY)) {
        const u32 pairs = planes * OH * (IW / 4);
        hipLaunchKernelGGL(maxpool2x2_bwd_kernel, dim3(ceil_div(pairs, 256)), dim3(256), 0, s, dX, dY, record, pairs, IW, FastDiv(IW / 4));
        return check_launch("crb_maxpool_bwd");
    }
    if (OH * rH != IH || OW * rW != IW) {  // rows / columns no window covers receive no gradient
        if (int st = crb_tensor_fill(dX, 0.f, planes * IH * IW, stream)) return st;
    }
    const u32 windows = planes * OH * OW;
    hipLaunchKernelGGL(maxpool_bwd_kernel, dim3(ceil_div(windows, 256)), dim3(256), 0, s, dX, dY, record, windows, IH, IW, rH, rW,
                       FastDiv(OW), FastDiv(OH));
    return check_launch("crb_maxpool_bwd");
}

int crb_softmax(const float *A, float *out, uint32_t rows, uint32_t step, void *stream) {
    if (!A || !out) return fail(CRB_ENULL, "crb_softmax: null operand");
    if (!rows || !step) return fail(CRB_EINVAL_SHAPE, "crb_softmax: zero dimension");
    if (uint64_t(rows) * step > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "crb_softmax: tensor exceeds 2^31 elements");
    hipStream_t s = hipStream_t(stream);
    if (step <= 64)
        hipLaunchKernelGGL(softmax_short_kernel, dim3(ceil_div(rows, 4)), dim3(256), 0, s, A, out, rows, step);
    else
        hipLaunchKernelGGL(softmax_rows_kernel, dim3(rows), dim3(256), 0, s, A, out, step);
    return check_launch("crb_softmax");
}

int crb_cross_entropy_grad(const float *Y, const float *labels, float *dY, uint32_t count, void *stream) {
    if (!Y || !labels || !dY) return fail(CRB_ENULL, "crb_cross_entropy_grad: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_cross_entropy_grad: zero size");
    return launch_map2(Y, labels, dY, count, SubF{}, hipStream_t(stream), "crb_cross_entropy_grad");
}

uint32_t crb_cross_entropy_scratch_floats(uint32_t count) {
    const u32 blocks = ceil_div(count, 4096u);
    return blocks > 1024 ? 1024 : blocks;
}

int crb_cross_entropy_loss(const float *Y, const float *labels, float *scratch, uint32_t scratch_floats, float *loss_out,
                           uint32_t count, void *stream) {
    if (!Y || !labels || !loss_out) return fail(CRB_ENULL, "crb_cross_entropy_loss: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_cross_entropy_loss: zero size");
    hipStream_t s = hipStream_t(stream);
    const u32 blocks = crb_cross_entropy_scratch_floats(count);
    if (blocks == 1) {
        hipLaunchKernelGGL(ce_partial_kernel, dim3(1), dim3(256), 0, s, Y, labels, loss_out, count, count);
        return check_launch("crb_cross_entropy_loss");
    }
    if (!scratch) return fail(CRB_ENULL, "crb_cross_entropy_loss: null scratch");
    if (scratch_floats < blocks)
        return fail(CRB_EWORKSPACE, "crb_cross_entropy_loss: scratch of %u floats < required %u", scratch_floats, blocks);
    const u32 chunk = ceil_div(count, blocks);
    hipLaunchKernelGGL(ce_partial_kernel, dim3(blocks), dim3(256), 0, s, Y, labels, scratch, count, chunk);
    if (int st = check_launch("crb_cross_entropy_loss")) return st;
    hipLaunchKernelGGL(sum_small_kernel, dim3(1), dim3(256), 0, s, scratch, loss_out, blocks);
    return check_launch("crb_cross_entropy_loss");
}

int crb_tensor_sub_inplace(float *a, const float *b, uint32_t count, void *stream) {
    if (!a || !b) return fail(CRB_ENULL, "crb_tensor_sub_inplace: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_sub_inplace: zero size");
    return launch_map2(a, b, a, count, SubF{}, hipStream_t(stream), "crb_tensor_sub_inplace");
}

int crb_tensor_scale_inplace(float *a, float factor, uint32_t count, void *stream) {
    if (!a) return fail(CRB_ENULL, "crb_tensor_scale_inplace: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_tensor_scale_inplace: zero size");
    return launch_map2(a, nullptr, a, count, ScaleF{factor}, hipStream_t(stream), "crb_tensor_scale_inplace");
}

static int bn_fwd(const char *what, const float *X, const float *beta, const float *gamma, float *mean, float *var, float *Y,
                  float *xHat, const float *addend, float *reluOut, uint32_t N, uint32_t F, void *stream) {
    if (int st = check_bn(what, N, F)) return st;
    hipStream_t s = hipStream_t(stream);
    switch (bn_features_per_wg(F)) {
        case 64: hipLaunchKernelGGL(batchnorm_fwd_kernel<64>, dim3(ceil_div(F, 64)), dim3(256), 0, s, X, beta, gamma, mean, var, Y, xHat, addend, reluOut, N, F); break;
        case 32: hipLaunchKernelGGL(batchnorm_fwd_kernel<32>, dim3(ceil_div(F, 32)), dim3(256), 0, s, X, beta, gamma, mean, var, Y, xHat, addend, reluOut, N, F); break;
        default: hipLaunchKernelGGL(batchnorm_fwd_kernel<16>, dim3(ceil_div(F, 16)), dim3(256), 0, s, X, beta, gamma, mean, var, Y, xHat, addend, reluOut, N, F);
    }
    return check_launch(what);
}

static int bn_bwd(const char *what, const float *dY, const float *dY2, float *dyOut, const float *gamma, const float *X, float *dX,
                  float *dGamma, float *dBeta, const float *reluOut, uint32_t N, uint32_t F, void *stream) {
    if (int st = check_bn(what, N, F)) return st;
    hipStream_t s = hipStream_t(stream);
    if (reluOut && dY2)
        bn_bwd_launch<true, true>(dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F, s);
    else if (reluOut)
        bn_bwd_launch<true, false>(dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F, s);
    else if (dY2)
        bn_bwd_launch<false, true>(dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F, s);
    else
        bn_bwd_launch<false, false>(dY, dY2, dyOut, gamma, X, dX, dGamma, dBeta, reluOut, N, F, s);
    return check_launch(what);
}

int crb_batchnorm_relu_fwd(const float *X, const float *beta, const float *gamma, float *mean, float *var, float *Y_or_null,
                           float *xHat_or_null, const float *addend_or_null, float *reluOut, uint32_t N, uint32_t F, void *stream) {
    if (!X || !beta || !gamma || !mean || !var || !reluOut) return fail(CRB_ENULL, "crb_batchnorm_relu_fwd: null operand");
    return bn_fwd("crb_batchnorm_relu_fwd", X, beta, gamma, mean, var, Y_or_null, xHat_or_null, addend_or_null, reluOut, N, F, stream);
}

int crb_batchnorm_relu_bwd(const float *dY, const float *dY2_or_null, const float *reluOut, const float *gamma, const float *X, float *dX,
                           float *dGamma_or_null, float *dBeta_or_null, float *dYmasked_or_null, uint32_t N, uint32_t F, void *stream) {
    if (!dY || !reluOut || !gamma || !X || !dX) return fail(CRB_ENULL, "crb_batchnorm_relu_bwd: null operand");
    if (!dGamma_or_null != !dBeta_or_null) return fail(CRB_ENULL, "crb_batchnorm_relu_bwd: dGamma and dBeta go together");
    return bn_bwd("crb_batchnorm_relu_bwd", dY, dY2_or_null, dYmasked_or_null, gamma, X, dX, dGamma_or_null, dBeta_or_null, reluOut, N, F, stream);
}

int crb_batchnorm_fwd(const float *X, const float *beta, const float *gamma, float *mean, float *var, float *Y, float *xHat,
                      uint32_t N, uint32_t F, void *stream) {
    if (!X || !beta || !gamma || !mean || !var || !Y || !xHat) return fail(CRB_ENULL, "crb_batchnorm_fwd: null operand");
    return bn_fwd("crb_batchnorm_fwd", X, beta, gamma, mean, var, Y, xHat, nullptr, nullptr, N, F, stream);
}

int crb_batchnorm_bwd(const float *dY, const float *gamma, const float *X, float *dX, float *dGamma_or_null, float *dBeta_or_null,
                      uint32_t N, uint32_t F, void *stream) {
    if (!dY || !gamma || !X || !dX) return fail(CRB_ENULL, "crb_batchnorm_bwd: null operand");
    if (!dGamma_or_null != !dBeta_or_null) return fail(CRB_ENULL, "crb_batchnorm_bwd: dGamma and dBeta go together");
    return bn_bwd("crb_batchnorm_bwd", dY, nullptr, nullptr, gamma, X, dX, dGamma_or_null, dBeta_or_null, nullptr, N, F, stream);
}

int crb_batchnorm_param_grads(const float *dY, const float *xHat, float *dGamma, float *dBeta, uint32_t N, uint32_t F,
                              void *stream) {
    if (!dY || !xHat || !dGamma || !dBeta) return fail(CRB_ENULL, "crb_batchnorm_param_grads: null operand");
    if (int st = check_bn("crb_batchnorm_param_grads", N, F)) return st;
    hipStream_t s = hipStream_t(stream);
    switch (bn_features_per_wg(F)) {
        case 64: hipLaunchKernelGGL(batchnorm_param_grads_kernel<64>, dim3(ceil_div(F, 64)), dim3(256), 0, s, dY, xHat, dGamma, dBeta, N, F); break;
        case 32: hipLaunchKernelGGL(batchnorm_param_grads_kernel<32>, dim3(ceil_div(F, 32)), dim3(256), 0, s, dY, xHat, dGamma, dBeta, N, F); break;
        default: hipLaunchKernelGGL(batchnorm_param_grads_kernel<16>, dim3(ceil_div(F, 16)), dim3(256), 0, s, dY, xHat, dGamma, dBeta, N, F);
    }
    return check_launch("crb_batchnorm_param_grads");
}

int crb_momentum_apply(float *X, float *G, float *M, uint32_t count, float lr, float beta, float decay, void *stream) {
    if (!X || !G || !M) return fail(CRB_ENULL, "crb_momentum_apply: null operand");
    if (!count) return fail(CRB_EINVAL_SHAPE, "crb_momentum_apply: zero size");
    const u32 vec = aligned16(X) && aligned16(G) && aligned16(M);
    hipLaunchKernelGGL(momentum_kernel, dim3(stream_grid(count)), dim3(256), 0, hipStream_t(stream), X, G, M, count, vec, lr, beta,
                       1.0f - beta, decay);
    return check_launch("crb_momentum_apply");
}

int crb_momentum_apply_multi(const crb_momentum_item *items_on_device, uint32_t n_items, uint32_t max_count, void *stream) {
    if (!items_on_device) return fail(CRB_ENULL, "crb_momentum_apply_multi: null table");
    if (!n_items || !max_count) return fail(CRB_EINVAL_SHAPE, "crb_momentum_apply_multi: empty table");
    if (n_items > 65535u) return fail(CRB_EINVAL_SHAPE, "crb_momentum_apply_multi: more than 65535 items");
    u32 bx = ceil_div(ceil_div(max_count, 4), 256);
    bx = bx > 64 ? 64 : bx;
    hipLaunchKernelGGL(momentum_multi_kernel, dim3(bx, n_items), dim3(256), 0, hipStream_t(stream), items_on_device);
    return check_launch("crb_momentum_apply_multi");
}

}  // extern "C"
