// Dataset records to network input on the device: byte pixels (as stored in the dataset file) are converted to float,
// normalised per image and optionally mirrored / shifted, all in one pass, so that a batch crosses the host link as
// bytes (a quarter of the float volume) and its float form is written to device memory exactly once.
// One workgroup per image: per-channel statistics by a fixed-order reduction (bit-reproducible, no atomics), then the
// output pass with 16-byte stores. HBM-bound: 1 byte read and 4 bytes written per value.
#include "igemm_engine.h"

namespace crb {

static constexpr int kMaxChannels = 64;

__device__ inline float wave_min(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fminf(v, __shfl_xor(v, m, 64));
    return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
    return v;
}
__device__ inline float wave_sum(float v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += __shfl_xor(v, m, 64);
    return v;
}
__device__ inline u32 wave_sum_u32(u32 v) {
#pragma unroll
    for (int m = 32; m >= 1; m >>= 1) v += u32(__shfl_xor(int(v), m, 64));
    return v;
}

struct PrepArgs {
    const uint8_t *src;  // images x C x H x W bytes
    float *dst;          // images x C x H x W floats
    const crb_image_aug *aug;  // per image, or null
    u32 C, H, W, step;   // step = H * W
    float p0, p1;        // uniform: desiredMin, desiredMax; distribution: desiredMean, desiredVar
};

// NORM 0: plain conversion; 1: min-max scaling with extrema running over the channels; 2: mean / deviation scaling.
// VEC: the plane size is a multiple of 4, so a lane reads 4 bytes and writes 4 floats at a time.
template <int NORM, bool VEC>
__global__ void __launch_bounds__(256) image_prep_kernel(PrepArgs a) {
#pragma clang fp contract(off)  // every operation rounded on its own, as in the scalar formulation
    __shared__ float s_part[2][4][kMaxChannels];  // per wave partials
    __shared__ float s_a[kMaxChannels], s_b[kMaxChannels];  // per channel: (min, max - min) or (mean, deviation)
    const u32 img = blockIdx.x, t = threadIdx.x, wave = t >> 6, lane = t & 63;
    const uint8_t *src = a.src + size_t(img) * a.C * a.step;
    float *dst = a.dst + size_t(img) * a.C * a.step;

    if (NORM == 1) {
        for (u32 c = 0; c < a.C; ++c) {
            float lo = 255.f, hi = 0.f;
            const uint8_t *p = src + size_t(c) * a.step;
            if (VEC) {
                for (u32 q = t; q < a.step / 4; q += 256) {
                    const u32 w = reinterpret_cast<const u32 *>(p)[q];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const float v = float((w >> (8 * k)) & 255u);
                        lo = fminf(lo, v), hi = fmaxf(hi, v);
                    }
                }
            } else {
                for (u32 i = t; i < a.step; i += 256) {
                    const float v = float(p[i]);
                    lo = fminf(lo, v), hi = fmaxf(hi, v);
                }
            }
            lo = wave_min(lo), hi = wave_max(hi);
            if (lane == 0) s_part[0][wave][c] = lo, s_part[1][wave][c] = hi;
        }
        __syncthreads();
        if (t == 0) {  // extrema run on from channel to channel
            float lo = 1e10f, hi = -1e10f;
            for (u32 c = 0; c < a.C; ++c) {
                for (int w = 0; w < 4; ++w) lo = fminf(lo, s_part[0][w][c]), hi = fmaxf(hi, s_part[1][w][c]);
                s_a[c] = lo, s_b[c] = hi - lo;
            }
        }
        __syncthreads();
    } else if (NORM == 2) {
        for (u32 c = 0; c < a.C; ++c) {  // sums of byte values are exact in integers
            u32 sum = 0;
            const uint8_t *p = src + size_t(c) * a.step;
            if (VEC) {
                for (u32 q = t; q < a.step / 4; q += 256) {
                    const u32 w = reinterpret_cast<const u32 *>(p)[q];
                    sum += (w & 255u) + ((w >> 8) & 255u) + ((w >> 16) & 255u) + (w >> 24);
                }
            } else {
                for (u32 i = t; i < a.step; i += 256) sum += p[i];
            }
            sum = wave_sum_u32(sum);
            if (lane == 0) reinterpret_cast<u32 *>(s_part[0][wave])[c] = sum;
        }
        __syncthreads();
        if (t < a.C) {
            const u32 *q0 = reinterpret_cast<const u32 *>(s_part[0][0]), *q1 = reinterpret_cast<const u32 *>(s_part[0][1]),
                      *q2 = reinterpret_cast<const u32 *>(s_part[0][2]), *q3 = reinterpret_cast<const u32 *>(s_part[0][3]);
            s_a[t] = float(q0[t] + q1[t] + q2[t] + q3[t]) / float(a.step);
        }
        __syncthreads();
        for (u32 c = 0; c < a.C; ++c) {
            const float mean = s_a[c];
            float acc = 0.f;
            const uint8_t *p = src + size_t(c) * a.step;
            for (u32 i = t; i < a.step; i += 256) {
                const float d = float(p[i]) - mean;
                acc += d * d;
            }
            acc = wave_sum(acc);
            if (lane == 0) s_part[1][wave][c] = acc;
        }
        __syncthreads();
        if (t < a.C) {
            const float var = (((s_part[1][0][t] + s_part[1][1][t]) + s_part[1][2][t]) + s_part[1][3][t]) / float(a.step);
            s_b[t] = float(sqrt(double(var) + 1e-8));
        }
        __syncthreads();
    }

    auto norm = [&](float v, u32 c) -> float {
        if (NORM == 1) {
            const float d = v - s_a[c];
            const float q = d / s_b[c];
            const float s = q * (a.p1 - a.p0);
            return s + a.p0;
        }
        if (NORM == 2) {
            const float d = v - s_a[c];
            const float s = d * a.p1;
            const float q = s / s_b[c];
            return q + a.p0;
        }
        return v;
    };

    u32 flags = 0;
    int dh = 0, dw = 0;
    if (a.aug) flags = a.aug[img].flags, dh = a.aug[img].dh, dw = a.aug[img].dw;
    const u32 total = a.C * a.step;
    if (!(flags & 3u)) {
        if (VEC) {
            for (u32 q = t; q < total / 4; q += 256) {
                const u32 w = reinterpret_cast<const u32 *>(src)[q];
                const u32 c = (q * 4) / a.step;
                reinterpret_cast<v4f *>(dst)[q] = v4f{norm(float(w & 255u), c), norm(float((w >> 8) & 255u), c),
                                                     norm(float((w >> 16) & 255u), c), norm(float(w >> 24), c)};
            }
        } else {
            for (u32 i = t; i < total; i += 256) dst[i] = norm(float(src[i]), i / a.step);
        }
        return;
    }
    // mirrored and / or shifted: out(h, w) = mirrored(h + dh, w + dw) where that lies strictly inside row 0 / column 0, else 0
    const bool flip = flags & 1u, crop = flags & 2u;
    for (u32 i = t; i < total; i += 256) {
        const u32 c = i / a.step, r = i % a.step;
        int h = int(r / a.W), w = int(r % a.W);
        bool inside = true;
        if (crop) {
            h += dh, w += dw;
            inside = h > 0 && h < int(a.H) && w > 0 && w < int(a.W);
        }
        if (flip) w = int(a.W) - 1 - w;
        dst[i] = inside ? norm(float(src[size_t(c) * a.step + u32(h) * a.W + u32(w)]), c) : 0.f;
    }
}

template <int NORM>
static void launch_prep(const PrepArgs &a, u32 images, bool vec, hipStream_t s) {
    if (vec)
        hipLaunchKernelGGL((image_prep_kernel<NORM, true>), dim3(images), dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL((image_prep_kernel<NORM, false>), dim3(images), dim3(256), 0, s, a);
}
}  // namespace crb

using namespace crb;

extern "C" int crb_images_from_bytes(const uint8_t *src, float *dst, uint32_t images, uint32_t channels, uint32_t H, uint32_t W,
                                     int norm, float p0, float p1, const crb_image_aug *aug_on_device, void *stream) {
    if (!src || !dst) return fail(CRB_ENULL, "crb_images_from_bytes: null operand");
    if (!images || !channels || !H || !W) return fail(CRB_EINVAL_SHAPE, "crb_images_from_bytes: zero dimension");
    if (channels > u32(kMaxChannels)) return fail(CRB_EINVAL_SHAPE, "crb_images_from_bytes: more than 64 channels");
    if (norm < CRB_NORM_NONE || norm > CRB_NORM_DISTRIBUTION) return fail(CRB_EINVAL_SHAPE, "crb_images_from_bytes: unknown normalisation");
    if (uint64_t(images) * channels * H * W > 0x7fffffffull || uint64_t(H) * W > (1u << 24))
        return fail(CRB_EINVAL_SHAPE, "crb_images_from_bytes: tensor exceeds 2^31 elements or a plane exceeds 2^24");
    PrepArgs a{src, dst, aug_on_device, channels, H, W, H * W, p0, p1};
    const bool vec = (a.step % 4 == 0) && (reinterpret_cast<uintptr_t>(src) % 4 == 0) && (reinterpret_cast<uintptr_t>(dst) % 16 == 0);
    hipStream_t s = hipStream_t(stream);
    if (norm == CRB_NORM_UNIFORM)
        launch_prep<1>(a, images, vec, s);
    else if (norm == CRB_NORM_DISTRIBUTION)
        launch_prep<2>(a, images, vec, s);
    else
        launch_prep<0>(a, images, vec, s);
    return check_launch("crb_images_from_bytes");
}
