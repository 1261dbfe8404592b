// Dataset records to network input on the device: byte pixels (as stored in the dataset file) are converted to float,
// normalised per image and optionally mirrored / shifted, all in one pass, so that a batch crosses the host link as
// bytes (a quarter of the float volume) and its float form is written to device memory exactly once.
// One workgroup per image: per-channel statistics by a fixed-order reduction (bit-reproducible, no atomics), then the
// output pass with 16-byte stores. HBM-bound: 1 byte read and 4 bytes written per value.
#include "igemm_engine.h"

namespace crb {

static constexpr int kMaxChannels = 64;
static constexpr int kTableChannels = 8;  // up to this many channels the output values are tabulated per byte value

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
    __shared__ float s_tbl[NORM ? kTableChannels * 256 : 1];
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

    auto compute = [&](float v, u32 c) -> float {
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
    // With few channels the result per (channel, byte value) is tabulated once and looked up in the output pass.
    const bool tabulated = NORM != 0 && a.C <= u32(kTableChannels);
    if (tabulated) {
        for (u32 e = t; e < a.C * 256; e += 256) s_tbl[e] = compute(float(e & 255u), e >> 8);
        __syncthreads();
    }
    auto norm = [&](u32 byte, u32 c) -> float { return tabulated ? s_tbl[c * 256 + byte] : compute(float(byte), c); };

    u32 flags = 0;
    int dh = 0, dw = 0;
    if (a.aug) flags = a.aug[img].flags, dh = a.aug[img].dh, dw = a.aug[img].dw;
    const u32 total = a.C * a.step;
    if (!(flags & 3u)) {
        if (VEC) {
            for (u32 q = t; q < total / 4; q += 256) {
                const u32 w = reinterpret_cast<const u32 *>(src)[q];
                const u32 c = (q * 4) / a.step;
                reinterpret_cast<v4f *>(dst)[q] = v4f{norm(w & 255u, c), norm((w >> 8) & 255u, c), norm((w >> 16) & 255u, c), norm(w >> 24, c)};
            }
        } else {
            for (u32 i = t; i < total; i += 256) dst[i] = norm(src[i], i / a.step);
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
        dst[i] = inside ? norm(src[size_t(c) * a.step + u32(h) * a.W + u32(w)], c) : 0.f;
    }
}

// Small images (at most 4 channels and 4096 bytes, plane a multiple of 4 bytes): one wave per image, the image held in
// registers between the statistics and the output pass, reductions by lane exchange only — no workgroup barrier and no
// serial section, so 32 images are in flight per compute unit. Mirrored / shifted images are staged in LDS (4 KB per
// wave) for the gather; that path also needs a width that is a multiple of 4.
static constexpr int kWaveWords = 16;  // 32-bit words per lane

template <int NORM, bool AUG>
__global__ void __launch_bounds__(256) image_prep_wave_kernel(PrepArgs a, u32 images) {
#pragma clang fp contract(off)
    __shared__ u32 s_img[AUG ? 4 : 1][AUG ? 64 * kWaveWords : 1];
    __shared__ float s_tbl[NORM ? 4 : 1][NORM ? 4 * 256 : 1];  // per wave: output value by (channel, byte value)
    const u32 wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const u32 img = blockIdx.x * 4 + wave;
    if (img >= images) return;  // no workgroup barrier below
    const u32 total = a.C * a.step, words = total / 4, wpc = a.step / 4;
    const u32 *src = reinterpret_cast<const u32 *>(a.src + size_t(img) * total);
    v4f *dst = reinterpret_cast<v4f *>(a.dst + size_t(img) * total);

    u32 cache[kWaveWords], chan[kWaveWords];
#pragma unroll
    for (int k = 0; k < kWaveWords; ++k) {
        const u32 q = lane + 64 * k;
        cache[k] = q < words ? src[q] : 0u;
        chan[k] = q < words ? q / wpc : 0xffu;
    }
    float A[4] = {0.f, 0.f, 0.f, 0.f}, B[4] = {1.f, 1.f, 1.f, 1.f};
    if (NORM == 1) {
        float lo_run = 1e10f, hi_run = -1e10f;
#pragma unroll
        for (u32 c = 0; c < 4; ++c) {
            if (c < a.C) {
                float lo = 255.f, hi = 0.f;
#pragma unroll
                for (int k = 0; k < kWaveWords; ++k) {
                    if (chan[k] == c) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float v = float((cache[k] >> (8 * j)) & 255u);
                            lo = fminf(lo, v), hi = fmaxf(hi, v);
                        }
                    }
                }
                lo_run = fminf(lo_run, wave_min(lo)), hi_run = fmaxf(hi_run, wave_max(hi));
                A[c] = lo_run, B[c] = hi_run - lo_run;
            }
        }
    } else if (NORM == 2) {
#pragma unroll
        for (u32 c = 0; c < 4; ++c) {
            if (c < a.C) {
                u32 sum = 0;
#pragma unroll
                for (int k = 0; k < kWaveWords; ++k)
                    if (chan[k] == c) sum += (cache[k] & 255u) + ((cache[k] >> 8) & 255u) + ((cache[k] >> 16) & 255u) + (cache[k] >> 24);
                const float mean = float(wave_sum_u32(sum)) / float(a.step);
                float acc = 0.f;
#pragma unroll
                for (int k = 0; k < kWaveWords; ++k) {
                    if (chan[k] == c) {
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float d = float((cache[k] >> (8 * j)) & 255u) - mean;
                            acc += d * d;
                        }
                    }
                }
                const float var = wave_sum(acc) / float(a.step);
                A[c] = mean, B[c] = float(sqrt(double(var) + 1e-8));
            }
        }
    }
    // A normalised value depends only on the channel and the byte, so the arithmetic (a correctly rounded division among
    // it) is done once per possible byte value and the output pass looks the result up.
    if (NORM) {
        float *tbl = s_tbl[wave];
#pragma unroll
        for (u32 c = 0; c < 4; ++c) {
            if (c < a.C) {
#pragma unroll
                for (u32 x = lane; x < 256; x += 64) {
                    const float v = float(x);
                    float r;
                    if (NORM == 1) {
                        const float d = v - A[c];
                        const float q = d / B[c];
                        const float t = q * (a.p1 - a.p0);
                        r = t + a.p0;
                    } else {
                        const float d = v - A[c];
                        const float t = d * a.p1;
                        const float q = t / B[c];
                        r = q + a.p0;
                    }
                    tbl[c * 256 + x] = r;
                }
            }
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    const float *tblr = s_tbl[NORM ? wave : 0];
    auto norm = [&](u32 byte, u32 c) -> float { return NORM ? tblr[c * 256 + byte] : float(byte); };

    u32 flags = 0;
    int dh = 0, dw = 0;
    if (AUG) flags = a.aug[img].flags, dh = a.aug[img].dh, dw = a.aug[img].dw;
    if (!AUG || !(flags & 3u)) {
#pragma unroll
        for (int k = 0; k < kWaveWords; ++k) {
            const u32 q = lane + 64 * k;
            if (q < words) {
                const u32 w = cache[k], c = chan[k];
                dst[q] = v4f{norm(w & 255u, c), norm((w >> 8) & 255u, c), norm((w >> 16) & 255u, c), norm(w >> 24, c)};
            }
        }
        return;
    }
    if (AUG) {
        u32 *mine = s_img[wave];
#pragma unroll
        for (int k = 0; k < kWaveWords; ++k) {
            const u32 q = lane + 64 * k;
            if (q < words) mine[q] = cache[k];
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        const uint8_t *bytes = reinterpret_cast<const uint8_t *>(mine);
        const bool flip = flags & 1u, crop = flags & 2u;
#pragma unroll
        for (int k = 0; k < kWaveWords; ++k) {
            const u32 q = lane + 64 * k;
            if (q < words) {
                const u32 c = chan[k], r = 4 * q - c * a.step;
                const int h = int(r / a.W) + (crop ? dh : 0), w0 = int(r % a.W) + (crop ? dw : 0);
                float o[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    int w = w0 + j;
                    const bool inside = !crop || (h > 0 && h < int(a.H) && w > 0 && w < int(a.W));
                    if (flip) w = int(a.W) - 1 - w;
                    o[j] = inside ? norm(bytes[c * a.step + u32(h) * a.W + u32(w)], c) : 0.f;
                }
                dst[q] = v4f{o[0], o[1], o[2], o[3]};
            }
        }
    }
}

template <int NORM>
static void launch_prep_wave(const PrepArgs &a, u32 images, hipStream_t s) {
    if (a.aug)
        hipLaunchKernelGGL((image_prep_wave_kernel<NORM, true>), dim3(ceil_div(images, 4u)), dim3(256), 0, s, a, images);
    else
        hipLaunchKernelGGL((image_prep_wave_kernel<NORM, false>), dim3(ceil_div(images, 4u)), dim3(256), 0, s, a, images);
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
    const bool small = vec && channels <= 4 && channels * a.step <= 4u * 64u * u32(kWaveWords) && (!aug_on_device || W % 4 == 0);
    if (small) {
        if (norm == CRB_NORM_UNIFORM)
            launch_prep_wave<1>(a, images, s);
        else if (norm == CRB_NORM_DISTRIBUTION)
            launch_prep_wave<2>(a, images, s);
        else
            launch_prep_wave<0>(a, images, s);
        return check_launch("crb_images_from_bytes");
    }
    if (norm == CRB_NORM_UNIFORM)
        launch_prep<1>(a, images, vec, s);
    else if (norm == CRB_NORM_DISTRIBUTION)
        launch_prep<2>(a, images, vec, s);
    else
        launch_prep<0>(a, images, vec, s);
    return check_launch("crb_images_from_bytes");
}
