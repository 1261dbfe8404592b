// 1x1 / stride 2 / unpadded convolutions on even-sized images (the projection shortcuts of residual networks): data
// gradient and weight gradient. At 2-3 flop per byte these are plain streaming kernels: no MFMA, the arithmetic is a few
// VALU operations per byte moved, and the general implicit-GEMM engine spends most of its time on tile bookkeeping for them.
//   dX[n,ic,2oh,2ow] = sum_oc W[oc,ic] * dY[n,oc,oh,ow], every other element of dX = 0
//   dW[oc,ic]       += sum_{n,oh,ow} dY[n,oc,oh,ow] * X[n,ic,2oh,2ow]
// Channel counts up to 64, input channels a multiple of 4.
#pragma once
#include "igemm_engine.h"

namespace crb {

constexpr u32 kScMaxC = 64;  // channel limit of both kernels
constexpr u32 kScTile = 64;  // output pixels per staged tile of the weight gradient (32 when that is what fills the chip)

// One thread per (image, output row, group of 4 input channels, output column): adjacent lanes write adjacent 8-byte pairs
// {value, 0} of an even dX row and {0, 0} of the odd row below it. Summation over oc in ascending order.
__global__ void __launch_bounds__(256) sc_dgrad_kernel(const float *__restrict__ W, const float *__restrict__ dY, float *__restrict__ dX,
                                                       u32 IC, u32 OC, u32 OH, u32 OW, u32 items, FastDiv d_ow, FastDiv d_icg,
                                                       FastDiv d_oh) {
    __shared__ __attribute__((aligned(16))) float sW[kScMaxC * kScMaxC];  // [oc][ic]
    for (u32 i = threadIdx.x; i < OC * IC; i += 256) sW[i] = W[i];
    __syncthreads();
    const u32 item = blockIdx.x * 256 + threadIdx.x;
    if (item >= items) return;
    u32 r, ow, icg, r2, oh, n;
    d_ow.divmod(item, r, ow);
    d_icg.divmod(r, r2, icg);
    d_oh.divmod(r2, n, oh);
    const u32 OHW = OH * OW, IW = 2 * OW, IH = 2 * OH;
    const float *dy = dY + (size_t(n) * OC * OH + oh) * OW + ow;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll 8
    for (u32 oc = 0; oc < OC; ++oc) {
        const float v = dy[size_t(oc) * OHW];
        const v4f w = *reinterpret_cast<const v4f *>(&sW[oc * IC + 4 * icg]);
        acc.x += v * w.x, acc.y += v * w.y, acc.z += v * w.z, acc.w += v * w.w;
    }
    float *base = dX + ((size_t(n) * IC + 4 * icg) * IH + 2 * oh) * IW + 2 * ow;
    const size_t plane = size_t(IH) * IW;
    const float out[4] = {acc.x, acc.y, acc.z, acc.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        *reinterpret_cast<v2f *>(base + j * plane) = v2f{out[j], 0.f};
        *reinterpret_cast<v2f *>(base + j * plane + IW) = v2f{0.f, 0.f};
    }
}

// Workgroup z sums its run of PT-pixel tiles into part[z][oc][ic]. A tile is staged pixel-major in LDS (dY: PT x OC, X at the
// even positions: PT x IC; every load of a tile is issued before the first is stored, a pixel past the end reads the last
// one and is zeroed on the way to LDS); a thread owns one output channel and four input channels (task = oc * IC/4 + ic/4; with at most
// 128 tasks the pixels of a tile are shared out over 256 / tasks subsets, combined in subset order at the end). Pixels in
// ascending order within a thread: a fixed association.
template <u32 PT>
__global__ void __launch_bounds__(256) sc_wgrad_kernel(const float *__restrict__ dY, const float *__restrict__ X, float *__restrict__ part,
                                                       u32 IC, u32 OC, u32 OH, u32 OW, u32 total_px, u32 tiles_per_z, FastDiv d_ow,
                                                       FastDiv d_ohw) {
    __shared__ float sY[PT][kScMaxC + 1];
    __shared__ __attribute__((aligned(16))) float sX[PT][kScMaxC + 4];
    __shared__ __attribute__((aligned(16))) v4f red[256];
    const u32 tasks = OC * (IC / 4);
    const u32 nsub = tasks <= 128 ? 256 / tasks : 1;     // pixel subsets per tile
    const u32 per_thread = tasks > 256 ? (tasks + 255) / 256 : 1;  // at most 4 (64 x 16 tasks)
    const u32 sub = tasks <= 128 ? threadIdx.x / tasks : 0;
    const bool worker = tasks > 128 || threadIdx.x < tasks * nsub;
    const u32 task0 = tasks <= 128 ? threadIdx.x % tasks : threadIdx.x;
    const u32 icq_n = IC / 4, OHW = OH * OW, IW = 2 * OW, IH = 2 * OH;
    v4f acc[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) acc[k] = v4f{0.f, 0.f, 0.f, 0.f};
    constexpr u32 CL = 256 / PT, NL = kScMaxC / CL;  // channel lanes of the staging; loads per lane and tensor at most
    const u32 p_lane = threadIdx.x % PT, c_lane = threadIdx.x / PT;  // staging: pixel of this lane, first channel
    const u32 t_begin = blockIdx.x * tiles_per_z;
    for (u32 t = t_begin; t < t_begin + tiles_per_z; ++t) {
        const u32 P = t * PT + p_lane;
        const bool ok = P < total_px;
        u32 n, q, oh, ow;
        d_ohw.divmod(ok ? P : total_px - 1, n, q);
        d_ow.divmod(q, oh, ow);
        const float *dy = dY + size_t(n) * OC * OHW + q;
        const float *x = X + (size_t(n) * IC * IH + 2 * oh) * IW + 2 * ow;
        float vy[NL], vx[NL];
#pragma unroll
        for (u32 i = 0; i < NL; ++i) {
            const u32 c = c_lane + i * CL;
            vy[i] = dy[size_t(c < OC ? c : 0) * OHW];
            vx[i] = x[size_t(c < IC ? c : 0) * IH * IW];
        }
        __syncthreads();  // the previous tile has been consumed
#pragma unroll
        for (u32 i = 0; i < NL; ++i) {
            const u32 c = c_lane + i * CL;
            if (c < OC) sY[p_lane][c] = ok ? vy[i] : 0.f;
            if (c < IC) sX[p_lane][c] = ok ? vx[i] : 0.f;
        }
        __syncthreads();
        if (worker) {
#pragma unroll
            for (u32 k = 0; k < 4; ++k) {
                const u32 task = task0 + k * 256;
                if (k < per_thread && task < tasks) {
                    const u32 oc = task / icq_n, icq = task - oc * icq_n;
                    for (u32 p = sub; p < PT; p += nsub) {
                        const float v = sY[p][oc];
                        const v4f xv = *reinterpret_cast<const v4f *>(&sX[p][4 * icq]);
                        acc[k].x += v * xv.x, acc[k].y += v * xv.y, acc[k].z += v * xv.z, acc[k].w += v * xv.w;
                    }
                }
            }
        }
    }
    float *out = part + size_t(blockIdx.x) * OC * IC;
    if (nsub > 1) {  // combine the pixel subsets in subset order
        __syncthreads();
        red[threadIdx.x] = acc[0];
        __syncthreads();
        if (threadIdx.x < tasks) {
            v4f r = red[threadIdx.x];
            for (u32 s = 1; s < nsub; ++s) {
                const v4f o = red[s * tasks + threadIdx.x];
                r.x += o.x, r.y += o.y, r.z += o.z, r.w += o.w;
            }
            *reinterpret_cast<v4f *>(out + 4 * threadIdx.x) = r;  // task -> (oc, 4*icq): element oc*IC + 4*icq = 4*task
        }
    } else {
#pragma unroll
        for (u32 k = 0; k < 4; ++k) {
            const u32 task = task0 + k * 256;
            if (k < per_thread && task < tasks) *reinterpret_cast<v4f *>(out + 4 * task) = acc[k];
        }
    }
}

struct ScWgradPlan {
    u32 splits, tiles_per_z, tile;  // tile: pixels per staged tile
    size_t workspace_bytes;
};

inline ScWgradPlan sc_wgrad_plan(u32 N, u32 IC, u32 OC, u32 OH, u32 OW) {
    ScWgradPlan p;
    p.tile = ceil_div(N * OH * OW, kScTile) < 512 ? kScTile / 2 : kScTile;  // few pixels: shorter tiles, one per workgroup
    const u32 tiles = ceil_div(N * OH * OW, p.tile);
    u32 splits = tiles < 512 ? tiles : 512;
    p.tiles_per_z = ceil_div(tiles, splits);
    p.splits = ceil_div(tiles, p.tiles_per_z);
    p.workspace_bytes = size_t(p.splits) * OC * IC * sizeof(float);
    return p;
}

inline int launch_sc_dgrad(const float *W, const float *dY, float *dX, u32 N, u32 IC, u32 OC, u32 OH, u32 OW, hipStream_t s,
                           const char *what) {
    const u32 icg = IC / 4;
    const uint64_t items = uint64_t(N) * OH * icg * OW;
    if (items > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL(sc_dgrad_kernel, dim3(ceil_div(u32(items), 256)), dim3(256), 0, s, W, dY, dX, IC, OC, OH, OW, u32(items),
                       FastDiv(OW), FastDiv(icg), FastDiv(OH));
    return check_launch(what);
}

// part: plan.workspace_bytes of scratch, 16-byte aligned; dW accumulated by the split reduction in fixed order
// (dW == nullptr: the slices are left in part, unsummed)
inline int launch_sc_wgrad(const float *dY, const float *X, float *dW, float *part, const ScWgradPlan &plan, u32 N, u32 IC, u32 OC,
                           u32 OH, u32 OW, hipStream_t s, const char *what) {
    if (plan.tile == kScTile)
        hipLaunchKernelGGL(sc_wgrad_kernel<kScTile>, dim3(plan.splits), dim3(256), 0, s, dY, X, part, IC, OC, OH, OW, N * OH * OW,
                           plan.tiles_per_z, FastDiv(OW), FastDiv(OH * OW));
    else
        hipLaunchKernelGGL(sc_wgrad_kernel<kScTile / 2>, dim3(plan.splits), dim3(256), 0, s, dY, X, part, IC, OC, OH, OW, N * OH * OW,
                           plan.tiles_per_z, FastDiv(OW), FastDiv(OH * OW));
    if (int st = check_launch(what)) return st;
    if (!dW) return CRB_OK;
    return launch_splitk_reduce(part, dW, OC * IC, plan.splits, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, what);
}

}  // namespace crb
