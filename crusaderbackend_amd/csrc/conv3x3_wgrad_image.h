// Weight gradient of a 3x3 / pad 1 / stride 1 convolution whose input has at most 3 channels (the image layers of the CIFAR
// networks: 3 -> 16, 3 -> 64 on 32x32 images). With 16 input channels per MFMA column block (conv3x3_wgrad.h) such a layer
// would multiply 13 planes of zeros; here the MFMA columns are the (input channel, tap) pairs instead — n = ic * 9 + tap,
// IC * 9 <= 27 of them in two 16-column blocks — which is also the order dW[oc][ic][fh][fw] has in memory.
//
// dW[oc][n] = sum over (image, y, x) of dY[oc][y][x] * X[ic(n)][y + fh(n) - 1][x + fw(n) - 1].
// A workgroup owns one block of 16 output channels and a slice z of the (image, TR rows) tiles, staged in double-buffered
// LDS as flat pixel runs (dY: TR rows; X: TR + 2 rows, zero outside the image). The tap shift fh * W + fw - 1 is part of a
// lane's base address (the lane is the column n), every step adds a compile-time immediate. The wrap-around of that shift
// at the left / right image border is removed by zeroing the X value of the lanes whose tap has fw = 0 (fw = 2) on the
// steps that sit on column 0 (W - 1). The four waves take different rows; their accumulators are summed through LDS in
// wave order, and the slices by the split reduction in fixed order: bit-reproducible.
//
// v_mfma_f32_16x16x4_f32 (wave64, lane l): A = dY[oc = l%16][pixel 4s + l/16], B = X'[pixel 4s + l/16][n = 16 b + l%16],
// accumulator register r of block b = dW[oc = 4*(l/16) + r][n = 16 b + l%16].
#pragma once
#include "conv3x3_wgrad.h"

namespace crb {

constexpr int kImgW = 32, kImgTR = 8, kImgMaxIC = 3, kImgNB = 2;

struct ImgWgradArgs {
    const float *dY;  // N x OC x H x 32
    const float *X;   // N x IC x H x 32
    float *out;       // splits > 1: partials [z][OC][IC * 9]; splits == 1: dW (accumulated)
    u32 OC, IC, H;
    u32 oc_blocks, tiles, tiles_per_z, tiles_per_img, splits, accumulate;
};

__global__ void __launch_bounds__(kThreads, 2) wgrad3x3_image_kernel(ImgWgradArgs a) {
    constexpr int W = kImgW, TR = kImgTR, NB = kImgNB;
    constexpr int YP = TR * W + 2;            // dY plane stride: == 2 mod 4 (16 planes x 2 lane groups on 32 distinct banks)
    constexpr int XP = (TR + 2) * W + 8 + 2;  // X plane: 4 leading + 4 trailing pad floats (kept zero), halo rows included
    constexpr int BUF = 16 * YP + kImgMaxIC * XP;
    constexpr int RW = TR / 4, NSTEP = RW * W / 4;  // rows and MFMA steps per wave per tile
    __shared__ __attribute__((aligned(16))) float smem[2 * BUF > 4 * NB * 256 ? 2 * BUF : 4 * NB * 256];
    const u32 t = threadIdx.x, bid = blockIdx.x;
    u32 ob, z;
    if (a.splits >= kXcds) {  // the oc blocks of one slice read the same X tiles: ids 8 apart share an XCD's L2
        const u32 xcd = bid % kXcds, slot = bid / kXcds;
        ob = slot % a.oc_blocks, z = (slot / a.oc_blocks) * kXcds + xcd;
        if (z >= a.splits) return;
    } else {
        ob = bid % a.oc_blocks, z = bid / a.oc_blocks;
    }
    const u32 HW = a.H * W;
    const u32 t_begin = z * a.tiles_per_z;
    const u32 t_end = t_begin + a.tiles_per_z < a.tiles ? t_begin + a.tiles_per_z : a.tiles;

    // ---- staging: 16-byte global loads, 8-byte LDS stores. dY: 16 planes x TR rows x 8 quads = 4 items per thread;
    // X: IC planes x (TR + 2) rows x 8 quads <= 240 items, one per thread.
    const u32 yq = t & 7, yrow = (t >> 3) & 7, yc0 = t >> 6;  // plane yc0 + 4 i
    const u32 xq = t & 7, xrow = (t >> 3) % (TR + 2), xc = t / (8 * (TR + 2));
    const bool x_on = xc < a.IC;
    v4f yreg[4], xreg;
    bool xin = false;  // whether xreg holds a row of the image (applied when it is stored: a select right behind the load would wait for it)
    auto fetch = [&](u32 tile) {
        const u32 n = tile / a.tiles_per_img;
        const int r0 = int(tile % a.tiles_per_img) * TR;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const u32 oc = ob * 16 + yc0 + 4 * i;
            yreg[i] = *reinterpret_cast<const v4f *>(a.dY + (size_t(n) * a.OC + (oc < a.OC ? oc : a.OC - 1)) * HW + (u32(r0) + yrow) * W + 4 * yq);
        }
        const int row = r0 - 1 + int(xrow);
        const bool in = x_on && row >= 0 && row < int(a.H);
        xreg = *reinterpret_cast<const v4f *>(a.X + (size_t(n) * a.IC + (x_on ? xc : 0)) * HW + u32(in ? row : 0) * W + 4 * xq);
        xin = in;
    };
    auto commit = [&](float *buf) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            // channels past the tensor's extent only reach rows of dW that are never stored: no need to zero them
            float *p = buf + (yc0 + 4 * i) * YP + yrow * W + 4 * yq;
            *reinterpret_cast<v2f *>(p) = v2f{yreg[i].x, yreg[i].y};
            *reinterpret_cast<v2f *>(p + 2) = v2f{yreg[i].z, yreg[i].w};
        }
        if (xc < kImgMaxIC) {
            float *p = buf + 16 * YP + xc * XP + 4 + xrow * W + 4 * xq;
            const v4f v = xin ? xreg : v4f{0.f, 0.f, 0.f, 0.f};
            *reinterpret_cast<v2f *>(p) = v2f{v.x, v.y};
            *reinterpret_cast<v2f *>(p + 2) = v2f{v.z, v.w};
        }
    };
    // pad floats of the X planes stay zero
    if (t < 2 * kImgMaxIC * 8) {
        float *plane = smem + (t / (kImgMaxIC * 8)) * BUF + 16 * YP + ((t / 8) % kImgMaxIC) * XP;
        const u32 k = t & 7;
        plane[k < 4 ? k : 4 + (TR + 2) * W + (k - 4)] = 0.f;
    }

    const u32 lane = t & 63, wave = t >> 6, li = lane & 15, kq = lane >> 4;
    // column n = 16 b + li of block b: (ic, fh, fw); columns past IC * 9 read what column 0 reads and are never stored
    int xbase[NB];
    bool fw0[NB], fw2[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        u32 n = b * 16 + li;
        if (n >= a.IC * 9) n = 0;
        const u32 ic = n / 9, fh = (n % 9) / 3, fw = n % 3;
        xbase[b] = int(16 * YP + ic * XP + 4 + (wave * RW + fh) * W + kq) + int(fw) - 1;
        fw0[b] = fw == 0, fw2[b] = fw == 2;
    }
    const int ybase = int(li * YP + wave * RW * W + kq);

    v4f acc[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) acc[b] = v4f{0.f, 0.f, 0.f, 0.f};

    fetch(t_begin);
    commit(smem);
    __syncthreads();
    for (u32 tile = t_begin; tile < t_end; ++tile) {
        const u32 cur = (tile - t_begin) & 1;
        const bool more = tile + 1 < t_end;
        if (more) fetch(tile + 1);
        const float *py = smem + cur * BUF + ybase, *px = smem + cur * BUF;
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            const float av = py[4 * s];
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float bv = px[xbase[b] + 4 * s];
                // this lane's pixel is column (4 s) % W + kq: taps with fw = 0 see nothing left of column 0, fw = 2 nothing right of W - 1
                if ((4 * s) % W == 0 && kq == 0 && fw0[b]) bv = 0.f;
                if ((4 * s + 4) % W == 0 && kq == 3 && fw2[b]) bv = 0.f;
                acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av, bv, acc[b], 0, 0, 0);
            }
        }
        if (more) commit(smem + (cur ^ 1) * BUF);
        __syncthreads();
    }

    // ---- sum of the four waves in wave order, then this (oc block, slice)'s part of the result ----------------------------
    float *red = smem;  // [wave][block][lane][4]
#pragma unroll
    for (int b = 0; b < NB; ++b) *reinterpret_cast<v4f *>(red + ((wave * NB + b) * 64 + lane) * 4) = acc[b];
    __syncthreads();
    const u32 K9 = a.IC * 9;
    float *out = a.out + size_t(z) * a.OC * K9 * (a.accumulate ? 0 : 1);
    // thread t: register r = t / 64 of lane l = t % 64: output channel 4 (l / 16) + r, column 16 b + l % 16
    const u32 r = t >> 6, l = t & 63;
    // dW's old values are requested together, the stores follow (a read in front of every store would make each store wait for
    // the one before it)
    float old[NB];
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const u32 oc = ob * 16 + 4 * (l >> 4) + r, n = b * 16 + (l & 15);
        old[b] = (a.accumulate && oc < a.OC && n < K9) ? out[size_t(oc) * K9 + n] : 0.f;
    }
#pragma unroll
    for (int b = 0; b < NB; ++b) asm volatile("" : "+v"(old[b]));
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        const u32 e = b * 256 + l * 4 + r;
        const float v = ((red[e] + red[NB * 256 + e]) + red[2 * NB * 256 + e]) + red[3 * NB * 256 + e];
        const u32 oc = ob * 16 + 4 * (l >> 4) + r, n = b * 16 + (l & 15);
        if (oc < a.OC && n < K9) out[size_t(oc) * K9 + n] = old[b] + v;
    }
}

inline bool wgrad_image_fits(u32 IC, u32 H, u32 Wd) { return IC <= u32(kImgMaxIC) && Wd == u32(kImgW) && H % kImgTR == 0; }

inline WgradDirectPlan wgrad_image_plan(u32 N, u32 IC, u32 OC, u32 H) {
    WgradDirectPlan p;
    p.pairs = ceil_div(OC, 16u);
    p.tiles = N * (H / kImgTR);
    const u32 target = 512;  // two workgroups per CU (20 KB of LDS each)
    u32 splits = p.pairs >= target ? 1u : target / p.pairs;
    if (splits > p.tiles) splits = p.tiles;
    p.tiles_per_z = ceil_div(p.tiles, splits);
    p.splits = ceil_div(p.tiles, p.tiles_per_z);
    p.workspace_bytes = p.splits > 1 ? size_t(p.splits) * OC * IC * 9 * sizeof(float) : 0;
    return p;
}

// dW == nullptr: the slices are left in ws, unsummed.
inline int launch_wgrad_image(const float *dY, const float *X, float *dW, float *ws, const WgradDirectPlan &p, u32 IC, u32 OC, u32 H,
                              hipStream_t s, const char *what) {
    ImgWgradArgs a;
    a.dY = dY, a.X = X, a.out = p.splits > 1 ? ws : dW;
    a.OC = OC, a.IC = IC, a.H = H;
    a.oc_blocks = p.pairs, a.tiles = p.tiles, a.tiles_per_z = p.tiles_per_z, a.tiles_per_img = H / kImgTR;
    a.splits = p.splits, a.accumulate = p.splits > 1 ? 0u : 1u;
    const uint64_t wgs = p.splits >= kXcds ? uint64_t(ceil_div(p.splits, kXcds)) * kXcds * p.pairs : uint64_t(p.splits) * p.pairs;
    if (wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL(wgrad3x3_image_kernel, dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    if (int st = check_launch(what)) return st;
    if (p.splits > 1 && dW) return launch_splitk_reduce(ws, dW, OC * IC * 9, p.splits, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, what);
    return CRB_OK;
}

}  // namespace crb
