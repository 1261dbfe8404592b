// Weight gradient of a 1x1 / stride 1 convolution for gfx950 (the bottleneck layers of densely connected networks):
// dW[oc][ic] += sum over (n, p) of dY[n][oc][p] * X[n][ic][p] — a product whose contraction index is the pixel and whose
// operands both lie pixel-contiguous in NCHW memory, read once each (the pass is bandwidth-bound).
//
// A workgroup owns ALL output channels (NOB blocks of 16, OC <= 16 * NOB), four blocks of 16 input channels (block
// w * groups + g for wave w of group g) and a slice z of the (image, 64-pixel run) tiles. Per tile it stages the dY planes
// and its 64 X planes in double-buffered LDS (16-byte global loads of whole 256-byte runs); wave w multiplies its ic block
// against every oc block, so a staged dY value feeds NOB MFMAs per wave and no accumulator is shared between waves (no
// cross-wave reduction). One partial result per (ic group, z), summed in fixed order by the split reduction:
// bit-reproducible.
//
// v_mfma_f32_16x16x4_f32 (wave64, lane l): A = dY[oc = l%16][pixel 4s + l/16], B = X[pixel 4s + l/16][ic = l%16],
// accumulator register r = dW[oc = 4*(l/16) + r][ic = l%16].
#pragma once
#include "igemm_engine.h"

namespace crb {

constexpr int kPwPT = 64;          // pixels per tile
constexpr int kPwOcc = 2;          // workgroups per CU (LDS-bound)
constexpr int kPwP = kPwPT + 2;    // plane stride (floats): == 2 mod 4, so 16 planes x 2 lane groups land on 32 distinct banks

struct PwWgradArgs {
    const float *dY;  // N x OC x HW
    const float *X;   // N x IC x HW
    float *out;       // splits > 1: partials [z][OC][IC]; splits == 1: dW (accumulated)
    u32 OC, IC, HW;
    u32 ic_groups;    // ceil(ceil(IC / 16) / 4)
    u32 tiles, tiles_per_z, tiles_per_img;
    u32 splits, accumulate;
};

template <int NOB>
__global__ void __launch_bounds__(kThreads, kPwOcc) pw_wgrad_kernel(PwWgradArgs a) {
    constexpr int P = kPwP, NCH = NOB * 16 + 64;  // staged planes per buffer
    __shared__ __attribute__((aligned(16))) float smem[2 * NCH * P];
    const u32 t = threadIdx.x, bid = blockIdx.x;
    // the ic groups of one slice read the same dY tiles: ids 8 apart run on the same XCD and share them through its L2
    u32 grp, z;
    if (a.splits >= kXcds) {
        const u32 xcd = bid % kXcds, slot = bid / kXcds;
        grp = slot % a.ic_groups, z = (slot / a.ic_groups) * kXcds + xcd;
        if (z >= a.splits) return;
    } else {
        grp = bid % a.ic_groups, z = bid / a.ic_groups;
    }
    const u32 t_begin = z * a.tiles_per_z;
    const u32 t_end = t_begin + a.tiles_per_z < a.tiles ? t_begin + a.tiles_per_z : a.tiles;

    // staging: thread t owns quad q of plane c0 + i * RPP for every item i (dY planes first, then the 4 X blocks).
    // Ragged channel blocks read a clamped (valid) row, zeroed when it is stored to LDS: no branch around a load.
    constexpr int QPR = kPwPT / 4, RPP = kThreads / QPR;  // quads per row; rows staged per pass of the workgroup
    const u32 q = t % QPR, c0 = t / QPR;
    constexpr int NI = (NCH + RPP - 1) / RPP;  // items per thread: plane i * RPP + c0
    v4f reg[NI];
    u32 row_off[NI];  // element offset of this thread's channel row inside one image, per item
    bool row_ok[NI];
#pragma unroll
    for (int i = 0; i < NI; ++i) {
        const u32 r = i * RPP + c0, xr = r - NOB * 16;  // plane; X plane
        const bool is_y = r < NOB * 16;
        const u32 ch = is_y ? r : ((xr >> 4) * a.ic_groups + grp) * 16 + (xr & 15), lim = is_y ? a.OC : a.IC;
        row_ok[i] = ch < lim && r < NCH;
        row_off[i] = (ch < lim ? ch : lim - 1) * a.HW + 4 * q;
    }
    auto fetch = [&](u32 tile) {
        const u32 n = tile / a.tiles_per_img, p0 = (tile % a.tiles_per_img) * kPwPT;
        const size_t ybase = size_t(n) * a.OC * a.HW + p0, xbase = size_t(n) * a.IC * a.HW + p0;
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const bool is_y = (i + 1) * RPP <= NOB * 16 ? true : (i * RPP >= NOB * 16 ? false : i * RPP + c0 < NOB * 16);
            reg[i] = *reinterpret_cast<const v4f *>((is_y ? a.dY + ybase : a.X + xbase) + row_off[i]);
        }
    };
    auto commit = [&](float *buf) {
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            if ((i + 1) * RPP > NCH && i * RPP + c0 >= NCH) continue;  // past the last plane (only when RPP does not divide NCH)
            float *p = buf + (i * RPP + c0) * P + 4 * q;
            const v4f v = row_ok[i] ? reg[i] : v4f{0.f, 0.f, 0.f, 0.f};
            *reinterpret_cast<v2f *>(p) = v2f{v.x, v.y};
            *reinterpret_cast<v2f *>(p + 2) = v2f{v.z, v.w};
        }
    };

    const u32 lane = t & 63, wave = t >> 6, li = lane & 15, kq = lane >> 4;
    const u32 ib = wave * a.ic_groups + grp;           // this wave's ic block: a ragged block count spreads over the groups
    const bool active = ib * 16 < a.IC;               // waves without a block only help staging
    v4f acc[NOB];
#pragma unroll
    for (int o = 0; o < NOB; ++o) acc[o] = v4f{0.f, 0.f, 0.f, 0.f};

    fetch(t_begin);
    commit(smem);
    __syncthreads();
    for (u32 tile = t_begin; tile < t_end; ++tile) {
        const u32 b = (tile - t_begin) & 1;
        const bool more = tile + 1 < t_end;
        if (more) fetch(tile + 1);
        if (active) {
            const float *py = smem + b * NCH * P + li * P + kq;
            const float *px = smem + b * NCH * P + (NOB * 16 + wave * 16 + li) * P + kq;
            constexpr int NSTEP = kPwPT / 4, PF = 2;  // LDS reads run PF steps (PF * NOB MFMAs) ahead of their use
            float av[PF + 1][NOB], bv[PF + 1];
            auto read_step = [&](int s, int slot) {
#pragma unroll
                for (int o = 0; o < NOB; ++o) av[slot][o] = py[o * 16 * P + 4 * s];
                bv[slot] = px[4 * s];
            };
#pragma unroll
            for (int s = 0; s < PF; ++s) read_step(s, s);
#pragma unroll
            for (int s = 0; s < NSTEP; ++s) {
                if (s + PF < NSTEP) read_step(s + PF, (s + PF) % (PF + 1));
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int o = 0; o < NOB; ++o)
                    acc[o] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s % (PF + 1)][o], bv[s % (PF + 1)], acc[o], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        if (more) commit(smem + (b ^ 1) * NCH * P);
        __syncthreads();
    }
    if (!active) return;
    float *out = a.out + size_t(z) * a.OC * a.IC * (a.accumulate ? 0 : 1);
    const u32 ic = ib * 16 + li;
    if (ic >= a.IC) return;
    // dW's old values are requested together, the stores follow (a read in front of every store would make each store wait for
    // the one before it)
    float old[NOB][4];
#pragma unroll
    for (int o = 0; o < NOB; ++o)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const u32 oc = o * 16 + 4 * kq + r;
            old[o][r] = (a.accumulate && oc < a.OC) ? out[size_t(oc) * a.IC + ic] : 0.f;
        }
#pragma unroll
    for (int o = 0; o < NOB; ++o)
#pragma unroll
        for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(old[o][r]));
#pragma unroll
    for (int o = 0; o < NOB; ++o)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const u32 oc = o * 16 + 4 * kq + r;
            if (oc < a.OC) out[size_t(oc) * a.IC + ic] = old[o][r] + acc[o][r];
        }
}

struct PwWgradPlan {
    u32 ic_groups, tiles, splits, tiles_per_z;
    size_t workspace_bytes;
};

// 1x1 / stride 1 / no padding with at most 64 output channels, whole 64-pixel runs and 16-byte aligned planes
inline bool pw_wgrad_fits(u32 IC, u32 OC, u32 HW) { return OC <= 64 && HW % kPwPT == 0 && IC >= 16; }

inline PwWgradPlan pw_wgrad_plan(u32 N, u32 IC, u32 OC, u32 HW) {
    PwWgradPlan p;
    p.ic_groups = ceil_div(ceil_div(IC, 16u), 4u);
    p.tiles = N * (HW / kPwPT);
    const u32 target = 256u * kPwOcc;  // resident workgroups
    u32 splits = p.ic_groups >= target ? 1u : target / p.ic_groups;
    if (splits > p.tiles) splits = p.tiles;
    p.tiles_per_z = ceil_div(p.tiles, splits);
    p.splits = ceil_div(p.tiles, p.tiles_per_z);
    p.workspace_bytes = p.splits > 1 ? size_t(p.splits) * OC * IC * sizeof(float) : 0;
    return p;
}

// dW == nullptr (a split plan only): the slices are left in ws, unsummed.
inline int launch_pw_wgrad(const float *dY, const float *X, float *dW, float *ws, const PwWgradPlan &p, u32 IC, u32 OC, u32 HW,
                           hipStream_t s, const char *what) {
    PwWgradArgs a;
    a.dY = dY, a.X = X, a.out = p.splits > 1 ? ws : dW;
    a.OC = OC, a.IC = IC, a.HW = HW;
    a.ic_groups = p.ic_groups, a.tiles = p.tiles, a.tiles_per_z = p.tiles_per_z, a.tiles_per_img = HW / kPwPT;
    a.splits = p.splits, a.accumulate = p.splits > 1 ? 0u : 1u;
    const uint64_t wgs = p.splits >= kXcds ? uint64_t(ceil_div(p.splits, kXcds)) * kXcds * p.ic_groups : uint64_t(p.splits) * p.ic_groups;
    if (wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    if (OC <= 48)
        hipLaunchKernelGGL(pw_wgrad_kernel<3>, dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    else
        hipLaunchKernelGGL(pw_wgrad_kernel<4>, dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    if (int st = check_launch(what)) return st;
    if (p.splits > 1 && dW) return launch_splitk_reduce(ws, dW, OC * IC, p.splits, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, what);
    return CRB_OK;
}

}  // namespace crb
