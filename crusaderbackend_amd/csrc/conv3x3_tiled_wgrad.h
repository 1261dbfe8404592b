// Weight gradient of a 3x3 / stride 1 convolution (padding p = 0, 1 or 2 on both axes) for gfx950 on images of ANY extent:
// dW[oc][ic][fh][fw] = sum over (n, y, x) of dY[n][oc][y][x] * X[n][ic][y + fh - p][x + fw - p].
//
// For each of the nine taps this is an (OC x IC) product whose contraction index is the pixel. A 256-thread workgroup owns
// a block of 32 NOB output channels x 32 NIB input channels for all nine taps and a slice z of the (image, TH x TW pixel
// tile) list; tile by tile it stages the block's dY planes and the X window ((TH + 2) x (TW + 2), zero outside the image) in
// LDS and multiplies them with v_mfma_f32_32x32x2_f32: a wave holds one (32 oc, 32 ic) pair, nine accumulator blocks (one per
// tap, 144 registers), and reads one dY value and nine X values (the tap shifts) per step of nine MFMAs, every address
// `lane base + immediate`. With fewer than four pairs in the block the waves split the tile's pixels instead (PS parts) and
// each writes a partial result of its own. Partial results [z * PS + part][OC][IC][9] are summed in fixed order by the
// split reduction: bit-reproducible.
//
// LDS holds two tiles: the next one is requested before the current one is multiplied and stored behind it. Plane strides are
// odd, so the 32 lanes of a fragment read (32 planes, one float each) land on 32 different banks.
//
// v_mfma_f32_32x32x2_f32 (wave64, lane l): A[i = l%32][k = l/32] = dY[oc = i][pixel], B[k = l/32][j = l%32] = X[pixel + tap][ic = j],
// accumulator register r = dW[oc = 8*(r/4) + 4*(l/32) + r%4][ic = l%32]. Within a group of 8 pixels (one image row of the
// tile), step s of lane half h takes pixel 4h + s.
#pragma once
#include <type_traits>

#include "igemm_engine.h"

namespace crb {

template <int TH_, int TW_, int NOB_, int NIB_>
struct TiledWgradCfg {
    static constexpr int TH = TH_, TW = TW_, NOB = NOB_, NIB = NIB_, OCC = 1;
    static constexpr int NT = 512;                               // eight waves: (pair, pixel part) x two tap halves
    static constexpr int TAP_SPLIT = 5;                          // waves 0..3 take taps 0..4, waves 4..7 taps 5..8
    static constexpr int PIX = TH * TW, OCT = 32 * NOB, ICT = 32 * NIB;
    static constexpr int PS = 4 / (NOB * NIB), PIXW = PIX / PS;  // pixel parts (waves per pair and tap half), pixels per part
    static constexpr int YS = PIX + 1;                           // dY plane stride (odd)
    static constexpr int XR = TH + 2, XC = TW + 2, XS = XC;
    static constexpr int XP = (XR * XS) | 1;                     // X plane stride (odd)
    static constexpr int Y_SIZE = OCT * YS, X_SIZE = ICT * XP, BUF = Y_SIZE + X_SIZE, SMEM_FLOATS = 2 * BUF;
    static_assert(NOB * NIB == 1 || NOB * NIB == 2 || NOB * NIB == 4, "pairs per workgroup");
    static_assert(TW % 8 == 0 && PIXW % 8 == 0 && (PIXW % TW == 0 || TW % PIXW == 0), "a part is whole rows or a piece of one row");
};

struct TiledWgradArgs {
    const float *dY;  // N x OC x H x W
    const float *X;   // N x IC x XH x XW
    float *out;       // partial results [z * PS + part][OC][IC][9]
    u32 OC, IC, H, W;  // H, W: extent of dY (the pixel grid)
    u32 XH, XW, pad;   // extent of X; the window of dY pixel (y, x) starts at X (y - pad, x - pad)
    u32 tiles_x, tiles_per_img, tiles_total;
    u32 ic_tiles, pairs, splits;
};

template <class Cfg>
__global__ void __launch_bounds__(Cfg::NT, 1) wgrad3x3_tiled_kernel(TiledWgradArgs a) {
    constexpr int TH = Cfg::TH, TW = Cfg::TW, PIX = Cfg::PIX, OCT = Cfg::OCT, ICT = Cfg::ICT, YS = Cfg::YS, NT = Cfg::NT;
    constexpr int XR = Cfg::XR, XC = Cfg::XC, XS = Cfg::XS, XP = Cfg::XP, PIXW = Cfg::PIXW;
    __shared__ float smem[Cfg::SMEM_FLOATS];  // 2 x (dY planes, X planes)

    const u32 t = threadIdx.x, bid = blockIdx.x;
    // the blocks of one slice z read the same tiles: ids 8 apart run on the same XCD and share them through its L2
    // (with fewer than 8 slices the ids map plainly, so that every XCD still gets work)
    u32 pair, z;
    if (a.splits >= kXcds) {
        const u32 xcd = bid % kXcds, slot = bid / kXcds;
        pair = slot % a.pairs, z = (slot / a.pairs) * kXcds + xcd;
        if (z >= a.splits) return;
    } else {
        pair = bid % a.pairs, z = bid / a.pairs;
    }
    const u32 oc0 = (pair / a.ic_tiles) * OCT, ic0 = (pair % a.ic_tiles) * ICT;
    const u32 HW = a.H * a.W, XHW = a.XH * a.XW;
    // slice z takes tiles [z T / splits, (z + 1) T / splits): sizes differ by at most one
    const u32 t_begin = u32(uint64_t(z) * a.tiles_total / a.splits), t_end = u32(uint64_t(z + 1) * a.tiles_total / a.splits);

    const int lane = t & 63, wave = t >> 6, i32 = lane & 31, h = lane >> 5;
    const int tap_half = wave >> 2, w4 = wave & 3;
    const int wt = w4 % (Cfg::NOB * Cfg::NIB), part = w4 / (Cfg::NOB * Cfg::NIB);
    const int wob = wt / Cfg::NIB, wib = wt % Cfg::NIB;
    const int p0 = part * PIXW;  // first pixel of this wave's part of the tile
    const int ybase = (wob * 32 + i32) * YS + p0 + 4 * h;
    const int xbase = (wib * 32 + i32) * XP + (p0 / TW) * XS + p0 % TW + 4 * h;

    v16f acc[Cfg::TAP_SPLIT];  // taps T0 .. T0 + 4 (the upper half holds four)
#pragma unroll
    for (int k = 0; k < Cfg::TAP_SPLIT; ++k)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[k][r] = 0.f;

    // ---- staging: thread t owns items t, t + 512, ... of the dY planes and of the X window. The next tile's values are
    // requested before this tile is multiplied and go to the other LDS buffer behind it; a value is judged (inside the
    // image, inside the channels) on its way to LDS, so that no load sits behind a branch.
    constexpr int YQ = OCT * PIX, XQ = ICT * XR * XC;
    constexpr int YNP = (YQ + NT - 1) / NT, XNP = (XQ + NT - 1) / NT;
    float yreg[YNP], xreg[XNP];
    u32 yok = 0, xok = 0;  // bit i: item i counts
    static_assert(YNP <= 32 && XNP <= 32, "validity masks");
    auto fetch = [&](u32 tile) {
        const u32 n = tile / a.tiles_per_img, tl = tile % a.tiles_per_img;
        const int y0 = int(tl / a.tiles_x) * TH, x0 = int(tl % a.tiles_x) * TW;
        // uniform bases, 32-bit byte offsets per item
        const char *dyn = reinterpret_cast<const char *>(a.dY + (size_t(n) * a.OC + oc0) * HW);
        const char *xn = reinterpret_cast<const char *>(a.X + (size_t(n) * a.IC + ic0) * XHW);
        yok = xok = 0;
#pragma unroll
        for (int i = 0; i < YNP; ++i) {
            const u32 e = t + i * NT, j = e / PIX, q = e % PIX;
            const int y = y0 + int(q / TW), x = x0 + int(q % TW);
            const bool ok = (YQ % NT == 0 || e < YQ) && oc0 + j < a.OC && y < int(a.H) && x < int(a.W);
            yok |= ok ? (1u << i) : 0u;
            yreg[i] = *reinterpret_cast<const float *>(dyn + (ok ? (j * HW + u32(y) * a.W + u32(x)) * 4u : 0u));
        }
#pragma unroll
        for (int i = 0; i < XNP; ++i) {
            const u32 e = t + i * NT, j = e / (XR * XC), lr = (e / XC) % XR, lc = e % XC;
            const int y = y0 - int(a.pad) + int(lr), x = x0 - int(a.pad) + int(lc);
            const bool ok = (XQ % NT == 0 || e < XQ) && ic0 + j < a.IC && y >= 0 && y < int(a.XH) && x >= 0 && x < int(a.XW);
            xok |= ok ? (1u << i) : 0u;
            xreg[i] = *reinterpret_cast<const float *>(xn + (ok ? (j * XHW + u32(y) * a.XW + u32(x)) * 4u : 0u));
        }
    };
    constexpr int NITEM = YNP + XNP;
    auto commit_item = [&](int i, float *buf) {  // i is a compile-time constant at every call site
        if (i < YNP) {
            const u32 e = t + i * NT;
            if (YQ % NT == 0 || e < YQ) buf[(e / PIX) * YS + e % PIX] = (yok >> i & 1u) ? yreg[i] : 0.f;
        } else {
            const int k = i - YNP;
            const u32 e = t + k * NT;
            if (XQ % NT == 0 || e < XQ) buf[Cfg::Y_SIZE + (e / (XR * XC)) * XP + ((e / XC) % XR) * XS + e % XC] = (xok >> k & 1u) ? xreg[k] : 0.f;
        }
    };
    // one tile: PIXW / 2 steps of the taps [T0, T1); fragments are read one step ahead (two register sets, scheduler fenced)
    auto compute = [&](auto T0c, auto T1c, const float *buf) {
        constexpr int T0 = decltype(T0c)::value, T1 = decltype(T1c)::value;
        const float *py = buf + ybase, *px = buf + Cfg::Y_SIZE + xbase;
        constexpr int NSTEP = PIXW / 2;
        float av[2], bv[2][T1 - T0];
        auto read_step = [&](int st, int set) {
            const int g = st / 4, s = st % 4, q = 8 * g;  // the group's first pixel, relative to the part's
            av[set] = py[q + s];
#pragma unroll
            for (int k = T0; k < T1; ++k) bv[set][k - T0] = px[(q / TW + k / 3) * XS + q % TW + s + k % 3];
        };
        read_step(0, 0);
#pragma unroll
        for (int st = 0; st < NSTEP; ++st) {
            if (st + 1 < NSTEP) read_step(st + 1, (st + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int k = T0; k < T1; ++k)
                acc[k - T0] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[st & 1], bv[st & 1][k - T0], acc[k - T0], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef std::integral_constant<int, 0> I0;
    typedef std::integral_constant<int, Cfg::TAP_SPLIT> IS;
    typedef std::integral_constant<int, 9> I9;

    fetch(t_begin);
#pragma unroll
    for (int i = 0; i < NITEM; ++i) commit_item(i, smem);
    __syncthreads();
    for (u32 tile = t_begin; tile < t_end; ++tile) {
        const u32 b = (tile - t_begin) & 1;
        // The next tile's values are requested before this one is multiplied and go to the other buffer behind it. (Spreading
        // those LDS stores over the last MFMA steps was measured slower: the first of them waits for loads that are 3 us old.)
        const bool more = tile + 1 < t_end;
        if (more) fetch(tile + 1);
        if (tap_half == 0)
            compute(I0(), IS(), smem + b * Cfg::BUF);
        else
            compute(IS(), I9(), smem + b * Cfg::BUF);
        if (more) {
#pragma unroll
            for (int i = 0; i < NITEM; ++i) commit_item(i, smem + (b ^ 1) * Cfg::BUF);
        }
        __syncthreads();
    }

    // ---- this wave's partial result: register r of tap k is dW[oc = ocb + 8*(r/4) + r%4][ic][k] ------------------------------
    const size_t count = size_t(a.OC) * a.IC * 9;
    float *out = a.out + (size_t(z) * Cfg::PS + part) * count;
    const u32 ocb = oc0 + wob * 32 + 4 * h, ic = ic0 + wib * 32 + i32;
    const int T0 = tap_half ? Cfg::TAP_SPLIT : 0, NTAP = tap_half ? 9 - Cfg::TAP_SPLIT : Cfg::TAP_SPLIT;
    if (ic < a.IC) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const u32 oc = ocb + 8 * (r / 4) + (r % 4);
            if (oc < a.OC) {
                float *dst = out + (size_t(oc) * a.IC + ic) * 9 + T0;
#pragma unroll
                for (int k = 0; k < Cfg::TAP_SPLIT; ++k)
                    if (k < NTAP) dst[k] = acc[k][r];
            }
        }
    }
}

struct TiledWgradPlan {
    u32 tiles_x, tiles_per_img, tiles_total, oc_tiles, ic_tiles, pairs, splits, slices;
    size_t workspace_bytes;
};

template <class Cfg>
inline TiledWgradPlan tiled_wgrad_plan(u32 N, u32 IC, u32 OC, u32 H, u32 W) {
    TiledWgradPlan p;
    p.tiles_x = ceil_div(W, u32(Cfg::TW));
    p.tiles_per_img = p.tiles_x * ceil_div(H, u32(Cfg::TH));
    p.tiles_total = N * p.tiles_per_img;
    p.oc_tiles = ceil_div(OC, u32(Cfg::OCT)), p.ic_tiles = ceil_div(IC, u32(Cfg::ICT));
    p.pairs = p.oc_tiles * p.ic_tiles;
    const u32 target = 256u;  // one eight-wave workgroup per CU
    u32 splits = p.pairs >= target ? 1u : target / p.pairs;
    if (splits > p.tiles_total) splits = p.tiles_total;
    p.splits = splits;
    p.slices = p.splits * Cfg::PS;
    p.workspace_bytes = size_t(p.slices) * OC * IC * 9 * sizeof(float);
    return p;
}

// The tensors' planes are addressed with 32-bit byte offsets inside one image; the tile list is indexed in 32 bits.
inline bool tiled_wgrad_fits(u32 N, u32 IC, u32 OC, u32 H, u32 W) {
    const uint64_t mx = IC > OC ? IC : OC;
    return mx * H * W * 4 <= 0xffffffffull && uint64_t(N) * ceil_div(H, 2u) * ceil_div(W, 8u) <= 0x7fffffffull;
}

// The partial results go to ws (plan.workspace_bytes); dW += their sum in fixed order.
template <class Cfg>
inline int launch_tiled_wgrad(const float *dY, const float *X, float *dW, float *ws, const TiledWgradPlan &p, u32 IC, u32 OC, u32 H, u32 W,
                              u32 XH, u32 XW, u32 pad, hipStream_t s, const char *what) {
    TiledWgradArgs a;
    a.dY = dY, a.X = X, a.out = ws;
    a.OC = OC, a.IC = IC, a.H = H, a.W = W;
    a.XH = XH, a.XW = XW, a.pad = pad;
    a.tiles_x = p.tiles_x, a.tiles_per_img = p.tiles_per_img, a.tiles_total = p.tiles_total;
    a.ic_tiles = p.ic_tiles, a.pairs = p.pairs, a.splits = p.splits;
    const uint64_t wgs = p.splits >= kXcds ? uint64_t(ceil_div(p.splits, kXcds)) * kXcds * p.pairs : uint64_t(p.splits) * p.pairs;
    if (wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL((wgrad3x3_tiled_kernel<Cfg>), dim3(u32(wgs)), dim3(Cfg::NT), 0, s, a);
    if (int st = check_launch(what)) return st;
    return launch_splitk_reduce(ws, dW, OC * IC * 9, p.slices, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, what);
}

}  // namespace crb
