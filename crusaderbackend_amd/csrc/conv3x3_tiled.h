// 3x3 / pad 1 / stride 1 convolution (forward and data gradient) for gfx950 on images of ANY extent: the layers whose width is
// not one of the widths the width-specialised direct kernels are built for (56, 28, 14, 7, 24, 12 ...).
//
// The output image is cut into TH x TW pixel tiles (ragged at the right and bottom edges). A 256-thread workgroup owns one
// tile of one image and OCT output channels and walks the input channels in chunks of CI: per chunk the (TH + 2) x (TW + 2)
// input window (halo included, zero outside the image) of CI channels and the matching OCT x CI x 9 filter slice are staged
// in double-buffered LDS (global -> registers -> LDS, the next chunk's loads in flight while this one is multiplied) and
// fed to v_mfma_f32_32x32x2_f32 with the filters on the row operand and the pixels on the column operand.
//
// Contraction order inside a chunk is the filters' own memory order, k = channel * 9 + tap, so a filter row is a straight
// copy of global memory (16-byte loads and LDS stores when the tensor allows). An MFMA consumes two k per step, one per lane
// half; lane half h takes k = s + h * KC / 2 (KC = 9 CI), i.e. the same tap of channel c + CI / 2: both halves share every
// compile-time address offset, the half is a per-lane base. Filter fragments are read four steps at a time (one 16-byte
// LDS read, row stride 4 mod 32 floats ... 28 mod 32: eight consecutive rows cover all banks), pixel fragments one float per
// step at `lane base + immediate` (the tap shift and the channel plane are the immediate).
//
// v_mfma_f32_32x32x2_f32 (wave64, lane l): A[i = l%32][k = l/32], B[k = l/32][j = l%32], accumulator register r =
// D[i = 8*(r/4) + 4*(l/32) + r%4][j = l%32]: i = output channel, j = pixel, so the 32 lanes of a half-wave store 32
// consecutive pixels (TW of them per image row) of one output channel per instruction.
//
// Data gradient: the same computation on dY with the filter's channel roles swapped and its taps mirrored
// (dX(y, x) = sum dY(y + 1 - fh, x + 1 - fw) W[oc][ic][fh][fw]): only the filter staging and the immediates differ.
//
// The same kernel also serves 5x5 filters, any padding 0 ... F - 1 at stride 1 (the window origin is an argument), the 3x3
// forward pass at stride 2, and the data gradient of strided layers one residue class of input pixels at a time (TiledClass).
#pragma once
#include <type_traits>

#include "igemm_engine.h"

namespace crb {

// F_: filter size (3, or 5 with pad 2 at stride 1); the header's "3x3", "9" and "halo of one" read F x F, F * F and F / 2.
// CLS_: one residue class of a strided data gradient (TiledClass below): F x F (1 ... 4) is the class's tap grid, the output
// pixels are scattered with the layer's stride.
// FW_ (class forms): the tap grid is F_ rows x FW_ columns.
template <int TH_, int TW_, int OCT_, int WP_, int CI_, bool DGRAD_, int OCC_, int S_ = 1, int F_ = 3, bool CLS_ = false, int FW_ = F_>
struct TiledCfg {
    static constexpr bool CLS = CLS_;
    static constexpr int TH = TH_, TW = TW_, OCT = OCT_, WP = WP_, WO = 4 / WP_, CI = CI_, OCC = OCC_, S = S_;
    static constexpr int F = F_, FW = FW_, NT = F_ * FW_, PAD = F_ / 2;
    static constexpr bool DGRAD = DGRAD_;
    static constexpr int PIX = TH * TW, NPB = PIX / 32, NOB = OCT / 32;  // 32-pixel and 32-channel MFMA blocks
    static constexpr int PB = NPB / WP, OB = NOB / WO;                  // blocks per wave
    static constexpr int RB = 32 / TW;                                  // image rows per pixel block
    // staged rows and columns of the input window; LDS row stride. Stride 2 (forward only): a staged row holds the window's
    // even columns (input columns 2 x0 - 1, 2 x0 + 1, ...: taps fw = 0 and 2) and then, HALF floats further, its odd columns
    // (tap fw = 1), so that neighbouring pixels read neighbouring floats for every tap.
    static constexpr int XR = S * (TH - 1) + F, XC = S * (TW - 1) + FW;
    static constexpr int HALF = TW + 2;
    static constexpr int XS = S == 1 ? TW + 4 : 2 * TW + 4;  // >= XC for both filter sizes
    static constexpr int col_pos(int lc) { return S == 1 ? lc : (lc % 2) * HALF + lc / 2; }
    static constexpr int tap_off(int fh, int fw) { return S == 1 ? fh * XS + fw : fh * XS + (fw == 1 ? HALF : fw / 2); }
    static_assert(S == 1 || (S == 2 && !DGRAD_ && F == 3), "stride 2: forward only, 3 x 3 only");
    static_assert(CLS_ ? (F >= 1 && F <= 4 && FW >= 1 && FW <= 4 && DGRAD_ && S == 1) : ((F == 3 || F == 5) && FW == F), "filter size");
    static constexpr int XP = XR * XS;                                  // channel plane stride
    static constexpr int X_SIZE = CI * XP;
    static constexpr int KC = CI * NT, KH = KC / 2;                     // contraction per chunk, per lane half
    static constexpr int WSTR = KC + 4;                                 // filter row stride: 12 mod 32 (3 x 3 and 5 x 5 with CI = 8), 20 (CI = 16)
    static constexpr int W_SIZE = OCT * WSTR;
    static constexpr int SMEM_FLOATS = 2 * (X_SIZE + W_SIZE);
    static_assert(TW == 8 || TW == 16 || TW == 32, "tile width");
    static_assert(WP * WO == 4 && NPB % WP == 0 && NOB % WO == 0 && PB >= 1 && OB >= 1, "wave tiling");
    static_assert(PIX % 32 == 0 && OCT % 32 == 0 && (TH % RB) == 0, "whole MFMA blocks");
    static_assert(CI % 8 == 0 && KH % 4 == 0 && (WSTR % 8) == 4, "16-byte filter fragments, conflict-free rows");
};

// A residue class of the data gradient at stride (sH, sW): the input pixels (y'' sH + py, x'' sW + px) receive only the taps
// fh = fh0 + i sH, fw = fw0 + j sW (i < nfh, j < nfw) and read dY (y'' + qh - i, x'' + qw - j): a unit-stride correlation on the
// class's own pixel grid with an nfh x nfw filter taken out of the layer's, embedded in the kernel's F x F tap grid (the taps
// beyond nfh x nfw are staged as zeros; F rows x FW columns in the class forms).
struct TiledClass {
    int pad_y, pad_x;                  // window origin of class pixel (y'', x'') in dY: (y'' - pad_y, x'' - pad_x), pad = F - 1 - qh, FW - 1 - qw
    u32 fhw, tap0, tap_i, tap_j;       // layer filter: taps per (oc, ic) pair; tap (i, j) of the class is tap0 + i tap_i + j tap_j
    u32 nfh, nfw;
    u32 out_hw, out_w;                 // dX: channel stride, row stride
    u32 osy, osx, oy0, ox0;            // class pixel (y'', x'') is dX pixel (y'' osy + oy0, x'' osx + ox0)
    u32 H, W, tiles_x, tiles_per_img;  // the class's pixel grid and its tiles (set by the launcher)
    u32 tile_begin;                    // the class's first tile in the launch's tile list (set by the launcher)
};
constexpr int kMaxTiledClasses = 16;  // residue classes of one launch (strides up to 4 x 4)

struct TiledArgs {
    const float *Wt;    // filters, OC x IC x 3 x 3 of the forward convolution
    const float *X;     // input of this pass  (forward: X, data gradient: dY), N x C_IN x H x W
    float *Y;           // output of this pass (forward: Y, data gradient: dX), N x C_OUT x H x W
    const float *bias;  // per output channel or nullptr
    u32 C_IN, C_OUT, H, W;  // H, W: extent of the output (the pixel grid)
    u32 IH, IW;             // extent of the staged tensor
    u32 tiles_x, tiles_per_img, oc_tiles, tiles_total;  // tiles_total = N * tiles_per_img
    u32 relu;
    TiledClass cls[kMaxTiledClasses];  // CLS configurations only: the launch's classes, tile lists one behind the other
    u32 ncls;
    u32 pad;  // the window of pixel (y, x) starts at staged (S y - pad, S x - pad): the layer's padding for the forward pass,
              // F - 1 - padding for the data gradient
};

// WVEC (forward only): filter rows are staged with 16-byte loads (C_IN % 4 == 0 and a 16-byte aligned tensor).
template <class Cfg, bool WVEC>
__global__ void __launch_bounds__(kThreads, Cfg::OCC) conv3x3_tiled_kernel(TiledArgs a) {
    constexpr int TH = Cfg::TH, TW = Cfg::TW, OCT = Cfg::OCT, CI = Cfg::CI, PB = Cfg::PB, OB = Cfg::OB;
    constexpr int XR = Cfg::XR, XC = Cfg::XC, XS = Cfg::XS, XP = Cfg::XP, KC = Cfg::KC, KH = Cfg::KH, WSTR = Cfg::WSTR;
    constexpr int F = Cfg::F, FW = Cfg::FW, NT = Cfg::NT;
    __shared__ __attribute__((aligned(16))) float smem[Cfg::SMEM_FLOATS];
    float(*sX)[Cfg::X_SIZE] = reinterpret_cast<float(*)[Cfg::X_SIZE]>(smem);
    float(*sW)[Cfg::W_SIZE] = reinterpret_cast<float(*)[Cfg::W_SIZE]>(smem + 2 * Cfg::X_SIZE);

    const u32 t = threadIdx.x, bid = blockIdx.x;
    // Workgroups are dealt round-robin to the 8 XCDs: the oc_tiles workgroups that read the same input window get ids 8
    // apart, land on the same XCD back to back and share the window through its L2.
    const u32 xcd = bid % kXcds, slot = bid / kXcds;
    const u32 oct = slot % a.oc_tiles;
    u32 rest = (slot / a.oc_tiles) * kXcds + xcd;
    if (rest >= a.tiles_total) return;
    // residue classes: the tile belongs to the last class whose list starts at or before it (uniform over the workgroup)
    u32 ci = 0;
    if constexpr (Cfg::CLS) {
        for (u32 k = 1; k < a.ncls; ++k)
            if (rest >= a.cls[k].tile_begin) ci = k;
        rest -= a.cls[ci].tile_begin;
    }
    const TiledClass &cl = a.cls[ci];
    const u32 gridH = Cfg::CLS ? cl.H : a.H, gridW = Cfg::CLS ? cl.W : a.W;
    const u32 tiles_x = Cfg::CLS ? cl.tiles_x : a.tiles_x, tiles_per_img = Cfg::CLS ? cl.tiles_per_img : a.tiles_per_img;
    const u32 n = rest / tiles_per_img, tile = rest % tiles_per_img;
    const int y0 = int(tile / tiles_x) * TH, x0 = int(tile % tiles_x) * TW;
    const u32 oc0 = oct * OCT;
    const u32 HW = a.H * a.W, IHW = a.IH * a.IW;

    // ---- staging: thread t owns items t, t + 256, ... of the window (channel, row, column) and of the filter slice --------
    // An item's byte offset from the chunk's (uniform) base address does not depend on the chunk: computed once. Loads are
    // issued whatever the item is worth (offset 0 when it is nothing) and the value is judged when it goes to LDS: with a
    // select behind every load, each load would wait for the one before it.
    constexpr int XQ = CI * XR * XC, XNP = (XQ + kThreads - 1) / kThreads;
    constexpr int WITEMS = WVEC ? OCT * KC / 4 : OCT * KC, WNP = (WITEMS + kThreads - 1) / kThreads;
    constexpr u32 kNone = ~0u;
    float xreg[XNP];
    u32 xoff[XNP], woff[WNP];
    typedef typename std::conditional<WVEC, v4f, float>::type WItem;
    WItem wreg[WNP];
    const char *xin = reinterpret_cast<const char *>(a.X + size_t(n) * a.C_IN * IHW);
#pragma unroll
    for (int i = 0; i < XNP; ++i) {
        const u32 e = t + i * kThreads;
        const u32 c = e / (XR * XC), lr = (e / XC) % XR, lc = e % XC;
        const int y = Cfg::S * y0 - (Cfg::CLS ? cl.pad_y : int(a.pad)) + int(lr), x = Cfg::S * x0 - (Cfg::CLS ? cl.pad_x : int(a.pad)) + int(lc);
        const bool ok = (XQ % kThreads == 0 || e < XQ) && y >= 0 && y < int(a.IH) && x >= 0 && x < int(a.IW);
        xoff[i] = ok ? (c * IHW + u32(y) * a.IW + u32(x)) * 4u : kNone;
    }
    // filter slice of chunk c0: LDS row j (output channel oc0 + j) holds k = c * 9 + tap for the chunk's channels c.
    // forward: row j is KC consecutive floats of Wt[oc0 + j] from channel c0 on; data gradient: the OCT * 9 consecutive floats
    // Wt[c0 + c][oc0 ..] hold (row j, tap) for contraction channel c.
#pragma unroll
    for (int i = 0; i < WNP; ++i) {
        const u32 e = t + i * kThreads;
        bool ok = WITEMS % kThreads == 0 || e < WITEMS;
        u32 off;
        if constexpr (Cfg::CLS) {
            const u32 c = e / (OCT * NT), f = e % (OCT * NT), row = f / NT, ti = (f % NT) / FW, tj = (f % NT) % FW;
            ok = ok && oc0 + row < a.C_OUT && ti < cl.nfh && tj < cl.nfw;
            off = (c * a.C_OUT + row) * cl.fhw + cl.tap0 + ti * cl.tap_i + tj * cl.tap_j;
        } else if constexpr (Cfg::DGRAD) {
            const u32 c = e / (OCT * NT), f = e % (OCT * NT);
            ok = ok && oc0 * NT + f < a.C_OUT * NT;
            off = c * a.C_OUT * NT + f;
        } else if constexpr (WVEC) {
            const u32 j = e / (KC / 4), q = e % (KC / 4);
            ok = ok && oc0 + j < a.C_OUT;
            off = j * a.C_IN * NT + 4 * q;
        } else {
            const u32 j = e / KC, k = e % KC;
            ok = ok && oc0 + j < a.C_OUT;
            off = j * a.C_IN * NT + k;
        }
        woff[i] = ok ? off * 4u : kNone;
    }
    // whether item e of the filter slice lies inside the tensor's channels in chunk c0 (ragged last chunk)
    auto w_in_chunk = [&](u32 e, u32 c0) -> bool {
        if constexpr (Cfg::DGRAD) return c0 + e / (OCT * NT) < a.C_IN;
        else if constexpr (WVEC) return c0 * NT + 4 * (e % (KC / 4)) < a.C_IN * NT;  // a 16-byte item never straddles the end: C_IN % 4 == 0
        else return c0 * NT + e % KC < a.C_IN * NT;
    };
    auto fetch = [&](u32 c0) {
        const char *xc = xin + size_t(c0) * IHW * 4;
        const u32 wtaps = Cfg::CLS ? cl.fhw : u32(NT);  // floats per (oc, ic) pair in the filter tensor
        const char *wc = reinterpret_cast<const char *>(Cfg::DGRAD ? a.Wt + (size_t(c0) * a.C_OUT + oc0) * wtaps : a.Wt + (size_t(oc0) * a.C_IN + c0) * NT);
#pragma unroll
        for (int i = 0; i < XNP; ++i) {
            const bool ok = xoff[i] != kNone && c0 + (t + i * kThreads) / (XR * XC) < a.C_IN;
            xreg[i] = *reinterpret_cast<const float *>(xc + (ok ? xoff[i] : 0u));
        }
#pragma unroll
        for (int i = 0; i < WNP; ++i) {
            const bool ok = woff[i] != kNone && w_in_chunk(t + i * kThreads, c0);
            wreg[i] = *reinterpret_cast<const WItem *>(wc + (ok ? woff[i] : 0u));
        }
    };
    auto commit = [&](float *dx, float *dw, u32 c0) {
#pragma unroll
        for (int i = 0; i < XNP; ++i) {
            const u32 e = t + i * kThreads, c = e / (XR * XC);
            const bool ok = xoff[i] != kNone && c0 + c < a.C_IN;
            if (XQ % kThreads == 0 || e < XQ) dx[c * XP + ((e / XC) % XR) * XS + Cfg::col_pos(e % XC)] = ok ? xreg[i] : 0.f;
        }
#pragma unroll
        for (int i = 0; i < WNP; ++i) {
            const u32 e = t + i * kThreads;
            const bool ok = woff[i] != kNone && w_in_chunk(e, c0);
            if (WITEMS % kThreads == 0 || e < WITEMS) {
                if constexpr (Cfg::DGRAD) {
                    const u32 c = e / (OCT * NT), f = e % (OCT * NT);
                    dw[(f / NT) * WSTR + c * NT + f % NT] = ok ? wreg[i] : 0.f;
                } else if constexpr (WVEC) {
                    *reinterpret_cast<v4f *>(dw + (e / (KC / 4)) * WSTR + 4 * (e % (KC / 4))) = ok ? wreg[i] : v4f{0.f, 0.f, 0.f, 0.f};
                } else {
                    dw[(e / KC) * WSTR + e % KC] = ok ? wreg[i] : 0.f;
                }
            }
        }
    };

    // ---- per-lane fragment addressing ---------------------------------------------------------------------------------------
    const int lane = t & 63, wave = t >> 6, j32 = lane & 31, h = lane >> 5;
    const int wp = wave % Cfg::WP, wo = wave / Cfg::WP;
    // this lane's pixel in the wave's first pixel block; block p is RB * p image rows further down
    // A wave with one pixel block takes image rows that are SPREAD apart instead of adjacent ones, so that the rows of a
    // fragment read land on disjoint banks (16-wide tiles: rows r and r + 4, 80 floats = 16 banks apart; 8-wide tiles: rows
    // r, r + 2, r + 4, r + 6, 24 floats apart: banks +24, +16, +8); adjacent rows overlapped on 2 to 4 banks.
    constexpr bool kSpread = PB == 1 && TW < 32 && Cfg::S == 1;
    constexpr int kRowStep = !kSpread ? 1 : (TW == 16 ? TH / 2 : 2);
    const int pix = wp * PB * 32 + j32, pcol = pix % TW;
    const int prow = !kSpread ? pix / TW : (TW == 16 ? wp + kRowStep * (j32 / TW) : (wp / 2) * 8 + wp % 2 + kRowStep * (j32 / TW));
    static_assert(!kSpread || (TW == 16 && Cfg::NPB == TH / 2) || (TW == 8 && TH % 8 == 0), "row spreading covers the tile");
    const int xbase = h * (CI / 2) * XP + Cfg::S * prow * XS + pcol;
    const int wbase = (wo * OB * 32 + j32) * WSTR + h * KH;

    v16f acc[OB][PB];
#pragma unroll
    for (int o = 0; o < OB; ++o)
#pragma unroll
        for (int p = 0; p < PB; ++p)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[o][p][r] = 0.f;

    u32 tapmask = 0;  // class forms: bit t = tap t of the F x FW grid belongs to this workgroup's class
    if constexpr (Cfg::CLS) {
#pragma unroll
        for (int tp = 0; tp < NT; ++tp) tapmask |= (u32(tp / FW) < cl.nfh && u32(tp % FW) < cl.nfw) ? (1u << tp) : 0u;
    }
    // Fragments are read one group of four steps ahead of the MFMAs that consume them (two register sets; the scheduler is
    // fenced so that it neither undoes the pipeline nor hoists every read of the chunk to its top).
    auto compute = [&](const float *cx, const float *cw) {
        const float *xfrag = cx + xbase, *wfrag = cw + wbase;
        v4f wv[2][OB];
        float xv[2][4][PB];
        auto read_group = [&](int sq, int set) {
#pragma unroll
            for (int o = 0; o < OB; ++o) wv[set][o] = *reinterpret_cast<const v4f *>(wfrag + o * 32 * WSTR + 4 * sq);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int s = 4 * sq + e, c = s / NT, tap = s % NT;
                const int fh = Cfg::DGRAD ? F - 1 - tap / FW : tap / FW, fw = Cfg::DGRAD ? FW - 1 - tap % FW : tap % FW;
#pragma unroll
                for (int p = 0; p < PB; ++p) xv[set][e][p] = xfrag[c * XP + Cfg::S * p * Cfg::RB * XS + Cfg::tap_off(fh, fw)];
            }
        };
        read_group(0, 0);
#pragma unroll
        for (int sq = 0; sq < KH / 4; ++sq) {
            if (sq + 1 < KH / 4) read_group(sq + 1, (sq + 1) & 1);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                // class forms: the taps of the shared grid that this class does not have were staged as zeros; their steps
                // are skipped (uniform over the workgroup)
                if (Cfg::CLS && !(tapmask >> ((4 * sq + e) % NT) & 1u)) continue;
#pragma unroll
                for (int o = 0; o < OB; ++o)
#pragma unroll
                    for (int p = 0; p < PB; ++p)
                        acc[o][p] = __builtin_amdgcn_mfma_f32_32x32x2f32(wv[sq & 1][o][e], xv[sq & 1][e][p], acc[o][p], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- main loop over input-channel chunks (double-buffered) -------------------------------------------------------------
    const u32 nchunk = (a.C_IN + CI - 1) / CI;
    fetch(0);
    commit(sX[0], sW[0], 0);
    __syncthreads();
    for (u32 ch = 0; ch < nchunk; ++ch) {
        const u32 b = ch & 1;
        const bool more = ch + 1 < nchunk;
        if (more) fetch((ch + 1) * CI);
        compute(sX[b], sW[b]);
        if (more) commit(sX[b ^ 1], sW[b ^ 1], (ch + 1) * CI);
        __syncthreads();
    }

    // ---- epilogue: register r of block (o, p) is output channel ocb + 8*(r/4) + 4h + r%4 at this lane's pixel ----------------
#pragma unroll
    for (int o = 0; o < OB; ++o) {
        const u32 ocb = oc0 + (wo * OB + o) * 32 + 4 * h;
        float bv[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const u32 oc = ocb + 8 * (r / 4) + (r % 4);
            bv[r] = (a.bias && oc < a.C_OUT) ? a.bias[oc] : 0.f;  // requested together, ahead of the stores
        }
        // ... and awaited here: a wait for them further down would also wait for every store issued before it
#pragma unroll
        for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(bv[r]));
#pragma unroll
        for (int p = 0; p < PB; ++p) {
            const int y = y0 + prow + p * Cfg::RB, x = x0 + pcol;
            const bool pok = y < int(gridH) && x < int(gridW);
            const u32 chan = Cfg::CLS ? cl.out_hw : HW;  // channel stride of the output tensor
            float *dst = a.Y + size_t(n) * a.C_OUT * chan;
            if constexpr (Cfg::CLS)
                dst += pok ? size_t(u32(y) * cl.osy + cl.oy0) * cl.out_w + u32(x) * cl.osx + cl.ox0 : size_t(0);
            else
                dst += size_t(pok ? y : 0) * a.W + (pok ? x : 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const u32 oc = ocb + 8 * (r / 4) + (r % 4);
                float v = acc[o][p][r] + bv[r];
                if (a.relu) v = v > 0.f ? v : 0.f;
                if (pok && oc < a.C_OUT) dst[size_t(oc) * chan] = v;
            }
        }
    }
}

// An item's byte offset inside its image / inside the filter tensor is kept in 32 bits.
inline bool tiled_fits(u32 C_IN, u32 C_OUT, u32 H, u32 W, u32 taps = 9) {
    return uint64_t(C_IN) * H * W * 4 <= 0xffffffffull && uint64_t(C_IN) * C_OUT * taps * 4 <= 0xffffffffull;
}

template <class Cfg>
inline int launch_tiled_args(TiledArgs &a, u32 N, uint64_t tiles, u32 taps, hipStream_t s, const char *what) {
    a.oc_tiles = ceil_div(a.C_OUT, u32(Cfg::OCT));
    const uint64_t wgs = uint64_t(ceil_div(u32(tiles > 0xffffffffull ? 0xffffffffu : tiles), kXcds)) * kXcds * a.oc_tiles;
    if (tiles > 0x7fffffffull || wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    a.tiles_total = u32(tiles);
    if (!tiled_fits(a.C_IN, a.C_OUT, a.IH, a.IW, taps)) return fail(CRB_EINVAL_SHAPE, "%s: image or filter tensor beyond 4 GB", what);
    if (!Cfg::DGRAD && a.C_IN % 4 == 0 && reinterpret_cast<uintptr_t>(a.Wt) % 16 == 0)
        hipLaunchKernelGGL((conv3x3_tiled_kernel<Cfg, !Cfg::DGRAD>), dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    else
        hipLaunchKernelGGL((conv3x3_tiled_kernel<Cfg, false>), dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    return check_launch(what);
}

template <class Cfg>
inline int launch_tiled(const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT, u32 H, u32 W, u32 relu,
                        hipStream_t s, const char *what, u32 IH = 0, u32 IW = 0, int pad = -1) {
    static_assert(!Cfg::CLS, "residue classes are launched by launch_tiled_classes");
    TiledArgs a = {};
    a.Wt = Wt, a.X = X, a.Y = Y, a.bias = bias;
    a.C_IN = C_IN, a.C_OUT = C_OUT, a.H = H, a.W = W;
    a.IH = IH ? IH : H, a.IW = IW ? IW : W;
    a.pad = pad < 0 ? u32(Cfg::PAD) : u32(pad);
    a.tiles_x = ceil_div(W, u32(Cfg::TW));
    a.tiles_per_img = a.tiles_x * ceil_div(H, u32(Cfg::TH));
    a.relu = relu;
    return launch_tiled_args<Cfg>(a, N, uint64_t(N) * a.tiles_per_img, Cfg::NT, s, what);
}

// One launch over `ncls` residue classes of a strided data gradient (every class with at most F x F taps): dX's class pixels
// from dY (N x C_IN x OH x OW) and the layer's filters. cls[k].H / W is the class's pixel grid; the tile fields are set here.
template <class Cfg>
inline int launch_tiled_classes(const float *Wt, const float *dY, float *dX, u32 N, u32 C_IN, u32 C_OUT, u32 OH, u32 OW, TiledClass *cls,
                                u32 ncls, hipStream_t s, const char *what) {
    static_assert(Cfg::CLS, "kernel form");
    if (ncls == 0 || ncls > u32(kMaxTiledClasses)) return fail(CRB_EINVAL_SHAPE, "%s: %u residue classes in one launch", what, ncls);
    TiledArgs a = {};
    a.Wt = Wt, a.X = dY, a.Y = dX, a.bias = nullptr;
    a.C_IN = C_IN, a.C_OUT = C_OUT, a.H = 0, a.W = 0, a.IH = OH, a.IW = OW;
    a.pad = 0, a.tiles_x = 0, a.tiles_per_img = 0, a.relu = 0;
    uint64_t tiles = 0;
    for (u32 k = 0; k < ncls; ++k) {
        cls[k].tiles_x = ceil_div(cls[k].W, u32(Cfg::TW));
        cls[k].tiles_per_img = cls[k].tiles_x * ceil_div(cls[k].H, u32(Cfg::TH));
        if (tiles > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
        cls[k].tile_begin = u32(tiles);
        tiles += uint64_t(N) * cls[k].tiles_per_img;
        a.cls[k] = cls[k];
    }
    a.ncls = ncls;
    return launch_tiled_args<Cfg>(a, N, tiles, cls[0].fhw, s, what);
}

}  // namespace crb
