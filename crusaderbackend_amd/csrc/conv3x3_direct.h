// Direct 3x3 / pad 1 convolution for gfx950, stride 1 or 2 (and 1x1 / stride 1): forward and data gradient in one template.
//
// A workgroup (4 wave64) owns ROWS rows of a "pixel grid" of one image and OCT output channels. The grid is the
// output image for the forward pass and for the stride-1 data gradient; for the stride-2 data gradient it is the
// dY image, each of whose pixels yields a 2x2 block of dX. The contraction runs over input channels in chunks of CI:
// for each chunk the raw input rows the tile needs (with their halo, zero outside the image) and the matching
// OCT x CI x 9 filter slice are staged in LDS, and every wave feeds v_mfma_f32_16x16x4_f32 directly from them.
// Inside a chunk the contraction index is ordered tap-major (k = tap*(CI+1) + channel), so an MFMA step covers one
// tap and four consecutive channels: the im2col gather is a per-lane base address (pixel + (lane/16) channel planes)
// plus a compile-time immediate per step, and the inner loop contains nothing but ds_read and MFMA. Fragments are
// read PF steps ahead of the MFMAs that consume them (explicit software pipeline; the scheduler is fenced so it
// cannot undo it).
//
// MFMA 16x16x4 f32 mapping (wave64, lane l): A value = A[i = l%16][k = l/16], B value = B[k = l/16][j = l%16],
// accumulator register r = D[i = 4*(l/16) + r][j = l%16]. Here i = pixel within a 16-pixel block of the grid,
// j = output channel within a 16-channel block, so a lane ends up with 4 consecutive grid pixels of one output
// channel: 16-byte stores, and bias / ReLU are per-lane scalars.
//
// Variants:
//   forward, stride S: grid pixel (y, x) reads input (S*y + fh - 1, S*x + fw - 1).
//   data gradient, stride 1: the same computation on dY with the filter's channel roles swapped and its taps
//     mirrored: grid pixel (y, x) reads dY (y + 1 - fh, x + 1 - fw).
//   data gradient, stride 2: dX (2y'+py, 2x'+px) only receives the taps with fh = 1 - py (mod 2), fw = 1 - px (mod 2):
//     four interleaved sub-convolutions of dY with 1, 2, 2 and 4 taps. Each tap accumulates into the accumulator of
//     its parity class, reading dY (y' + (fh == 0), x' + (fw == 0)); the structural zeros a zero-upsampled
//     formulation would multiply are never touched. The two column parities held by a lane interleave into 8
//     consecutive dX floats per row parity.
#pragma once
#include <type_traits>

#include "igemm_engine.h"

namespace crb {

// NBUF_ = 2: double-buffered chunk pipeline (any C_IN). NBUF_ = 1: the whole contraction is one chunk (C_IN <= CI),
// half the LDS, so more workgroups fit on a CU and overlap each other's staging.
// FS_ = 3: 3x3 filter with pad 1. FS_ = 1: 1x1 filter, no padding, stride 1 (one tap, no halo) — the bottleneck layers,
// which are bandwidth-bound: same staging and MFMA mapping, the contraction is just the channel chunk.
// PGS_ > 1 (single-chunk configurations only): a wave finishes its pixel blocks in PGS groups, one after the other, and
// stores each group as soon as it is complete, so the stores of all groups but the last overlap the MFMAs of the next.
// KS_ = 2 (single-chunk configurations only): the contraction runs in two halves of the chunk's channels. The
// first half's rows are requested first and multiplied (all pixel blocks) while the second half's are still arriving; the
// second half then runs group by group with the stores in between, as with KS_ = 1.
template <int W_, int ROWS_, int CI_, int OCT_, int PBW_, int OBW_, bool DGRAD_, int OCC_, int NBUF_ = 2, int S_ = 1, int FS_ = 3, int PGS_ = 1,
          int KS_ = 1>
struct DirectCfg {
    static constexpr int W = W_, ROWS = ROWS_, CI = CI_, OCT = OCT_, PBW = PBW_, OBW = OBW_, OCC = OCC_, NBUF = NBUF_, S = S_;
    static constexpr int FS = FS_, NT = FS_ * FS_;  // filter size, taps
    static constexpr int PGS = PGS_, PGC = PBW_ / PGS_;  // pixel-block groups per wave, blocks per group
    static constexpr int KS = KS_;
    static constexpr bool STREAM_OUT = PGS_ > 1 || FS_ == 1;  // non-temporal output stores (see store_out)
    static constexpr bool DGRAD = DGRAD_;
    // W = 4: the grid is a 4x4 image and a tile is ROWS / 4 whole images stacked, each staged with its own halo rows
    static constexpr bool MI = W_ == 4;
    static constexpr int IMGS = MI ? ROWS_ / 4 : 1;
    static constexpr bool DG2 = DGRAD && S == 2;  // stride-2 data gradient (4 parity classes)
    static constexpr bool FW2 = !DGRAD && S == 2; // stride-2 forward
    static constexpr int NPH = DG2 ? 4 : 1;       // accumulator sets per MFMA tile
    static constexpr int TP = ROWS * W;           // grid pixels per workgroup tile
    static constexpr int NPB = TP / 16;           // 16-pixel blocks
    static constexpr int NOB = OCT / 16;          // 16-channel blocks
    static constexpr int NPBW = NPB / PBW;        // wave groups along pixels
    static constexpr int NOBW = NOB / OBW;        // wave groups along channels
    // staged input: row width, row count, the input row LDS row 0 holds (ROW0_MUL*r0 + ROW0_ADD for first grid row r0)
    static constexpr int SW = FW2 ? 2 * W : W;
    static constexpr int XR = MI ? IMGS * 6 : (FS == 1 ? ROWS : (DG2 ? ROWS + 1 : S * (ROWS - 1) + 3));
    static constexpr int ROW0_MUL = FW2 ? 2 : 1;
    static constexpr int ROW0_ADD = (DG2 || FS == 1) ? 0 : -1;
    // Stride-2 forward: a staged row holds the input row's odd columns (with the left halo column -1 in front) and then
    // its even columns, W floats each, so that neighbouring grid pixels are neighbouring floats for every tap (fw = 0 and
    // 2 read the odd half, fw = 1 the even half) and a fragment read touches 16 consecutive banks per lane group, as at
    // stride 1, instead of every other bank twice.
    static constexpr int RSTEP = FW2 ? 2 : 1;     // staged rows between neighbouring grid rows
    static constexpr int XS = SW + 8;  // LDS row stride: 3 pad, left halo, SW interior (16-byte aligned), right halo, 3 pad
    // channel plane stride (floats): the four lane groups (lane/16) of a fragment read sit one plane apart;
    // 16 mod 32 (8 mod 32 for the 2-row blocks of W = 8) puts them on disjoint LDS banks. Multiple of 4.
    static constexpr int XP_MIN = XR * XS;
    static constexpr int XP_RES = W == 8 ? 8 : 16;
    static constexpr int XP = XP_MIN + ((XP_RES - XP_MIN % 32) + 32) % 32;
    static constexpr int NSTEP = CI * NT / 4;     // MFMA steps per chunk
    static constexpr int CQ = CI / 4;             // steps per tap
    static constexpr int MPS = PBW * OBW;         // MFMAs per step
    static constexpr int CIP = CI + 1;            // k index of (tap, channel) in a filter row is tap*CIP + channel: odd tap stride
    static constexpr int WSTR_MIN = NT * CIP;      // filter row stride == 2 mod 4: the 32 lanes of a half-wave (16 rows x 2 k) hit distinct banks
    static constexpr int WSTR = WSTR_MIN + ((2 - WSTR_MIN % 4) + 4) % 4;
    static constexpr int X_SIZE = CI * XP;
    static constexpr int W_SIZE = OCT * WSTR;
    static constexpr int SMEM_FLOATS = NBUF_ * (X_SIZE + W_SIZE);
    static_assert(W == 4 || W == 8 || W == 16 || W == 32, "grid width");
    static_assert(!MI || (S == 1 && FS == 3 && ROWS % 4 == 0), "stacked 4x4 images: 3x3 stride 1 only");
    static_assert(S == 1 || S == 2, "stride");
    static_assert(FS == 3 || (FS == 1 && S == 1), "1x1 filters are handled at stride 1 only");
    static_assert(TP % 16 == 0 && NPB % PBW == 0 && NOB % OBW == 0 && NPBW * NOBW == 4, "wave tiling must use 4 waves");
    static_assert((PBW * 16) % W == 0 || PBW == 1, "a wave's pixel blocks must start on a row boundary");
    static_assert(CI % 4 == 0, "chunk channel count");
    static_assert(PBW % PGS == 0 && (PGS == 1 || NBUF == 1), "pixel groups need a single-chunk configuration");
    static_assert(KS == 1 || (KS == 2 && NBUF == 1 && (CI / 4) % 2 == 0 && !(W_ == 4)), "two-half contraction: single chunk, whole steps per half");

    // LDS offset of tap (fh, fw) relative to the lane's pixel base (which points one float left of the pixel)
    static constexpr int tap_off(int tap) {
        const int fh = tap / 3, fw = tap % 3;
        if (FS == 1) return 1;  // the pixel itself: interior starts one float past the lane's base
        if (DG2) return (fh == 0 ? 1 : 0) * XS + (fw == 0 ? 1 : 0) + 1;
        if (DGRAD) return (2 - fh) * XS + (2 - fw);
        if (FW2) return fh * XS + (fw == 0 ? 0 : (fw == 2 ? 1 : W + 1));
        return fh * XS + fw;
    }
    // parity class 2*py + px of dX that tap (fh, fw) contributes to (stride-2 data gradient), else 0
    static constexpr int tap_phase(int tap) { return DG2 ? (tap / 3 == 1 ? 0 : 2) + (tap % 3 == 1 ? 0 : 1) : 0; }
    static constexpr int pix_off(int q) {
        if (MI) return ((q / 16) * 6 + (q % 16) / 4) * XS + q % 4;  // image q/16 of the stack, 6 staged rows each
        return (q / W) * RSTEP * XS + (q % W);
    }
};

// Output stores. STREAM: non-temporal (written through as they are issued instead of sitting in L2 until the release
// at the end of the kernel writes every dirty line back at once). It pays when a workgroup's stores are spread over its
// lifetime (pixel groups), so that the write-back overlaps the remaining MFMAs: 16 -> 16 @ 32x32, batch 128 (8.4 MB of
// output) 9.1 -> 8.6 us per launch; it changes nothing when all stores come at the end, and costs the stride-2 data
// gradient 0.3 us. The 1x1 layers (bandwidth-bound, outputs of 12-50 MB) always stream: 204 -> 48 @ 32x32 21.5 -> 20.5 us.
template <bool STREAM>
__device__ __forceinline__ void store_out(float *p, v4f v) {
    if constexpr (STREAM)
        __builtin_nontemporal_store(v, reinterpret_cast<v4f *>(p));
    else
        *reinterpret_cast<v4f *>(p) = v;
}

struct DirectArgs {
    const float *Wt;    // filters, OC x IC x 3 x 3 of the forward convolution
    const float *X;     // input of this pass  (forward: X, dgrad: dY), N x C_IN x in_H x SW
    float *Y;           // output of this pass (forward: Y, dgrad: dX), N x C_OUT x (grid_H x W, or twice that for stride-2 dgrad)
    const float *bias;  // per output channel or nullptr
    u32 C_IN, C_OUT;
    u32 in_H;           // rows of the staged tensor
    u32 grid_H;         // rows of the pixel grid
    u32 tiles_per_img, oc_tiles, tiles_total;  // tiles_total = N * tiles_per_img (stacked 4x4 images: ceil(N / IMGS))
    u32 n_images;
    u32 relu;
    u32 xcd_shift;      // log2 of the run of consecutive tiles that shares an XCD (0: tiles are dealt to XCDs one by one)
};

// The work of workgroup `bid` of the grid launch_direct sizes; `smem` = Cfg::SMEM_FLOATS floats of LDS, 16-byte aligned.
// A device function so that a kernel can run it next to another kind of work in one launch.
template <class Cfg>
__device__ __forceinline__ void conv3x3_body(const DirectArgs &a, const u32 bid, float *smem) {
    constexpr int W = Cfg::W, ROWS = Cfg::ROWS, CI = Cfg::CI, OCT = Cfg::OCT, PBW = Cfg::PBW, OBW = Cfg::OBW;
    constexpr int XS = Cfg::XS, XR = Cfg::XR, XP = Cfg::XP, WSTR = Cfg::WSTR, SW = Cfg::SW;
    constexpr int NBUF = Cfg::NBUF, NPH = Cfg::NPH;
    float(*sX)[Cfg::X_SIZE] = reinterpret_cast<float(*)[Cfg::X_SIZE]>(smem);
    float(*sW)[Cfg::W_SIZE] = reinterpret_cast<float(*)[Cfg::W_SIZE]>(smem + NBUF * Cfg::X_SIZE);

    const u32 t = threadIdx.x;
    // Workgroups are dealt round-robin to the 8 XCDs. Decode the id so that the oc_tiles workgroups that read the same
    // input rows get ids 8 apart: they land on the same XCD, back to back, and share those rows through its L2.
    const u32 xcd = bid % kXcds, slot = bid / kXcds;
    const u32 oct = slot % a.oc_tiles;
    // runs of 2^xcd_shift consecutive tiles stay on one XCD (the XCD that a companion kernel body reads the same rows on)
    const u32 sp = slot / a.oc_tiles;
    const u32 rest = ((((sp >> a.xcd_shift) * kXcds) + xcd) << a.xcd_shift) + (sp & ((1u << a.xcd_shift) - 1u));
    if (rest >= a.tiles_total) return;
    const u32 tile = Cfg::MI ? 0 : rest % a.tiles_per_img;
    const u32 n = Cfg::MI ? rest * Cfg::IMGS : rest / a.tiles_per_img;  // (first) image of this tile
    const int r0 = int(tile) * ROWS;  // first grid row of this tile
    const int srow0 = Cfg::ROW0_MUL * r0 + Cfg::ROW0_ADD;  // input row held by LDS row 0
    const u32 oc0 = oct * OCT;
    const u32 in_HW = a.in_H * SW;

    // ---- staging helpers ----------------------------------------------------------------------------
    // input rows: CI planes x XR rows x SW/4 quads
    constexpr int XQ = CI * XR * (SW / 4);
    constexpr int XNP = (XQ + kThreads - 1) / kThreads;
    // filter slice: one (filter row j, chunk channel c) pair per item, 9 contiguous taps each
    constexpr int WQ = OCT * CI;
    constexpr int WNP = (WQ + kThreads - 1) / kThreads;
    constexpr int NT = Cfg::NT;
    v4f xreg[XNP];
    float wreg[WNP * NT];
    bool xok[XNP], wok[WNP];  // two-half form: what a request that was issued regardless is worth

    auto fetch_x = [&](u32 c0, auto lo, auto hi) {
#pragma unroll
        for (int i = decltype(lo)::value; i < decltype(hi)::value; ++i) {
            const u32 e = t + i * kThreads;
            v4f v = {0.f, 0.f, 0.f, 0.f};
            if constexpr (Cfg::KS == 2) {
                // Requested whatever the row is (a halo row outside the image or a channel past the extent reads row 0 of
                // channel 0 and is zeroed on the way to LDS): behind a branch the compiler could not tell how many requests are
                // in flight, and the wait for the first half would cover the second half too.
                const u32 q = e % (SW / 4), lr = (e / (SW / 4)) % XR, c = e / ((SW / 4) * XR);
                const int row = srow0 + int(lr);
                const bool ok = row >= 0 && row < int(a.in_H) && c0 + c < a.C_IN && (XQ % kThreads == 0 || e < XQ);
                xok[i] = ok;
                v = *reinterpret_cast<const v4f *>(a.X + (size_t(n) * a.C_IN + (ok ? c0 + c : 0u)) * in_HW + (ok ? u32(row) : 0u) * SW + 4 * q);
            } else if (XQ % kThreads == 0 || e < XQ) {
                const u32 q = e % (SW / 4), lr = (e / (SW / 4)) % XR, c = e / ((SW / 4) * XR);
                // stacked images: staged row lr is row lr % 6 - 1 of image lr / 6 (rows -1 and 4 are its halo)
                const int row = Cfg::MI ? int(lr % 6) - 1 : srow0 + int(lr);
                const u32 img = Cfg::MI ? n + lr / 6 : n;
                if (row >= 0 && row < int(a.in_H) && c0 + c < a.C_IN && (!Cfg::MI || img < a.n_images))
                    v = *reinterpret_cast<const v4f *>(a.X + (size_t(img) * a.C_IN + c0 + c) * in_HW + u32(row) * SW + 4 * q);
            }
            xreg[i] = v;
        }
    };
    auto fetch_w = [&](u32 c0) {
#pragma unroll
        for (int i = 0; i < WNP; ++i) {
            const u32 e = t + i * kThreads;
            // forward: lanes run over chunk channels c (filter row j = e / CI): W[oc0 + j][c0 + c][0..8]
            // dgrad:   lanes run over filter rows j (gradient channel c = e / OCT): W[c0 + c][oc0 + j][0..8]
            const u32 j = Cfg::DGRAD ? e % OCT : e / CI, c = Cfg::DGRAD ? e / OCT : e % CI;
            const float *src = Cfg::DGRAD ? a.Wt + ((size_t(c0) + c) * a.C_OUT + oc0 + j) * NT
                                          : a.Wt + ((size_t(oc0) + j) * a.C_IN + c0 + c) * NT;
            // channels past the tensor's extent (ragged last chunk / last channel tile) are staged as zeros
            const bool ok = (WQ % kThreads == 0 || e < WQ) && c0 + c < a.C_IN && oc0 + j < a.C_OUT;
            if constexpr (Cfg::KS == 2) {
                static_assert(!Cfg::DGRAD || Cfg::KS == 1, "two-half form: forward filter addressing only");
                wok[i] = ok;
                const float *src0 = a.Wt + ((size_t(oc0) + (ok ? j : 0u)) * a.C_IN + c0 + (ok ? c : 0u)) * NT;
#pragma unroll
                for (int tap = 0; tap < NT; ++tap) wreg[i * NT + tap] = src0[tap];
            } else if (ok) {  // one branch around the 9 contiguous loads keeps them mergeable into wide loads
#pragma unroll
                for (int tap = 0; tap < NT; ++tap) wreg[i * NT + tap] = src[tap];
            } else {
#pragma unroll
                for (int tap = 0; tap < NT; ++tap) wreg[i * NT + tap] = 0.f;
            }
        }
    };

    using std::integral_constant;
    typedef integral_constant<int, 0> XLo;
    typedef integral_constant<int, XNP> XHi;
    auto fetch = [&](u32 c0) {
        fetch_x(c0, XLo{}, XHi{});
        fetch_w(c0);
    };

    auto commit_x = [&](float *dX, auto lo, auto hi) {
#pragma unroll
        for (int i = decltype(lo)::value; i < decltype(hi)::value; ++i) {
            const u32 e = t + i * kThreads;
            if (XQ % kThreads == 0 || e < XQ) {
                const u32 q = e % (SW / 4), lr = (e / (SW / 4)) % XR, c = e / ((SW / 4) * XR);
                if constexpr (Cfg::FW2) {  // columns 4q..4q+3: odd ones to the first half of the row, even ones to the second
                    *reinterpret_cast<v2f *>(dX + c * XP + lr * XS + 4 + 2 * q) = v2f{xreg[i].y, xreg[i].w};
                    *reinterpret_cast<v2f *>(dX + c * XP + lr * XS + 4 + W + 2 * q) = v2f{xreg[i].x, xreg[i].z};
                } else if constexpr (Cfg::KS == 2) {
                    *reinterpret_cast<v4f *>(dX + c * XP + lr * XS + 4 + 4 * q) = xok[i] ? xreg[i] : v4f{0.f, 0.f, 0.f, 0.f};
                } else {
                    *reinterpret_cast<v4f *>(dX + c * XP + lr * XS + 4 + 4 * q) = xreg[i];
                }
            }
        }
    };
    auto commit_w = [&](float *dW) {
#pragma unroll
        for (int i = 0; i < WNP; ++i) {
            const u32 e = t + i * kThreads;
            if (WQ % kThreads == 0 || e < WQ) {
                const u32 j = Cfg::DGRAD ? e % OCT : e / CI, c = Cfg::DGRAD ? e / OCT : e % CI;
#pragma unroll
                for (int tap = 0; tap < NT; ++tap)
                    dW[j * WSTR + tap * Cfg::CIP + c] = (Cfg::KS == 2 && !wok[i]) ? 0.f : wreg[i * NT + tap];
            }
        }
    };
    auto commit = [&](float *dX, float *dW) {
        commit_x(dX, XLo{}, XHi{});
        commit_w(dW);
    };

    // ---- zero the halo columns of both buffers once (never overwritten afterwards) ---------------------
    for (u32 e = t; e < u32(NBUF) * CI * XR; e += kThreads) {
        float *row = &sX[0][0] + (e / (CI * XR)) * Cfg::X_SIZE + ((e % (CI * XR)) / XR) * XP + (e % XR) * XS;
        row[3] = 0.f;
        row[SW + 4] = 0.f;
    }

    // ---- per-lane fragment addressing ---------------------------------------------------------------------
    const int lane = t & 63, wave = t >> 6;
    const int wp = wave % Cfg::NPBW, wo = wave / Cfg::NPBW;
    const int li = lane & 15, kq = lane >> 4;
    // grid pixel of this lane in the wave's first block; lane group kq reads channel plane kq of each 4-channel step
    const int q0 = (wp * PBW) * 16 + li;
    const int xbase = kq * XP + Cfg::pix_off(q0) + 3;
    const int wbase = (wo * OBW * 16 + li) * WSTR + kq;

    // The bias values of this lane's output channels, requested before the main loop: a load in the epilogue would wait,
    // through the in-order memory counter, for every store issued before it.
    float bias_v[OBW];
#pragma unroll
    for (int o = 0; o < OBW; ++o) {
        const u32 oc = oc0 + (wo * OBW + o) * 16 + li;
        bias_v[o] = (a.bias && oc < a.C_OUT) ? a.bias[oc] : 0.f;
    }

    v4f acc[NPH][PBW][OBW];
#pragma unroll
    for (int ph = 0; ph < NPH; ++ph)
#pragma unroll
        for (int p = 0; p < PBW; ++p)
#pragma unroll
            for (int o = 0; o < OBW; ++o) acc[ph][p][o] = v4f{0.f, 0.f, 0.f, 0.f};

    // MFMAs of one chunk for the pixel blocks [P0, P0 + PC) of this wave, channel quads [Q0, Q0 + QN) of every tap
    auto compute_k = [&](const float *cx, const float *cw, auto p0c, auto pcc, auto q0c, auto qnc) {
        constexpr int P0 = decltype(p0c)::value, PC = decltype(pcc)::value;
        constexpr int Q0 = decltype(q0c)::value, CQ = decltype(qnc)::value, NSTEP = CQ * Cfg::NT;
        constexpr int MPS = PC * OBW, PF = (8 / MPS) < 1 ? 1 : ((8 / MPS) > 4 ? 4 : (8 / MPS));  // read-ahead (steps)
        const float *px = cx + xbase, *pw = cw + wbase;
        float av[PF + 1][PC], bv[PF + 1][OBW];
        auto read_step = [&](int s, int slot) {
            const int tap = s / CQ, cq = Q0 + s % CQ;
            const int xo = cq * 4 * XP + Cfg::tap_off(tap);
#pragma unroll
            for (int p = 0; p < PC; ++p) av[slot][p] = px[xo + Cfg::pix_off((P0 + p) * 16)];
#pragma unroll
            for (int o = 0; o < OBW; ++o) bv[slot][o] = pw[o * 16 * WSTR + tap * Cfg::CIP + 4 * cq];
        };
#pragma unroll
        for (int s = 0; s < PF && s < NSTEP; ++s) read_step(s, s % (PF + 1));
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            if (s + PF < NSTEP) read_step(s + PF, (s + PF) % (PF + 1));
            __builtin_amdgcn_sched_barrier(0);
            const int ph = Cfg::tap_phase(s / CQ);
#pragma unroll
            for (int p = 0; p < PC; ++p)
#pragma unroll
                for (int o = 0; o < OBW; ++o)
                    acc[ph][P0 + p][o] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s % (PF + 1)][p], bv[s % (PF + 1)][o], acc[ph][P0 + p][o], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    typedef integral_constant<int, 0> AllP0;
    typedef integral_constant<int, PBW> AllPC;
    auto compute = [&](const float *cx, const float *cw, auto p0c, auto pcc) {
        compute_k(cx, cw, p0c, pcc, integral_constant<int, 0>{}, integral_constant<int, Cfg::CQ>{});
    };

    // ---- epilogue for the pixel blocks [p_lo, p_lo + p_cnt): a lane holds 4 consecutive grid pixels of one output channel ----
    auto store = [&](int p_lo, int p_cnt) {
#pragma unroll
        for (int o = 0; o < OBW; ++o) {
            const u32 oc = oc0 + (wo * OBW + o) * 16 + li;
            if (oc >= a.C_OUT) continue;
            const float b = bias_v[o];
#pragma unroll
            for (int p = 0; p < PBW; ++p) {
                if (p < p_lo || p >= p_lo + p_cnt) continue;
                const int q = (wp * PBW + p) * 16 + 4 * kq;
                const u32 gy = Cfg::MI ? u32((q % 16) / 4) : u32(r0 + q / W), gx = u32(q % W);
                const u32 img = Cfg::MI ? n + u32(q / 16) : n;
                if (Cfg::MI && img >= a.n_images) continue;
                if constexpr (Cfg::DG2) {
                    // grid pixel (gy, gx..gx+3) -> dX rows 2gy, 2gy+1, columns 2gx .. 2gx+7 (column parities interleaved)
                    float *base = a.Y + ((size_t(n) * a.C_OUT + oc) * (2 * a.grid_H) + 2 * gy) * (2 * W) + 2 * gx;
#pragma unroll
                    for (int py = 0; py < 2; ++py) {
                        const v4f e = acc[2 * py][p][o], d = acc[2 * py + 1][p][o];  // px = 0, px = 1
                        store_out<Cfg::STREAM_OUT>(base + py * 2 * W, v4f{e.x, d.x, e.y, d.y});
                        store_out<Cfg::STREAM_OUT>(base + py * 2 * W + 4, v4f{e.z, d.z, e.w, d.w});
                    }
                } else {
                    v4f v = acc[0][p][o];
                    v.x += b, v.y += b, v.z += b, v.w += b;
                    if (a.relu) {
                        v.x = v.x > 0.f ? v.x : 0.f, v.y = v.y > 0.f ? v.y : 0.f;
                        v.z = v.z > 0.f ? v.z : 0.f, v.w = v.w > 0.f ? v.w : 0.f;
                    }
                    store_out<Cfg::STREAM_OUT>(a.Y + ((size_t(img) * a.C_OUT + oc) * a.grid_H + gy) * W + gx, v);
                }
            }
        }
    };

    // ---- main loop over input-channel chunks (double-buffered) ---------------------------------------------
    if constexpr (Cfg::KS == 2) {
        // items [0, XH) of a thread's rows cover the first half of the channels (items run channel-major over the workgroup)
        constexpr int HQ = Cfg::CQ / 2;
        constexpr int XH = ((CI / 2) * XR * (SW / 4) + kThreads - 1) / kThreads;
        typedef integral_constant<int, XH> XMid;
        fetch_w(0);
        __builtin_amdgcn_sched_barrier(0);
        fetch_x(0, XLo{}, XMid{});
        __builtin_amdgcn_sched_barrier(0);  // the second half's requests stay behind the first half's
        fetch_x(0, XMid{}, XHi{});
        __builtin_amdgcn_sched_barrier(0);
        commit_w(sW[0]);
        commit_x(sX[0], XLo{}, XMid{});
        lds_barrier();
        compute_k(sX[0], sW[0], AllP0{}, AllPC{}, integral_constant<int, 0>{}, integral_constant<int, HQ>{});
        commit_x(sX[0], XMid{}, XHi{});
        lds_barrier();
        auto group = [&](auto g) {
            constexpr int G = decltype(g)::value;
            compute_k(sX[0], sW[0], integral_constant<int, G * Cfg::PGC>{}, integral_constant<int, Cfg::PGC>{}, integral_constant<int, HQ>{},
                      integral_constant<int, Cfg::CQ - HQ>{});
            store(G * Cfg::PGC, Cfg::PGC);
        };
        group(integral_constant<int, 0>{});
        if constexpr (Cfg::PGS > 1) group(integral_constant<int, 1>{});
        if constexpr (Cfg::PGS > 2) group(integral_constant<int, 2>{});
        if constexpr (Cfg::PGS > 3) group(integral_constant<int, 3>{});
        return;
    }
    fetch(0);
    commit(sX[0], sW[0]);
    __syncthreads();
    if constexpr (NBUF == 1 && Cfg::PGS > 1) {
        // group by group: the stores of a finished group drain while the next group's MFMAs run
        auto group = [&](auto g) {
            constexpr int G = decltype(g)::value;
            compute(sX[0], sW[0], integral_constant<int, G * Cfg::PGC>{}, integral_constant<int, Cfg::PGC>{});
            store(G * Cfg::PGC, Cfg::PGC);
        };
        group(integral_constant<int, 0>{});
        if constexpr (Cfg::PGS > 1) group(integral_constant<int, 1>{});
        if constexpr (Cfg::PGS > 2) group(integral_constant<int, 2>{});
        if constexpr (Cfg::PGS > 3) group(integral_constant<int, 3>{});
        return;
    } else if constexpr (NBUF == 1) {
        compute(sX[0], sW[0], AllP0{}, AllPC{});
    } else {
        const u32 nchunk = (a.C_IN + CI - 1) / CI;
        for (u32 ch = 0; ch < nchunk; ++ch) {
            const bool more = ch + 1 < nchunk;
            if (more) fetch((ch + 1) * CI);
            if (ch & 1) {
                compute(sX[NBUF - 1], sW[NBUF - 1], AllP0{}, AllPC{});
                if (more) commit(sX[0], sW[0]);
            } else {
                compute(sX[0], sW[0], AllP0{}, AllPC{});
                if (more) commit(sX[NBUF - 1], sW[NBUF - 1]);
            }
            __syncthreads();
        }
    }
    store(0, PBW);
}

template <class Cfg>
__global__ void __launch_bounds__(kThreads, Cfg::OCC) conv3x3_kernel(DirectArgs a) {
    __shared__ __attribute__((aligned(16))) float smem[Cfg::SMEM_FLOATS];
    conv3x3_body<Cfg>(a, blockIdx.x, smem);
}

// Shape gate of one configuration. Channel counts need not divide CI / OCT: ragged chunks and tiles are zero-filled.
// (grid_H, grid_W) = extent of the pixel grid: the output image, or dY for the stride-2 data gradient.
template <class Cfg>
inline bool direct_fits(u32 C_IN, u32 grid_H, u32 grid_W) {
    if (Cfg::MI) return grid_W == 4 && grid_H == 4 && (Cfg::NBUF == 1 ? C_IN <= u32(Cfg::CI) : true);
    return grid_W == u32(Cfg::W) && grid_H % Cfg::ROWS == 0 && (Cfg::NBUF == 1 ? C_IN <= u32(Cfg::CI) : true);
}

// Kernel arguments and grid size of one configuration for one call.
template <class Cfg>
inline uint64_t direct_args(DirectArgs &a, const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT,
                            u32 grid_H, u32 in_H, u32 relu) {
    a.Wt = Wt, a.X = X, a.Y = Y, a.bias = bias;
    a.C_IN = C_IN, a.C_OUT = C_OUT, a.grid_H = grid_H, a.in_H = in_H;
    a.tiles_per_img = Cfg::MI ? 1 : grid_H / Cfg::ROWS;
    a.oc_tiles = ceil_div(C_OUT, u32(Cfg::OCT));
    a.tiles_total = Cfg::MI ? ceil_div(N, u32(Cfg::IMGS)) : N * a.tiles_per_img;
    a.n_images = N;
    a.relu = relu;
    a.xcd_shift = 0;
    return uint64_t(ceil_div(a.tiles_total, kXcds)) * kXcds * a.oc_tiles;  // padded to whole XCD rounds
}

template <class Cfg>
inline int launch_direct(const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT, u32 grid_H,
                         u32 in_H, u32 relu, hipStream_t s, const char *what) {
    DirectArgs a;
    const uint64_t wgs = direct_args<Cfg>(a, Wt, X, Y, bias, N, C_IN, C_OUT, grid_H, in_H, relu);
    if (wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL((conv3x3_kernel<Cfg>), dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    return check_launch(what);
}

}  // namespace crb
