// Direct 3x3 / stride 1 / pad 1 convolution for gfx950: forward and data gradient in one template.
//
// A workgroup (4 wave64) owns ROWS full image rows of one image and OCT output channels. The contraction
// runs over input channels in chunks of CI: for each chunk the raw input rows (with their one-pixel halo,
// zero outside the image) and the matching OCT x CI x 9 filter slice are staged in LDS, and every wave
// feeds v_mfma_f32_16x16x4_f32 directly from them. Inside a chunk the contraction index is ordered tap-major
// (k = tap*CI + channel), so MFMA step s covers one tap and four consecutive channels: the im2col gather is
// a per-lane base address (pixel + (lane/16) channel planes) plus a compile-time immediate per step, and the
// inner loop contains nothing but ds_read and MFMA. Fragments are read PF steps ahead of the MFMAs that
// consume them (explicit software pipeline; the scheduler is fenced so it cannot undo it).
//
// MFMA 16x16x4 f32 mapping (wave64, lane l): A value = A[i = l%16][k = l/16], B value = B[k = l/16][j = l%16],
// accumulator register r = D[i = 4*(l/16) + r][j = l%16]. Here i = pixel within a 16-pixel block,
// j = output channel within a 16-channel block, so a lane ends up with 4 consecutive pixels of one output
// channel: one 16-byte store per MFMA tile, and bias / ReLU are per-lane scalars.
//
// The data gradient of a stride-1 pad-1 3x3 convolution is the same computation on dY with the filter's
// channel roles swapped and its taps mirrored: DGRAD only changes how the filter slice is gathered into LDS
// and the sign of the tap offsets.
#pragma once
#include "igemm_engine.h"

namespace crb {

// NBUF_ = 2: double-buffered chunk pipeline (any C_IN). NBUF_ = 1: the whole contraction is one
// chunk (C_IN <= CI), half the LDS, so more workgroups fit on a CU and overlap each other's staging.
template <int W_, int ROWS_, int CI_, int OCT_, int PBW_, int OBW_, bool DGRAD_, int OCC_, int NBUF_ = 2>
struct DirectCfg {
    static constexpr int W = W_, ROWS = ROWS_, CI = CI_, OCT = OCT_, PBW = PBW_, OBW = OBW_, OCC = OCC_, NBUF = NBUF_;
    static constexpr bool DGRAD = DGRAD_;
    static constexpr int TP = ROWS * W;          // pixels per workgroup tile
    static constexpr int NPB = TP / 16;          // 16-pixel blocks
    static constexpr int NOB = OCT / 16;         // 16-channel blocks
    static constexpr int NPBW = NPB / PBW;       // wave groups along pixels
    static constexpr int NOBW = NOB / OBW;       // wave groups along channels
    static constexpr int XS = W + 8;             // LDS row stride: 3 pad, left halo, W interior (16-byte aligned), right halo, 3 pad
    static constexpr int XR = ROWS + 2;          // rows incl. halo
    // channel plane stride (floats): the four lane groups (lane/16) of a fragment read sit one plane apart;
    // 16 mod 32 (8 mod 32 for the 2-row blocks of W = 8) puts them on disjoint LDS banks. Multiple of 4.
    static constexpr int XP_MIN = XR * XS;
    static constexpr int XP_RES = W == 8 ? 8 : 16;
    static constexpr int XP = XP_MIN + ((XP_RES - XP_MIN % 32) + 32) % 32;
    static constexpr int KC = CI * 9;            // contraction length per chunk
    static constexpr int NSTEP = KC / 4;         // MFMA steps per chunk
    static constexpr int CQ = CI / 4;            // steps per tap
    static constexpr int PF = (8 / (PBW * OBW)) < 1 ? 1 : ((8 / (PBW * OBW)) > 4 ? 4 : (8 / (PBW * OBW)));  // read-ahead
    static constexpr int CIP = CI + 1;           // k index of (tap, channel) in a filter row is tap*CIP + channel: odd tap stride
    static constexpr int WSTR_MIN = 9 * CIP;     // filter row stride == 2 mod 4: the 32 lanes of a half-wave (16 rows x 2 k) hit distinct banks
    static constexpr int WSTR = WSTR_MIN + ((2 - WSTR_MIN % 4) + 4) % 4;
    static constexpr int X_SIZE = CI * XP;
    static constexpr int W_SIZE = OCT * WSTR;
    static_assert(W == 8 || W == 16 || W == 32, "image width");
    static_assert(TP % 16 == 0 && NPB % PBW == 0 && NOB % OBW == 0 && NPBW * NOBW == 4, "wave tiling must use 4 waves");
    static_assert((PBW * 16) % W == 0 || PBW == 1, "a wave's pixel blocks must start on a row boundary");
    static_assert(CI % 4 == 0, "chunk channel count");
};

struct DirectArgs {
    const float *Wt;    // filters, OC x IC x 3 x 3 of the forward convolution
    const float *X;     // input of this pass  (forward: X, dgrad: dY), N x C_IN x H x W
    float *Y;           // output of this pass (forward: Y, dgrad: dX), N x C_OUT x H x W
    const float *bias;  // per output channel or nullptr
    u32 C_IN, C_OUT, H;
    u32 tiles_per_img, oc_tiles, tiles_total;  // tiles_total = N * tiles_per_img
    u32 relu;
};

template <class Cfg>
__global__ void __launch_bounds__(kThreads, Cfg::OCC) conv3x3s1_kernel(DirectArgs a) {
    constexpr int W = Cfg::W, ROWS = Cfg::ROWS, CI = Cfg::CI, OCT = Cfg::OCT, PBW = Cfg::PBW, OBW = Cfg::OBW;
    constexpr int XS = Cfg::XS, XR = Cfg::XR, XP = Cfg::XP, NSTEP = Cfg::NSTEP, WSTR = Cfg::WSTR;
    constexpr int NBUF = Cfg::NBUF;
    __shared__ __attribute__((aligned(16))) float sX[NBUF][Cfg::X_SIZE];
    __shared__ __attribute__((aligned(16))) float sW[NBUF][Cfg::W_SIZE];

    const u32 t = threadIdx.x;
    // Workgroups are dealt round-robin to the 8 XCDs. Decode the id so that the oc_tiles workgroups that read the same
    // input rows get ids 8 apart: they land on the same XCD, back to back, and share those rows through its L2.
    const u32 xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
    const u32 oct = slot % a.oc_tiles;
    const u32 rest = (slot / a.oc_tiles) * kXcds + xcd;
    if (rest >= a.tiles_total) return;
    const u32 tile = rest % a.tiles_per_img;
    const u32 n = rest / a.tiles_per_img;
    const int r0 = int(tile) * ROWS;  // first output row of this tile
    const u32 oc0 = oct * OCT;
    const u32 HW = a.H * W;

    // ---- staging helpers ----------------------------------------------------------------------------
    // input rows: CI planes x XR rows x W/4 quads
    constexpr int XQ = CI * XR * (W / 4);
    constexpr int XNP = (XQ + kThreads - 1) / kThreads;
    // filter slice: one (filter row j, chunk channel c) pair per item, 9 contiguous taps each
    constexpr int WQ = OCT * CI;
    constexpr int WNP = (WQ + kThreads - 1) / kThreads;
    v4f xreg[XNP];
    float wreg[WNP * 9];

    auto fetch = [&](u32 c0) {
#pragma unroll
        for (int i = 0; i < XNP; ++i) {
            const u32 e = t + i * kThreads;
            v4f v = {0.f, 0.f, 0.f, 0.f};
            if (XQ % kThreads == 0 || e < XQ) {
                const u32 q = e % (W / 4), lr = (e / (W / 4)) % XR, c = e / ((W / 4) * XR);
                const int row = r0 - 1 + int(lr);
                if (row >= 0 && row < int(a.H) && c0 + c < a.C_IN)
                    v = *reinterpret_cast<const v4f *>(a.X + (size_t(n) * a.C_IN + c0 + c) * HW + u32(row) * W + 4 * q);
            }
            xreg[i] = v;
        }
#pragma unroll
        for (int i = 0; i < WNP; ++i) {
            const u32 e = t + i * kThreads;
            // forward: lanes run over chunk channels c (filter row j = e / CI): W[oc0 + j][c0 + c][0..8]
            // dgrad:   lanes run over filter rows j (gradient channel c = e / OCT): W[c0 + c][oc0 + j][0..8]
            const u32 j = Cfg::DGRAD ? e % OCT : e / CI, c = Cfg::DGRAD ? e / OCT : e % CI;
            const float *src = Cfg::DGRAD ? a.Wt + ((size_t(c0) + c) * a.C_OUT + oc0 + j) * 9
                                          : a.Wt + ((size_t(oc0) + j) * a.C_IN + c0 + c) * 9;
            // channels past the tensor's extent (ragged last chunk / last channel tile) are staged as zeros
            const bool ok = (WQ % kThreads == 0 || e < WQ) && c0 + c < a.C_IN && oc0 + j < a.C_OUT;
            if (ok) {  // one branch around the 9 contiguous loads keeps them mergeable into wide loads
#pragma unroll
                for (int tap = 0; tap < 9; ++tap) wreg[i * 9 + tap] = src[tap];
            } else {
#pragma unroll
                for (int tap = 0; tap < 9; ++tap) wreg[i * 9 + tap] = 0.f;
            }
        }
    };

    auto commit = [&](float *dX, float *dW) {
#pragma unroll
        for (int i = 0; i < XNP; ++i) {
            const u32 e = t + i * kThreads;
            if (XQ % kThreads == 0 || e < XQ) {
                const u32 q = e % (W / 4), lr = (e / (W / 4)) % XR, c = e / ((W / 4) * XR);
                *reinterpret_cast<v4f *>(dX + c * XP + lr * XS + 4 + 4 * q) = xreg[i];
            }
        }
#pragma unroll
        for (int i = 0; i < WNP; ++i) {
            const u32 e = t + i * kThreads;
            if (WQ % kThreads == 0 || e < WQ) {
                const u32 j = Cfg::DGRAD ? e % OCT : e / CI, c = Cfg::DGRAD ? e / OCT : e % CI;
#pragma unroll
                for (int tap = 0; tap < 9; ++tap) dW[j * WSTR + tap * Cfg::CIP + c] = wreg[i * 9 + tap];
            }
        }
    };

    // ---- zero the halo columns of both buffers once (never overwritten afterwards) ---------------------
    for (u32 e = t; e < u32(NBUF) * CI * XR; e += kThreads) {
        float *row = &sX[0][0] + (e / (CI * XR)) * Cfg::X_SIZE + ((e % (CI * XR)) / XR) * XP + (e % XR) * XS;
        row[3] = 0.f;
        row[W + 4] = 0.f;
    }

    // ---- per-lane fragment addressing ---------------------------------------------------------------------
    const int lane = t & 63, wave = t >> 6;
    const int wp = wave % Cfg::NPBW, wo = wave / Cfg::NPBW;
    const int li = lane & 15, kq = lane >> 4;
    // pixel of this lane in the wave's first block; lane group kq reads channel plane kq of each 4-channel step
    const int q0 = (wp * PBW) * 16 + li;
    const int xbase = kq * XP + (q0 / W) * XS + (q0 % W) + 3;
    const int wbase = (wo * OBW * 16 + li) * WSTR + kq;

    v4f acc[PBW][OBW];
#pragma unroll
    for (int p = 0; p < PBW; ++p)
#pragma unroll
        for (int o = 0; o < OBW; ++o) acc[p][o] = v4f{0.f, 0.f, 0.f, 0.f};

    constexpr int PF = Cfg::PF, CQ = Cfg::CQ;
    auto compute = [&](const float *cx, const float *cw) {
        const float *px = cx + xbase, *pw = cw + wbase;
        float av[PF + 1][PBW], bv[PF + 1][OBW];
        auto read_step = [&](int s, int slot) {
            const int tap = s / CQ, cq = s % CQ;
            const int fh = Cfg::DGRAD ? 2 - tap / 3 : tap / 3, fw = Cfg::DGRAD ? 2 - tap % 3 : tap % 3;
            const int xo = cq * 4 * XP + fh * XS + fw;
#pragma unroll
            for (int p = 0; p < PBW; ++p) av[slot][p] = px[xo + ((p * 16) / W) * XS + (p * 16) % W];
#pragma unroll
            for (int o = 0; o < OBW; ++o) bv[slot][o] = pw[o * 16 * WSTR + tap * Cfg::CIP + 4 * cq];
        };
#pragma unroll
        for (int s = 0; s < PF && s < NSTEP; ++s) read_step(s, s % (PF + 1));
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            if (s + PF < NSTEP) read_step(s + PF, (s + PF) % (PF + 1));
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int p = 0; p < PBW; ++p)
#pragma unroll
                for (int o = 0; o < OBW; ++o)
                    acc[p][o] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s % (PF + 1)][p], bv[s % (PF + 1)][o], acc[p][o], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };

    // ---- main loop over input-channel chunks (double-buffered) ---------------------------------------------
    fetch(0);
    commit(sX[0], sW[0]);
    __syncthreads();
    if constexpr (NBUF == 1) {
        compute(sX[0], sW[0]);
    } else {
        const u32 nchunk = (a.C_IN + CI - 1) / CI;
        for (u32 ch = 0; ch < nchunk; ++ch) {
            const bool more = ch + 1 < nchunk;
            if (more) fetch((ch + 1) * CI);
            if (ch & 1) {
                compute(sX[NBUF - 1], sW[NBUF - 1]);
                if (more) commit(sX[0], sW[0]);
            } else {
                compute(sX[0], sW[0]);
                if (more) commit(sX[NBUF - 1], sW[NBUF - 1]);
            }
            __syncthreads();
        }
    }

    // ---- epilogue: lane holds 4 consecutive pixels of one output channel per tile ---------------------------
#pragma unroll
    for (int o = 0; o < OBW; ++o) {
        const u32 oc = oc0 + (wo * OBW + o) * 16 + li;
        if (oc >= a.C_OUT) continue;
        const float b = a.bias ? a.bias[oc] : 0.f;
#pragma unroll
        for (int p = 0; p < PBW; ++p) {
            const int q = (wp * PBW + p) * 16 + 4 * kq;
            v4f v = acc[p][o];
            v.x += b, v.y += b, v.z += b, v.w += b;
            if (a.relu) {
                v.x = v.x > 0.f ? v.x : 0.f, v.y = v.y > 0.f ? v.y : 0.f;
                v.z = v.z > 0.f ? v.z : 0.f, v.w = v.w > 0.f ? v.w : 0.f;
            }
            *reinterpret_cast<v4f *>(a.Y + (size_t(n) * a.C_OUT + oc) * HW + u32(r0 + q / W) * W + (q % W)) = v;
        }
    }
}

template <class Cfg>
inline int launch_direct(const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT, u32 H,
                         u32 relu, hipStream_t s, const char *what) {
    DirectArgs a;
    a.Wt = Wt, a.X = X, a.Y = Y, a.bias = bias;
    a.C_IN = C_IN, a.C_OUT = C_OUT, a.H = H;
    a.tiles_per_img = H / Cfg::ROWS;
    a.oc_tiles = ceil_div(C_OUT, u32(Cfg::OCT));
    a.relu = relu;
    a.tiles_total = N * a.tiles_per_img;
    const uint64_t wgs = uint64_t(ceil_div(a.tiles_total, kXcds)) * kXcds * a.oc_tiles;  // padded to whole XCD rounds
    if (wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL((conv3x3s1_kernel<Cfg>), dim3(u32(wgs)), dim3(kThreads), 0, s, a);
    return check_launch(what);
}

// Shape gate of one configuration. Channel counts need not divide CI / OCT: ragged chunks and tiles are zero-filled.
template <class Cfg>
inline bool direct_fits(u32 C_IN, u32 C_OUT, u32 H, u32 Wd) {
    (void)C_OUT;
    return Wd == u32(Cfg::W) && H % Cfg::ROWS == 0 && (Cfg::NBUF == 1 ? C_IN <= u32(Cfg::CI) : true);
}

}  // namespace crb
