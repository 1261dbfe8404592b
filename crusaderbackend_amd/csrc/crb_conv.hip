// C-ABI entry points of the convolution family: forward, data gradient, weight gradient and the
// standalone bias add, all as implicit GEMMs on the MFMA engine (no im2col buffer is materialised).
#include "conv3x3_direct.h"
#include "conv3x3_tiled.h"
#include "conv3x3_tiled_wgrad.h"
#include "conv3x3_wgrad.h"
#include "conv3x3_wgrad_image.h"
#include "conv1x1_s2.h"
#include "conv1x1_wgrad.h"
#include "conv1x1_stream.h"
#include "gemm_internal.h"
#include "operands.h"

#include <mutex>

namespace crb {

// Macro-tiles chosen by the channel extent on the GEMM-M side; the pixel (or tap) side is 128 wide.
typedef TileCfg<32, 128, 16, 1, 4, 2> CfgM32;
typedef TileCfg<64, 128, 16, 2, 2, 2> CfgM64;
typedef TileCfg<128, 128, 16, 2, 2, 2> CfgM128;

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

static int check_geom(const char *what, const crb_conv_geom *g) {
    if (!g) return fail(CRB_ENULL, "%s: null geometry", what);
    if (!g->N || !g->IC || !g->IH || !g->IW || !g->OC || !g->FH || !g->FW || !g->OH || !g->OW || !g->sH || !g->sW)
        return fail(CRB_EINVAL_SHAPE, "%s: zero dimension or stride", what);
    // the relations the reference's assertConv enforces (cuConv.cu:731-755)
    if (g->IH + 2 * g->pH < g->FH || g->OH != (g->IH + 2 * g->pH - g->FH) / g->sH + 1)
        return fail(CRB_EINVAL_SHAPE, "%s: assertConv: rows (h) relationship did not satisfy", what);
    if (g->IW + 2 * g->pW < g->FW || g->OW != (g->IW + 2 * g->pW - g->FW) / g->sW + 1)
        return fail(CRB_EINVAL_SHAPE, "%s: assertConv: cols (w) relationship did not satisfy", what);
    const uint64_t lim = 0x7fffffffull;
    if (uint64_t(g->N) * g->IC * g->IH * g->IW > lim || uint64_t(g->N) * g->OC * g->OH * g->OW > lim ||
        uint64_t(g->OC) * g->IC * g->FH * g->FW > lim)
        return fail(CRB_EINVAL_SHAPE, "%s: tensor exceeds 2^31 elements", what);
    return CRB_OK;
}

static Im2col make_im2col(const float *X, const crb_conv_geom *g) {
    Im2col m;
    m.X = X;
    m.npix = g->N * g->OH * g->OW;
    m.ntap = g->IC * g->FH * g->FW;
    m.IH = g->IH, m.IW = g->IW;
    m.img_stride = g->IC * g->IH * g->IW;
    m.chan_stride = g->IH * g->IW;
    m.sH = g->sH, m.sW = g->sW, m.pH = g->pH, m.pW = g->pW;
    m.ohw.init(g->OH * g->OW), m.ow.init(g->OW), m.fhw.init(g->FH * g->FW), m.fw.init(g->FW);
    return m;
}

template <class Cfg, class AOp, class BOp, class Epi>
static int launch_cfg(const AOp &a, const BOp &b, const Epi &e, u32 M, u32 N, u32 K, u32 zdim, u32 split_k, u32 k_per_z,
                      hipStream_t s, const char *what) {
    return launch_igemm<Cfg>(a, b, e, M, N, K, zdim, split_k, k_per_z, s, what);
}

template <class AOp, class BOp, class Epi>
static int run_by_m(const AOp &a, const BOp &b, const Epi &e, u32 M, u32 N, u32 K, u32 zdim, u32 split_k, u32 k_per_z,
                    hipStream_t s, const char *what) {
    if (M <= 32) return launch_cfg<CfgM32>(a, b, e, M, N, K, zdim, split_k, k_per_z, s, what);
    if (M <= 64) return launch_cfg<CfgM64>(a, b, e, M, N, K, zdim, split_k, k_per_z, s, what);
    return launch_cfg<CfgM128>(a, b, e, M, N, K, zdim, split_k, k_per_z, s, what);
}

// Forward / data gradient through the engine with an NCHW result. When the tile grid is too small to occupy the chip
// the contraction is cut into slices: partial NCHW results go to scratch, a second kernel sums them in fixed order and
// applies bias / ReLU.
template <class AOp, class BOp>
static int run_nchw(const AOp &a, const BOp &b, NchwEpi e, u32 M, u32 N, u32 K, hipStream_t s, const char *what) {
    const u32 bm = M <= 32 ? 32 : (M <= 64 ? 64 : 128);
    const SplitPlan sp = plan_split(M, N, K, bm, 128, 16, 1);
    if (sp.splits == 1) return run_by_m(a, b, e, M, N, K, 1, 0, K, s, what);
    const u32 count = M * N;  // N = batch * H * W, so M*N is the whole NCHW tensor
    const size_t need = size_t(sp.splits) * count * sizeof(float);
    float *ws = nullptr;
    if (int st = scratch_get(need, s, what, &ws)) return st;
    NchwEpi pe = e;
    pe.T = ws, pe.row_bias = nullptr, pe.flags = 0u, pe.zstride = count;
    if (int st = run_by_m(a, b, pe, M, N, K, sp.splits, 1, sp.k_per_z, s, what)) return st;
    return launch_splitk_reduce(ws, e.T, count, sp.splits, ReduceEpi{e.row_bias, e.HW, e.C, e.flags}, s, what);
}

// Data gradient at stride > 1 through the engine, one residue class of input pixels per launch (operands.h: ClassTaps,
// ClassGather, NchwClassEpi). Classes no tap reaches (filters smaller than the stride) are zero-filled.
static int dgrad_by_classes(const float *W, const float *dY, float *dX, const crb_conv_geom *g, hipStream_t s) {
    const char *what = "crb_conv_dgrad";
    const u32 FHW = g->FH * g->FW;
    bool empty_class = false;
    for (u32 py = 0; py < g->sH && py < g->IH; ++py)
        for (u32 px = 0; px < g->sW && px < g->IW; ++px)
            if ((py + g->pH) % g->sH >= g->FH || (px + g->pW) % g->sW >= g->FW) empty_class = true;
    if (empty_class) {
        const uint64_t count = uint64_t(g->N) * g->IC * g->IH * g->IW;
        if (int st = crb_tensor_fill(dX, 0.f, uint32_t(count), s)) return st;
    }
    for (u32 py = 0; py < g->sH && py < g->IH; ++py)
        for (u32 px = 0; px < g->sW && px < g->IW; ++px) {
            const u32 fh0 = (py + g->pH) % g->sH, fw0 = (px + g->pW) % g->sW;
            if (fh0 >= g->FH || fw0 >= g->FW) continue;
            const u32 nfh = ceil_div(g->FH - fh0, g->sH), nfw = ceil_div(g->FW - fw0, g->sW);
            const u32 CH = ceil_div(g->IH - py, g->sH), CW = ceil_div(g->IW - px, g->sW);  // the class's pixel grid
            const u32 M = g->IC, N = g->N * CH * CW, K = g->OC * nfh * nfw;
            ClassTaps a{W, g->IC, FHW, g->IC * FHW, fh0 * g->FW + fw0, g->sH * g->FW, g->sW, FastDiv(nfh * nfw), FastDiv(nfw)};
            ClassGather b;
            b.dY = dY, b.npix = N;
            b.OH = g->OH, b.OW = g->OW, b.img_stride = g->OC * g->OH * g->OW, b.chan_stride = g->OH * g->OW;
            b.qh = int((py + g->pH) / g->sH), b.qw = int((px + g->pW) / g->sW);
            b.chw.init(CH * CW), b.cw.init(CW), b.ntap.init(nfh * nfw), b.nfw.init(nfw);
            NchwClassEpi e;
            e.T = dX, e.C = g->IC, e.HW = g->IH * g->IW, e.W = g->IW;
            e.sH = g->sH, e.sW = g->sW, e.py = py, e.px = px;
            e.chw.init(CH * CW), e.cw.init(CW);
            if (int st = run_by_m(a, b, e, M, N, K, 1, 0, K, s, what)) return st;
        }
    return CRB_OK;
}

// The class launches do not cut the contraction, so a class must bring enough tiles of its own: with fewer the one gather
// over all taps, cut over K, is faster in spite of the zeros it multiplies (64 -> 64 @16x16 7x7 stride 2 batch 4, 8 tiles a
// class: 360 against 29 us; 256 -> 32 @28 7x7 stride 2 batch 32, 98 tiles: 261 against 411).
static bool dgrad_classes_pay(const crb_conv_geom *g) {
    const u32 CH = ceil_div(g->IH, g->sH), CW = ceil_div(g->IW, g->sW);
    const u32 bm = g->IC <= 32 ? 32 : (g->IC <= 64 ? 64 : 128);
    const uint64_t tiles = uint64_t(ceil_div(g->IC, bm)) * ceil_div(g->N * CH * CW, 128u);
    if (tiles < 48) return false;
    // Each class writes every sW-th float of a row, and there are sH * sW launches: beyond stride 2 that only pays under a
    // long contraction (256 -> 16 @32 4x4 stride 3 batch 32, K = 256: 107 against 77 us; 16 -> 32 @64 4x4 stride 3, K = 512: 73 against 142).
    return (g->sH <= 2 && g->sW <= 2) || g->OC * g->FH * g->FW >= 512;
}

// Scratch bytes run_nchw asks for (0: the contraction is not cut).
static size_t nchw_scratch_bytes(u32 M, u32 N, u32 K) {
    const u32 bm = M <= 32 ? 32 : (M <= 64 ? 64 : 128);
    const SplitPlan sp = plan_split(M, N, K, bm, 128, 16, 1);
    return sp.splits > 1 ? size_t(sp.splits) * M * N * sizeof(float) : 0;
}

static u32 tile_m_for(u32 M) { return M <= 32 ? 32 : (M <= 64 ? 64 : 128); }

// Split plan of the weight gradient: the contraction runs over n*OH*OW (up to 131072) while the result
// is only OC x IC*FH*FW, so the K range is cut into `splits` slices handled by separate workgroups.
struct WgradPlan {
    u32 M, Ncols, K, splits, k_per_z;
};
static WgradPlan wgrad_plan(const crb_conv_geom *g) {
    WgradPlan p;
    p.M = g->OC;
    p.Ncols = g->IC * g->FH * g->FW;
    p.K = g->N * g->OH * g->OW;
    const u32 tiles = ceil_div(p.M, tile_m_for(p.M)) * ceil_div(p.Ncols, 128);
    const u32 target_wgs = 1024;  // ~4 workgroups per CU
    u32 splits = tiles >= target_wgs ? 1 : target_wgs / tiles;
    const u32 min_k = 256;  // do not cut slices thinner than 16 slabs
    if (splits > ceil_div(p.K, min_k)) splits = ceil_div(p.K, min_k);
    if (splits < 1) splits = 1;
    u32 kz = ceil_div(ceil_div(p.K, splits), 16) * 16;
    p.k_per_z = kz;
    p.splits = ceil_div(p.K, kz);
    return p;
}

// ---- direct 3x3 / pad 1 path (stride 1 and 2) ----------------------------------------------------------------
// Configurations <W, ROWS, CI, OCT, PBW, OBW, DGRAD, OCC, NBUF, S>, picked by grid width and channel counts.
// Tried in order; the first whose constraints hold is used, otherwise the implicit-GEMM engine runs.
// (gH, gW) is the pixel grid: the output image, or dY for the stride-2 data gradient; in_H the rows of the staged tensor.
// Shape rules shared by try_direct and bwd_fused (which must chunk the contraction exactly as the separate data-gradient
// call does, so that both produce the same bits). C_IN / C_OUT: channels the pass reads / writes; gH: rows of its pixel grid.
static bool one_chunk_w16(u32 N, u32 C_IN, u32 C_OUT, u32 gH) {  // stride 1, width 16: all 17..32 input channels LDS-resident
    return C_IN > 16 && C_IN <= 32 && N * (gH / 8) * ceil_div(C_OUT, 16u) >= 512;
}
static bool one_chunk_w8(u32 N, u32 C_IN, u32 C_OUT, u32 gH) {  // stride 1, width 8: all 33..64 input channels LDS-resident
    return C_IN > 32 && C_IN <= 64 && C_OUT <= 64 && N * (gH / 8) * ceil_div(C_OUT, 16u) >= 512;
}
static bool s2_dgrad_w16_c16(u32 N, u32 C_IN, u32 C_OUT, u32 gH) { return C_IN > 8 && C_OUT <= 16 && N * (gH / 4) >= 512; }
static bool s2_dgrad_w8_c16(u32 N, u32 C_IN, u32 C_OUT) { return C_IN > 8 && N * ceil_div(C_OUT, 16u) >= 256; }

template <bool DG, int S>
static int try_direct(const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT, u32 gH,
                      u32 gW, u32 in_H, u32 relu, hipStream_t s, const char *what, bool &done, bool probe = false) {
    done = true;
    // probe: only report (through `done`) whether a configuration takes the shape, launch nothing
#define CRB_TRY(...)                                                                                          \
    if (direct_fits<DirectCfg<__VA_ARGS__>>(C_IN, gH, gW))                                                     \
        return probe ? int(CRB_OK) : launch_direct<DirectCfg<__VA_ARGS__>>(Wt, X, Y, bias, N, C_IN, C_OUT, gH, in_H, relu, s, what);
    // output-channel tile: the smallest of 16 / 32 / 64 that covers C_OUT, 64 beyond; chunks of 16 input channels at
    // stride 1 when C_IN > 8, chunks of 8 otherwise (stride 2 stages wider / more rows per chunk)
    if constexpr (S == 1) {
        if (gW == 32) {
            // forward: the contraction in two halves, the second half's rows still arriving while the first is multiplied
            // (16 -> 16, batch 128, operands not cached: 8.6 -> 8.1 us; cached 8.0 -> 7.95 us). The data gradient keeps the
            // one-pass form it shares with the one-launch backward kernel.
            if constexpr (!DG) {
                if (C_IN <= 16 && C_IN > 8 && C_OUT <= 16) { CRB_TRY(32, 8, 16, 16, 4, 1, DG, 2, 1, 1, 3, 4, 2) }
            }
            if (C_IN <= 16 && C_IN > 8 && C_OUT <= 16) { CRB_TRY(32, 8, 16, 16, 4, 1, DG, 2, 1, 1, 3, 4) }  // one LDS-resident chunk
            // 9..12 channels in, 33..48 out (the data gradient of a growth-12 dense layer): one 12-channel chunk, stores in two
            // pixel groups (12 -> 48, batch 64: 13.0 -> 9.7 us)
            if (C_IN > 8 && C_IN <= 12 && C_OUT > 32 && C_OUT <= 48) { CRB_TRY(32, 4, 12, 48, 2, 3, DG, 2, 1, 1, 3, 2) }
            // too few 8-row tiles for two workgroups per CU: 4-row tiles
            if (C_OUT <= 16 && C_IN > 16 && N * (gH / 8) < 512) { CRB_TRY(32, 4, 16, 16, 2, 1, DG, 2, 2, 1) }
            // 33..48 output channels: a 48-wide tile instead of a quarter-empty 64-wide one
            // image layers (3 input channels): one 4-channel chunk instead of an 8-channel one that is 5/8 zeros
            // (3 -> 64, batch 128: 21.0 -> 13.4 us; 3 -> 16: 6.8 -> 4.6 us)
            if (C_IN <= 4 && C_OUT > 32) { CRB_TRY(32, 8, 4, 64, 4, 4, DG, 2, 1, 1, 3, 4) }
            if (C_IN <= 4 && C_OUT > 16) { CRB_TRY(32, 8, 4, 32, 4, 2, DG, 2, 1, 1, 3, 4) }
            if (C_IN <= 4) { CRB_TRY(32, 8, 4, 16, 4, 1, DG, 2, 1, 1, 3, 4) }
            if (C_OUT > 32 && C_OUT <= 48 && N * (gH / 8) < 512) { CRB_TRY(32, 4, 8, 48, 2, 3, DG, 2, 2, 1) }
            if (C_OUT > 32 && C_OUT <= 48) { CRB_TRY(32, 8, 8, 48, 4, 3, DG, 2, 2, 1) }
            if (C_OUT > 32) { CRB_TRY(32, 8, 8, 64, 4, 4, DG, 2, 2, 1) }
            if (C_OUT > 16) { CRB_TRY(32, 8, 8, 32, 4, 2, DG, 2, 2, 1) }
            CRB_TRY(32, 8, 8, 16, 4, 1, DG, 2, 2, 1)
            CRB_TRY(32, 4, 8, 16, 2, 1, DG, 2, 2, 1)
        } else if (gW == 16) {
            // 17..32 input channels and enough tiles for two workgroups per CU: the whole contraction as one LDS-resident
            // chunk, stores in two pixel groups (32 -> 32, batch 128: 9.2 -> 8.3 us forward, 9.0 -> 8.3 us data gradient)
            // growth-12 dense layers, 48 -> 12 and back: the whole contraction as one LDS-resident chunk
            // (batch 64: forward 7.8 -> 6.8 us, data gradient 5.9 -> 4.65 us)
            if (!DG && C_IN > 32 && C_IN <= 48 && C_OUT <= 16) { CRB_TRY(16, 8, 48, 16, 2, 1, DG, 2, 1, 1, 3, 2) }
            if (C_IN > 8 && C_IN <= 12 && C_OUT > 32 && C_OUT <= 48) { CRB_TRY(16, 4, 12, 48, 1, 3, DG, 2, 1, 1) }
            if (one_chunk_w16(N, C_IN, C_OUT, gH)) { CRB_TRY(16, 8, 32, 16, 2, 1, DG, 2, 1, 1, 3, 2) }
            if (C_OUT > 64) { CRB_TRY(16, 8, 8, 64, 2, 4, DG, 2, 2, 1) }
            if (C_OUT > 16 && C_IN > 8) { CRB_TRY(16, 4, 16, 32, 1, 2, DG, 2, 2, 1) }
            if (C_OUT > 16) { CRB_TRY(16, 4, 8, 32, 1, 2, DG, 2, 2, 1) }
            CRB_TRY(16, 8, 8, 16, 2, 1, DG, 2, 2, 1)
            CRB_TRY(16, 4, 8, 16, 1, 1, DG, 2, 2, 1)
        } else if (gW == 8) {
            // 33..64 input channels, at most 64 output channels: one LDS-resident chunk (64 -> 64, batch 128: 9.0 -> 8.65 us).
            // Forward only: the data gradient keeps the chunking of the one-launch backward kernel, which has no room in
            // LDS for a resident 64-channel chunk next to the weight-gradient workgroup and is slower with 16-wide tiles.
            if (!DG && one_chunk_w8(N, C_IN, C_OUT, gH)) { CRB_TRY(8, 8, 64, 16, 1, 1, DG, 2, 1, 1) }
            if (!DG && C_IN > 32 && C_IN <= 48 && C_OUT <= 16) { CRB_TRY(8, 8, 48, 16, 1, 1, DG, 2, 1, 1) }  // (batch 64: 5.0 -> 4.6 us)
            // 64 output channels with chunks of 8: chunks of 16 would need more LDS than lets two workgroups share a CU, and a
            // SIMD with a single wave issues its MFMAs a third slower
            if (C_OUT > 128 && C_IN > 8) { CRB_TRY(8, 8, 8, 64, 1, 4, DG, 2, 2, 1) }
            if (C_OUT > 64 && C_IN > 8) { CRB_TRY(8, 8, 16, 32, 1, 2, DG, 2, 2, 1) }
            if (C_IN > 8) { CRB_TRY(8, 8, 16, 16, 1, 1, DG, 2, 2, 1) }
            CRB_TRY(8, 8, 8, 16, 1, 1, DG, 2, 2, 1)
            CRB_TRY(8, 4, 8, 32, 1, 1, DG, 2, 2, 1)
        } else if (gW == 4) {  // 4x4 images, four stacked per tile
            // at most 32 output channels per workgroup: 64 need 95-115 KB of LDS, one workgroup per CU and so one wave per
            // SIMD (512 -> 512 at batch 128: forward 105.9 -> 96.9 us, data gradient 100.5 -> 91.3 us with 32)
            if (C_OUT > 16 && C_IN > 8) { CRB_TRY(4, 16, 16, 32, 1, 2, DG, 2, 2, 1) }
            if (C_IN > 8) { CRB_TRY(4, 16, 16, 16, 1, 1, DG, 2, 2, 1) }
            CRB_TRY(4, 16, 8, 16, 1, 1, DG, 2, 2, 1)
        }
    } else {
        if (gW == 32) {
            // forward only: the data gradient holds four parity classes per MFMA tile, and 32 of them do not fit the registers
            if constexpr (!DG) {
                if (C_OUT > 16) { CRB_TRY(32, 8, 8, 32, 4, 2, false, 2, 2, 2) }
            }
            CRB_TRY(32, 8, 8, 16, 4, 1, DG, 2, 2, 2)
            CRB_TRY(32, 4, 8, 16, 2, 1, DG, 2, 2, 2)
        } else if (gW == 16) {
            // measured on the residual-network transitions at batch 128 (16 -> 32: forward 7.2 -> 6.2 us, data gradient 8.5 -> 7.2 us)
            if (!DG && C_IN > 8 && C_IN <= 16 && C_OUT > 16 && N * (gH / 4) >= 512) { CRB_TRY(16, 4, 16, 32, 1, 2, DG, 2, 1, 2) }
            if (DG && s2_dgrad_w16_c16(N, C_IN, C_OUT, gH)) { CRB_TRY(16, 4, 16, 16, 1, 1, DG, 2, 2, 2) }
            if (C_OUT > 16) { CRB_TRY(16, 8, 8, 32, 2, 2, DG, 2, 2, 2) }
            CRB_TRY(16, 8, 8, 16, 2, 1, DG, 2, 2, 2)
            CRB_TRY(16, 4, 8, 16, 1, 1, DG, 2, 2, 2)
        } else if (gW == 8) {
            // (32 -> 64: forward 7.2 -> 6.65 us, data gradient 10.9 -> 7.1 us: 16-channel tiles give every CU a workgroup)
            if (!DG && C_IN > 8 && C_OUT > 16 && N * (gH / 4) >= 256) { CRB_TRY(8, 4, 16, 32, 1, 1, DG, 2, 2, 2) }
            if (DG && s2_dgrad_w8_c16(N, C_IN, C_OUT)) { CRB_TRY(8, 8, 16, 16, 1, 1, DG, 2, 2, 2) }
            if (C_OUT > 16) { CRB_TRY(8, 8, 8, 32, 1, 2, DG, 2, 2, 2) }
            CRB_TRY(8, 8, 8, 16, 1, 1, DG, 2, 2, 2)
            CRB_TRY(8, 4, 8, 32, 1, 1, DG, 2, 2, 2)
        }
    }
#undef CRB_TRY
    done = false;
    return CRB_OK;
}

// 3x3 / pad 1 / stride 1 on images of any extent (conv3x3_tiled.h), <TH, TW, OCT, WP, CI, DGRAD, OCC>: 128-pixel tiles of the
// shape that pads the image least, 32 output channels per workgroup (measured at batch 32-128 on 56 / 28 / 14 / 48 / 24 / 12
// wide images with 32-256 channels: within 3 % of the best of eighteen tile shapes everywhere; 256-pixel and 64- or
// 128-channel tiles and chunks of 16 channels were 5-80 % slower), 8 x 8 tiles with 64 channels for images up to 8 x 8.
// Against the implicit-GEMM engine, forward / data gradient: 64->64 @56x56 batch 32 157 / 168 -> 93 / 99 us,
// 128->128 @28 146 / 184 -> 93 / 99, 256->256 @14 124 / 143 -> 96 / 97, 512->512 @7 141 / 162 -> 118 / 141,
// 64->64 @24 batch 64 84 / 99 -> 40 / 40, 32->32 @48 72 / 80 -> 37 / 37.
// Whether the tiled kernel is the better choice for a 3x3 (or 5x5) pass that reads C_IN channels and writes C_OUT on an
// H x W pixel grid: not with fewer than 5 contraction channels (a chunk of 8 would be mostly zeros: 3 -> 64 @224 batch 8
// 82 us against the engine's 43), and not when the grid is a handful of workgroups under a long contraction, which the
// engine cuts over K (256 -> 256 @14 batch 4: 62 against 31 us). Checked on 35 random shapes (3-256 channels, 7-224 wide, batch 1-64)
// against the engine: forward -58 ... +2 %, data gradient -72 ... +8 %.
static bool tiled_pays(u32 N, u32 C_IN, u32 C_OUT, u32 H, u32 W, u32 taps) {
    if (C_IN < 5) return false;
    // a contraction under 64 long into more than 16 output channels on 8192 pixels or more: the engine's 32-row tiles are full,
    // its flat pixel list wastes nothing and fills the chip (6 -> 128 @10x10 batch 128: 16.6 against 14.1 us, 6 -> 64 @30x30
    // batch 64: 18.8 against 15.9; but 6 -> 256 @64x64 batch 1: 8.0 against 13.5)
    if (C_IN * taps < 64 && C_OUT > 16 && uint64_t(N) * H * W >= 8192) return false;
    // a contraction from 2304 on a grid the tiles fill less than 60 % (256 -> 256 @18x18 batch 16, 51 % full: 132 against 105 us;
    // shorter contractions still gain at that fill: 64 -> 256 @18x18 batch 16 40 against 46, 128 -> 256 @12x12 batch 32 52 against 60)
    if (C_IN * taps >= 2304) {
        auto padded = [&](u32 th, u32 tw) { return uint64_t(ceil_div(H, th)) * th * ceil_div(W, tw) * tw; };
        const uint64_t best = (H <= 8 && W <= 8) ? 64 : std::min(padded(8, 16), std::min(padded(16, 8), padded(4, 32)));
        if (5 * uint64_t(H) * W < 3 * best) return false;
    }
    const uint64_t wgs = uint64_t(N) * ceil_div(H, 8u) * ceil_div(W, 16u) * ceil_div(C_OUT, 32u);
    // short contractions from a few dozen workgroups on (96 -> 24 @7x7 batch 4, four workgroups: 25 against 16 us); long ones
    // need two workgroups per CU (256 -> 256 @28 stride 2 batch 16, 256 workgroups: 82 against 69 us; batch 32 -> 512 channels,
    // 1024 workgroups: 237 against 292)
    // (with at most 16 output channels the engine's 32-row tile is mostly empty: 128 -> 3 @20 batch 64, 384 workgroups, 50 against 90 us)
    return C_IN * taps < 1152 ? wgs >= 48 : (wgs >= 512 || (wgs >= 192 && C_OUT <= 16));
}

// S = 2 (forward only): H, W are the output's extent, IH, IW the input's. F = 5: 5x5 / pad 2 / stride 1 (16 -> 32 @28x28 batch 64:
// forward 48 -> 21 us, data gradient 111 -> 39 us against the engine).
template <bool DG, int S = 1, int F = 3>
static int launch_tiled_any(const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT, u32 H, u32 W, u32 relu,
                            hipStream_t s, const char *what, u32 IH = 0, u32 IW = 0, int pad = -1) {
#define CRB_TILED(TH, TW, OCT, WP) \
    return launch_tiled<TiledCfg<TH, TW, OCT, WP, 8, DG, 2, S, F>>(Wt, X, Y, bias, N, C_IN, C_OUT, H, W, relu, s, what, IH, IW, pad)
    if (H <= 8 && W <= 8) CRB_TILED(8, 8, 64, 2);
    auto padded = [&](u32 th, u32 tw) { return uint64_t(ceil_div(H, th)) * th * ceil_div(W, tw) * tw; };
    const uint64_t p816 = padded(8, 16), p168 = padded(16, 8), p432 = padded(4, 32);
    if (p816 <= p168 && p816 <= p432) CRB_TILED(8, 16, 32, 4);
    if (p168 <= p432) CRB_TILED(16, 8, 32, 4);
    CRB_TILED(4, 32, 32, 4);
#undef CRB_TILED
}

// Direct kernel configurations for 1x1 / stride 1 / no padding layers <W, ROWS, CI, OCT, PBW, OBW, DGRAD, OCC, NBUF, S, FS=1>.
// The output-channel tile is the widest of 64 / 48 / 32 / 16 that wastes at most a quarter of its channels and still
// yields enough workgroups for the chip; if none does, the batched GEMM forms run instead.
template <bool DG>
static int try_pointwise(const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 C_IN, u32 C_OUT, u32 gH, u32 gW,
                         u32 relu, hipStream_t s, const char *what, bool &done, bool probe = false) {
    done = true;
    // large layers whose short side (forward: the output channels; data gradient: the contraction) fits one wave: the
    // activations go from global memory straight into the MFMAs (204 -> 48 @ 32x32, batch 64: forward 20.2 -> 17.0 us,
    // data gradient 23.0 -> 17.6 us)
    if (pw_stream_fits(N, DG ? C_IN : C_OUT, gH * gW))
        return probe ? int(CRB_OK) : launch_pw_stream(DG, Wt, X, Y, bias, N, DG ? C_OUT : C_IN, DG ? C_IN : C_OUT, gH * gW, relu, s, what);
    if ((gW != 32 && gW != 16 && gW != 8) || gH % 8 != 0) {  // every configuration below tiles rows by 8 or 4
        done = false;
        return CRB_OK;
    }
    const u32 tiles = N * (gH / 8);
    auto good = [&](u32 oct) {
        const u32 nt = ceil_div(C_OUT, oct);
        return nt * oct * 3 <= C_OUT * 4 + 3 * 15 && tiles * nt >= 192;  // <= 25 % padding (one ragged 16-block allowed)
    };
#define CRB_TRY(...)                                                                                          \
    if (direct_fits<DirectCfg<__VA_ARGS__>>(C_IN, gH, gW))                                                     \
        return probe ? int(CRB_OK) : launch_direct<DirectCfg<__VA_ARGS__>>(Wt, X, Y, bias, N, C_IN, C_OUT, gH, gH, relu, s, what);
    // long contractions with few workgroups: half-height tiles, so two workgroups share a CU and one multiplies while
    // the other waits for its next channel chunk
    const bool half = C_IN > 64 && tiles * ceil_div(C_OUT, 48u) < 512;
    auto good_half = [&](u32 oct) {  // the same test for half-height tiles (twice as many of them)
        const u32 nt = ceil_div(C_OUT, oct);
        return nt * oct * 3 <= C_OUT * 4 + 3 * 15 && 2 * tiles * nt >= 192;
    };
    // a contraction of at most 48 channels (the data gradient of a bottleneck layer): one LDS-resident chunk, stores in
    // pixel groups (48 -> 204 at batch 64: 28.1 -> 25.6 us @32x32, 9.7 -> 8.9 us @16x16, 5.1 -> 4.5 us @8x8)
    const bool resident = DG && C_IN > 16 && C_IN <= 48;
    if (resident && gW == 32) {
        if (good(64)) { CRB_TRY(32, 8, 48, 64, 4, 4, DG, 2, 1, 1, 1, 4) }
        if (good(48)) { CRB_TRY(32, 8, 48, 48, 4, 3, DG, 2, 1, 1, 1, 4) }
    } else if (resident && gW == 16) {
        if (good(64)) { CRB_TRY(16, 8, 48, 64, 2, 4, DG, 2, 1, 1, 1, 2) }
        if (good(48)) { CRB_TRY(16, 8, 48, 48, 2, 3, DG, 2, 1, 1, 1, 2) }
    } else if (resident) {
        if (good(64)) { CRB_TRY(8, 8, 48, 64, 1, 4, DG, 2, 1, 1, 1) }
        if (good(48)) { CRB_TRY(8, 8, 48, 48, 1, 3, DG, 2, 1, 1, 1) }
    }
    if (gW == 32) {
        if (half && good(48)) { CRB_TRY(32, 4, 16, 48, 2, 3, DG, 2, 2, 1, 1) }
        if (half && good(64)) { CRB_TRY(32, 4, 16, 64, 2, 4, DG, 2, 2, 1, 1) }
        if (good(64)) { CRB_TRY(32, 8, 16, 64, 4, 4, DG, 2, 2, 1, 1) }
        if (good(48)) { CRB_TRY(32, 8, 16, 48, 4, 3, DG, 2, 2, 1, 1) }
        if (good(32)) { CRB_TRY(32, 8, 16, 32, 4, 2, DG, 2, 2, 1, 1) }
        if (good(16)) { CRB_TRY(32, 8, 16, 16, 4, 1, DG, 2, 2, 1, 1) }
    } else if (gW == 16) {
        // long contractions on few pixels: many small workgroups (16 output channels, four rows), three to a CU, so that one
        // waits for its next chunk while the others multiply (batch 64: 108 -> 48 6.6 -> 5.9 us, 204 -> 48 9.9 -> 8.4 us,
        // 288 -> 48 in chunks of 48 channels 11.2 -> 9.9 us)
        if (!DG && C_IN >= 256 && N * (gH / 4) * ceil_div(C_OUT, 16u) >= 512) { CRB_TRY(16, 4, 48, 16, 1, 1, DG, 3, 2, 1, 1) }
        if (!DG && C_IN > 64 && N * (gH / 4) * ceil_div(C_OUT, 16u) >= 512) { CRB_TRY(16, 4, 16, 16, 1, 1, DG, 3, 2, 1, 1) }
        if (half && good_half(48)) { CRB_TRY(16, 4, 16, 48, 1, 3, DG, 2, 2, 1, 1) }
        if (good(64)) { CRB_TRY(16, 8, 16, 64, 2, 4, DG, 2, 2, 1, 1) }
        if (good(48)) { CRB_TRY(16, 8, 16, 48, 2, 3, DG, 2, 2, 1, 1) }
        if (good(32)) { CRB_TRY(16, 8, 16, 32, 2, 2, DG, 2, 2, 1, 1) }
        if (good(16)) { CRB_TRY(16, 8, 16, 16, 2, 1, DG, 2, 2, 1, 1) }
    } else {
        if (!DG && C_IN >= 192 && good(16)) { CRB_TRY(8, 8, 48, 16, 1, 1, DG, 2, 2, 1, 1) }  // 330 -> 48 @8x8: 7.7 -> 6.7 us
        if (good(64)) { CRB_TRY(8, 8, 16, 64, 1, 4, DG, 2, 2, 1, 1) }
        if (good(48)) { CRB_TRY(8, 8, 16, 48, 1, 3, DG, 2, 2, 1, 1) }
        if (good(32)) { CRB_TRY(8, 8, 16, 32, 1, 2, DG, 2, 2, 1, 1) }
        if (good(16)) { CRB_TRY(8, 8, 16, 16, 1, 1, DG, 2, 2, 1, 1) }
    }
#undef CRB_TRY
    done = false;
    return CRB_OK;
}

// 1x1 / stride 1 / no padding: per image Y[n] (OC x HW) = W (OC x IC) * X[n] (IC x HW) on the native layout, i.e. the
// batched forms of the GEMM family (forward NN with a per-row bias, data gradient TN, weight gradient accumulate-NT).
static bool pointwise_shape(const crb_conv_geom *g) {
    return g->FH == 1 && g->FW == 1 && g->sH == 1 && g->sW == 1 && g->pH == 0 && g->pW == 0;
}

// 3x3, pad 1, stride 1 (output = input extent) or stride 2 with even input extents (output = half)
static bool direct_shape(const crb_conv_geom *g, u32 stride) {
    return g->FH == 3 && g->FW == 3 && g->sH == stride && g->sW == stride && g->pH == 1 && g->pW == 1 &&
           g->IH == stride * g->OH && g->IW == stride * g->OW;
}

// 3x3 / pad 1 / stride 2 on any extent whose images the tiled kernel can address
static bool tiled_s2_shape(const crb_conv_geom *g) {
    return g->FH == 3 && g->FW == 3 && g->sH == 2 && g->sW == 2 && g->pH == 1 && g->pW == 1 && g->IC >= 8 &&
           uint64_t(g->IC) * g->IH * g->IW * 4 <= 0xffffffffull && uint64_t(g->IC) * g->OC * 36 <= 0xffffffffull;
}

// Data gradient at stride > 1 through the tiled kernel, one residue class of input pixels per launch (conv3x3_tiled.h,
// TiledClass): every class is a unit-stride correlation of dY with at most ceil(FH / sH) x ceil(FW / sW) taps, run on the
// smallest square tap grid F = 1 ... 4 that holds them. Classes no tap reaches (filters smaller than the stride) are zero-filled.
static bool tiled_class_shape(const crb_conv_geom *g) {
    return (g->sH > 1 || g->sW > 1) && g->sH * g->sW <= u32(kMaxTiledClasses) && ceil_div(g->FH, g->sH) <= 4 && ceil_div(g->FW, g->sW) <= 4 &&
           uint64_t(g->OC) * g->OH * g->OW * 4 <= 0xffffffffull && uint64_t(g->IC) * g->OC * g->FH * g->FW * 4 <= 0xffffffffull;
}
template <int FH, int FW>
static int launch_tiled_class_group(const float *W, const float *dY, float *dX, const crb_conv_geom *g, TiledClass *cls, u32 ncls,
                                    hipStream_t s, const char *what) {
    // few taps: more channels per chunk, so that a chunk still holds 32 ... 128 contraction steps between two barriers
    constexpr int CI = FH * FW == 1 ? 32 : (FH * FW <= 4 ? 16 : 8);
    for (u32 k = 0; k < ncls; ++k) cls[k].pad_y += FH - 1, cls[k].pad_x += FW - 1;
    if (ceil_div(g->IH, g->sH) <= 8 && ceil_div(g->IW, g->sW) <= 8)
        return launch_tiled_classes<TiledCfg<8, 8, 64, 2, CI, true, 2, 1, FH, true, FW>>(W, dY, dX, g->N, g->OC, g->IC, g->OH, g->OW, cls, ncls, s,
                                                                                        what);
    // 8 x 16 tiles, or 4 x 32 where those pad the class grid less (28 x 28: 28 x 32 instead of 32 x 32)
    const u32 CH = ceil_div(g->IH, g->sH), CW = ceil_div(g->IW, g->sW);
    constexpr int OCT = 32;  // (64 channels for the grids of up to four taps: 3x3 stride 2 128 -> 128 @56 158 -> 151 us, but 256 -> 256 @28 151 -> 173)
    if (uint64_t(ceil_div(CH, 4u)) * 4 * ceil_div(CW, 32u) * 32 < uint64_t(ceil_div(CH, 8u)) * 8 * ceil_div(CW, 16u) * 16)
        return launch_tiled_classes<TiledCfg<4, 32, OCT, 4, CI, true, 2, 1, FH, true, FW>>(W, dY, dX, g->N, g->OC, g->IC, g->OH, g->OW, cls, ncls,
                                                                                          s, what);
    return launch_tiled_classes<TiledCfg<8, 16, OCT, 4, CI, true, 2, 1, FH, true, FW>>(W, dY, dX, g->N, g->OC, g->IC, g->OH, g->OW, cls, ncls, s,
                                                                                      what);
}
// The tap grids that have a kernel; a class runs on the smallest one that holds its nfh x nfw taps.
struct TapGrid {
    int fh, fw;
};
static constexpr TapGrid kTapGrids[] = {{1, 1}, {1, 2}, {2, 1}, {2, 2}, {2, 3}, {3, 2}, {3, 3}, {3, 4}, {4, 3}, {4, 4}};
static int tap_grid_for(u32 nfh, u32 nfw) {
    int best = -1;
    for (int i = 0; i < int(sizeof(kTapGrids) / sizeof(kTapGrids[0])); ++i)
        if (kTapGrids[i].fh >= int(nfh) && kTapGrids[i].fw >= int(nfw) &&
            (best < 0 || kTapGrids[i].fh * kTapGrids[i].fw < kTapGrids[best].fh * kTapGrids[best].fw))
            best = i;
    return best;
}
// `together`: all classes in one launch on the smallest tap grid that holds them all (a workgroup skips the steps of the taps
// its class does not have; one launch fills the chip where four would not); otherwise one launch per tap grid.
static int dgrad_by_tiled_classes(const float *W, const float *dY, float *dX, const crb_conv_geom *g, bool together, hipStream_t s) {
    const char *what = "crb_conv_dgrad";
    TiledClass cls[kMaxTiledClasses];
    int grid[kMaxTiledClasses];
    u32 ncls = 0, mh = 1, mw = 1;
    bool empty_class = false;
    for (u32 py = 0; py < g->sH && py < g->IH; ++py)
        for (u32 px = 0; px < g->sW && px < g->IW; ++px) {
            const u32 fh0 = (py + g->pH) % g->sH, fw0 = (px + g->pW) % g->sW;
            if (fh0 >= g->FH || fw0 >= g->FW) {
                empty_class = true;
                continue;
            }
            TiledClass &c = cls[ncls];
            c = TiledClass{};
            c.nfh = ceil_div(g->FH - fh0, g->sH), c.nfw = ceil_div(g->FW - fw0, g->sW);
            c.H = ceil_div(g->IH - py, g->sH), c.W = ceil_div(g->IW - px, g->sW);  // the class's pixel grid
            c.pad_y = -int((py + g->pH) / g->sH), c.pad_x = -int((px + g->pW) / g->sW);  // + tap grid - 1 at the launch
            c.fhw = g->FH * g->FW, c.tap0 = fh0 * g->FW + fw0, c.tap_i = g->sH * g->FW, c.tap_j = g->sW;
            c.out_hw = g->IH * g->IW, c.out_w = g->IW, c.osy = g->sH, c.osx = g->sW, c.oy0 = py, c.ox0 = px;
            grid[ncls] = tap_grid_for(c.nfh, c.nfw);
            mh = c.nfh > mh ? c.nfh : mh, mw = c.nfw > mw ? c.nfw : mw;
            ++ncls;
        }
    if (empty_class) {
        const uint64_t count = uint64_t(g->N) * g->IC * g->IH * g->IW;
        if (int st = crb_tensor_fill(dX, 0.f, uint32_t(count), s)) return st;
    }
    const int all = tap_grid_for(mh, mw);
    for (int gi = 0; gi < int(sizeof(kTapGrids) / sizeof(kTapGrids[0])); ++gi) {
        TiledClass grp[kMaxTiledClasses];
        u32 n = 0;
        for (u32 k = 0; k < ncls; ++k)
            if (together ? gi == all : grid[k] == gi) grp[n++] = cls[k];
        if (n == 0) continue;
        int st;
        switch (gi) {
            case 0: st = launch_tiled_class_group<1, 1>(W, dY, dX, g, grp, n, s, what); break;
            case 1: st = launch_tiled_class_group<1, 2>(W, dY, dX, g, grp, n, s, what); break;
            case 2: st = launch_tiled_class_group<2, 1>(W, dY, dX, g, grp, n, s, what); break;
            case 3: st = launch_tiled_class_group<2, 2>(W, dY, dX, g, grp, n, s, what); break;
            case 4: st = launch_tiled_class_group<2, 3>(W, dY, dX, g, grp, n, s, what); break;
            case 5: st = launch_tiled_class_group<3, 2>(W, dY, dX, g, grp, n, s, what); break;
            case 6: st = launch_tiled_class_group<3, 3>(W, dY, dX, g, grp, n, s, what); break;
            case 7: st = launch_tiled_class_group<3, 4>(W, dY, dX, g, grp, n, s, what); break;
            case 8: st = launch_tiled_class_group<4, 3>(W, dY, dX, g, grp, n, s, what); break;
            default: st = launch_tiled_class_group<4, 4>(W, dY, dX, g, grp, n, s, what); break;
        }
        if (st) return st;
    }
    return CRB_OK;
}
// The launches must bring work: 128 workgroups over the classes (24 and 16 contraction channels, 64 on class grids up to 8 x 8,
// when there is a single class, as for 1x1 filters), tiles at least a quarter full, five contraction channels. `together`: a class
// brings fewer than 1024 workgroups, so all classes share one launch (the steps of the taps a class does not have are skipped). Against the engine's class launches / its one gather over all
// taps on random layers: 32 -> 16 @56 5x5 stride 3 batch 128 317 -> 85 us, 256 -> 32 @28 7x7 stride 2 batch 32 261 -> 97,
// 64 -> 256 @14 2x2 stride 2 batch 128 131 -> 23, 3 -> 128 @28 4x4 stride 2 batch 128 208 -> 60; class grids that fill their
// tiles less stay with the engine (256 -> 32 @8 7x7 stride 3 batch 32, 3 x 3 pixel classes on 8 x 8 tiles: 55 against 115 us).
static bool tiled_classes_pay(const crb_conv_geom *g, bool *together = nullptr) {
    if (!tiled_class_shape(g) || g->OC < 5) return false;
    u32 nc = 0;
    for (u32 py = 0; py < g->sH && py < g->IH; ++py)
        for (u32 px = 0; px < g->sW && px < g->IW; ++px)
            if ((py + g->pH) % g->sH < g->FH && (px + g->pW) % g->sW < g->FW) ++nc;
    const u32 CH = ceil_div(g->IH, g->sH), CW = ceil_div(g->IW, g->sW);
    const bool small = CH <= 8 && CW <= 8;
    const uint64_t tiles = small ? uint64_t(g->N) : uint64_t(g->N) * ceil_div(CH, 8u) * ceil_div(CW, 16u);
    const uint64_t wgs = tiles * ceil_div(g->IC, small ? 64u : 32u);  // per class
    const uint64_t padded = small ? 64 : uint64_t(ceil_div(CH, 8u)) * 8 * ceil_div(CW, 16u) * 16;
    if (together) *together = wgs < 1024;
    // (8 -> 3 @64 1x1 stride 2 batch 4: 6.8 against 4.3 us; 32 -> 256 @16 1x1 stride 2 batch 32, 8 x 8 class grid: 16.6 against 10.4)
    if (nc == 1) return wgs >= 24 && g->OC >= (small ? 64u : 16u);
    return wgs * nc >= 128 && 4 * uint64_t(CH) * CW >= padded;
}

// F x F (3 or 5), stride 1, the same padding 0 ... F - 1 on both axes, and tensors the tiled kernel can address
static bool tiled_s1_shape(const crb_conv_geom *g, u32 F) {
    return g->FH == F && g->FW == F && g->sH == 1 && g->sW == 1 && g->pH == g->pW && g->pH <= F - 1 &&
           tiled_fits(g->IC > g->OC ? g->IC : g->OC, g->IC > g->OC ? g->OC : g->IC, g->IH > g->OH ? g->IH : g->OH,
                      g->IW > g->OW ? g->IW : g->OW, F * F);
}

// 1x1, stride 2, no padding, even input extents, at most 64 channels on either side (conv1x1_s2.h)
static bool shortcut_shape(const crb_conv_geom *g) {
    return g->FH == 1 && g->FW == 1 && g->sH == 2 && g->sW == 2 && g->pH == 0 && g->pW == 0 && g->IH == 2 * g->OH &&
           g->IW == 2 * g->OW && g->IC % 4 == 0 && g->IC <= kScMaxC && g->OC <= kScMaxC;
}

// 3x3 / pad 1 / stride 1 on 2x2 images: dense products over (channel, pixel) pairs (gemm_internal.h)
static bool tiny2x2_shape(const crb_conv_geom *g) {
    return direct_shape(g, 1) && g->IH == 2 && g->IW == 2 && uint64_t(g->OC) * g->IC * 16 <= 0x7fffffffull;
}

// Weight gradient of 3x3 / stride 1 layers with padding 0 ... 2 on any extent (conv3x3_tiled_wgrad.h), <TH, TW, NOB, NIB, OCC>: 64-pixel tiles of
// the shape that pads the image least, blocks of 64 x 64 channels (32 on a side with at most 32 channels).
// `run` = false only computes the plan (workspace size).
static bool wgrad_tiled(const crb_conv_geom *g, bool run, const float *dY, const float *X, float *dW, float *ws, hipStream_t s,
                        TiledWgradPlan &plan, int &status) {
    // (images below 12 x 12 pad their 8 x 8 tiles too much: the engine's flat pixel contraction is as fast or faster there)
    const bool shape_ok = g->FH == 3 && g->FW == 3 && g->sH == 1 && g->sW == 1 && g->pH == g->pW && g->pH <= 2;
    if (!shape_ok || !tiled_wgrad_fits(g->N, g->IC, g->OC, std::max(g->IH, g->OH), std::max(g->IW, g->OW)) || g->OH * g->OW < 144)
        return false;
    const u32 H = g->OH, W = g->OW;
    auto padded = [&](u32 th, u32 tw) { return uint64_t(ceil_div(H, th)) * th * ceil_div(W, tw) * tw; };
    const uint64_t p416 = padded(4, 16), p88 = padded(8, 8), p232 = padded(2, 32);
    const int shape = (p416 <= p88 && p416 <= p232) ? 0 : (p88 <= p232 ? 1 : 2);
    // tiles at least two thirds full (256 -> 256 @18x18 batch 32, 56 % full: 208 against the engine's 155 us)
    if (3 * uint64_t(H) * W < 2 * std::min(p416, std::min(p88, p232))) return false;
    // blocks of 32 channels at least three quarters full on both sides, and at least four tiles per workgroup (below that the
    // engine's flat pixel contraction is as fast or faster: 3 -> 64 @224 batch 8 99 against 143 us, 8 -> 8 @100 33 against 43)
    if (g->IC < 24 || g->OC < 24) return false;
#define CRB_TW(TH, TW, NOB, NIB)                                                                                        \
    {                                                                                                                   \
        typedef TiledWgradCfg<TH, TW, NOB, NIB> C;                                                                      \
        plan = tiled_wgrad_plan<C>(g->N, g->IC, g->OC, H, W);                                                           \
        if (uint64_t(plan.tiles_total) * plan.pairs < 1024) return false;                                               \
        if (run) status = launch_tiled_wgrad<C>(dY, X, dW, ws, plan, g->IC, g->OC, H, W, g->IH, g->IW, g->pH, s, "crb_conv_wgrad"); \
        return true;                                                                                                    \
    }
#define CRB_TW_SHAPES(NOB, NIB)            \
    {                                      \
        if (shape == 0) CRB_TW(4, 16, NOB, NIB) \
        if (shape == 1) CRB_TW(8, 8, NOB, NIB)  \
        CRB_TW(2, 32, NOB, NIB)            \
    }
    if (g->OC > 32 && g->IC > 32) CRB_TW_SHAPES(2, 2)
    if (g->OC > 32) CRB_TW_SHAPES(2, 1)
    if (g->IC > 32) CRB_TW_SHAPES(1, 2)
    CRB_TW_SHAPES(1, 1)
#undef CRB_TW_SHAPES
#undef CRB_TW
}

// ---- direct 3x3 / pad 1 weight gradient (stride 1 and 2) ---------------------------------------------------------
// One entry per configuration <W, TR, TI, OCC>; `run` = false only computes the plan (workspace size).
constexpr u32 kWgradTargetWgs = 256;  // one workgroup per CU: pairs x splits (two per CU for wide layers, see wgrad_direct_plan)

// dW == nullptr (with run): the slices are left in ws, unsummed.
template <class Cfg>
static bool wgrad_cfg(const crb_conv_geom *g, bool run, const float *dY, const float *X, float *dW, float *ws, hipStream_t s,
                      WgradDirectPlan &plan, int &status) {
    if (!wgrad_direct_fits<Cfg>(g->N, g->IC, g->OC, g->OH, g->OW)) return false;
    plan = wgrad_direct_plan<Cfg>(g->N, g->IC, g->OC, g->OH, kWgradTargetWgs);
    if (run) status = launch_wgrad_direct<Cfg>(dY, X, dW, ws, plan, g->N, g->IC, g->OC, g->OH, s, "crb_conv_wgrad");
    return true;
}

// Configurations <W (dY width), TR, TI, OCC, S, WAVES>.
// One workgroup per CU (the usual plan: pairs x splits = 256) runs the eight-wave form, so that every SIMD holds two waves;
// wide layers, whose plan puts two four-wave workgroups on a CU anyway, keep the four-wave form (measured: 1-5 % faster
// there). Both forms produce identical bits, and the plan (splits, workspace) does not depend on the form.
template <int W, int TR, int TI, int OCC, int S>
static bool wgrad_cfg2(const crb_conv_geom *g, bool run, const float *dY, const float *X, float *dW, float *ws, hipStream_t s,
                       WgradDirectPlan &plan, int &status) {
    typedef WgradCfg<W, TR, TI, OCC, S, 4> Four;
    typedef WgradCfg<W, TR, TI, 1, S, 8> Eight;
    if (!wgrad_direct_fits<Four>(g->N, g->IC, g->OC, g->OH, g->OW)) return false;
    const WgradDirectPlan p = wgrad_direct_plan<Four>(g->N, g->IC, g->OC, g->OH, kWgradTargetWgs);
    if (uint64_t(p.pairs) * p.splits > kWgradTargetWgs) return wgrad_cfg<Four>(g, run, dY, X, dW, ws, s, plan, status);
    return wgrad_cfg<Eight>(g, run, dY, X, dW, ws, s, plan, status);
}
static bool wgrad_direct(const crb_conv_geom *g, bool run, const float *dY, const float *X, float *dW, float *ws,
                         hipStream_t s, WgradDirectPlan &plan, int &status) {
    if (direct_shape(g, 1) && wgrad_image_fits(g->IC, g->OH, g->OW)) {  // image layers: (channel, tap) pairs on the MFMA columns
        plan = wgrad_image_plan(g->N, g->IC, g->OC, g->OH);
        if (run) status = launch_wgrad_image(dY, X, dW, ws, plan, g->IC, g->OC, g->OH, s, "crb_conv_wgrad");
        return true;
    }
    if (direct_shape(g, 1)) {
        if (g->OW == 32) return wgrad_cfg2<32, 8, 1, 2, 1>(g, run, dY, X, dW, ws, s, plan, status);
        if (g->OW == 16)
            return wgrad_cfg2<16, 16, 1, 2, 1>(g, run, dY, X, dW, ws, s, plan, status) ||
                   wgrad_cfg2<16, 8, 1, 2, 1>(g, run, dY, X, dW, ws, s, plan, status);
        if (g->OW == 8)
            return wgrad_cfg2<8, 8, 4, 2, 1>(g, run, dY, X, dW, ws, s, plan, status) ||
                   wgrad_cfg2<8, 8, 2, 2, 1>(g, run, dY, X, dW, ws, s, plan, status);
        if (g->OW == 4)  // 4x4 images: 8 (or 4) whole images per tile
            return wgrad_cfg2<4, 4, 8, 2, 1>(g, run, dY, X, dW, ws, s, plan, status) ||
                   wgrad_cfg2<4, 4, 4, 2, 1>(g, run, dY, X, dW, ws, s, plan, status);
    } else if (direct_shape(g, 2)) {
        if (g->OW == 32) return wgrad_cfg2<32, 4, 1, 1, 2>(g, run, dY, X, dW, ws, s, plan, status);
        if (g->OW == 16)
            return wgrad_cfg2<16, 4, 1, 2, 2>(g, run, dY, X, dW, ws, s, plan, status) ||
                   wgrad_cfg2<16, 8, 1, 1, 2>(g, run, dY, X, dW, ws, s, plan, status);
        if (g->OW == 8)
            return wgrad_cfg2<8, 8, 2, 1, 2>(g, run, dY, X, dW, ws, s, plan, status) ||
                   wgrad_cfg2<8, 4, 2, 1, 2>(g, run, dY, X, dW, ws, s, plan, status);
    }
    return false;
}

// ---- data gradient and weight gradient of one layer in one launch ------------------------------------------------------
// The two gradients of a layer are independent (dX = f(W, dY), dW += f(dY, X)), and each of their kernels alone leaves the
// chip idle while it ramps up, loads its first tiles and drains. Launched as one grid — the longer-running kind of workgroup
// first — they share every compute unit and those fixed phases are paid once.
template <class DCfg, class WCfg>
__global__ void __launch_bounds__(kThreads, 2) conv_bwd_kernel(DirectArgs d, WgradArgs w, u32 first_wgs, u32 dgrad_first) {
    constexpr int SM = DCfg::SMEM_FLOATS > WCfg::SMEM ? DCfg::SMEM_FLOATS : WCfg::SMEM;
    __shared__ __attribute__((aligned(16))) float smem[SM];
    // the longer-running kind takes the low workgroup ids, which are dispatched first
    const bool first = blockIdx.x < first_wgs;
    const u32 bid = first ? blockIdx.x : blockIdx.x - first_wgs;
    if (first == (dgrad_first != 0))
        conv3x3_body<DCfg>(d, bid, smem);
    else
        wgrad3x3_body<WCfg>(w, bid, smem);
}

// One (data-gradient configuration, weight-gradient configuration) pair; `run` = false only computes the plan.
template <class DCfg, class WCfg, bool DGRAD_FIRST = false>
static bool bwd_pair(const crb_conv_geom *g, bool run, const float *Wt, const float *dY, const float *X, float *dX, float *dW,
                     float *ws, hipStream_t s, WgradDirectPlan &plan, int &status) {
    if (!direct_fits<DCfg>(g->OC, g->OH, g->OW) || !wgrad_direct_fits<WCfg>(g->N, g->IC, g->OC, g->OH, g->OW)) return false;
    plan = wgrad_direct_plan<WCfg>(g->N, g->IC, g->OC, g->OH, kWgradTargetWgs);
    if (!run) return true;
    DirectArgs d;
    WgradArgs w;
    uint64_t dwgs = direct_args<DCfg>(d, Wt, dY, dX, nullptr, g->N, g->OC, g->IC, g->OH, g->OH, 0);
    const uint64_t wwgs = wgrad_direct_args<WCfg>(w, dY, X, dW, ws, plan, g->IC, g->OC, g->OH);
    // Both bodies read dY. A weight-gradient slice z runs on XCD z % 8 and covers tiles_per_z consecutive tiles; the data
    // gradient's tiles over the same rows are dealt to that XCD too, so that its L2 serves the second reader.
    if (!DCfg::MI && plan.splits >= kXcds) {
        const u32 run = plan.tiles_per_z * u32(WCfg::TR * WCfg::TI) / u32(DCfg::ROWS);  // data-gradient tiles per slice
        if (run >= 2 && (run & (run - 1)) == 0 && u32(WCfg::TR * WCfg::TI) % u32(DCfg::ROWS) == 0) {
            u32 sh = 0;
            while ((1u << sh) < run) ++sh;
            d.xcd_shift = sh;
            const u32 round = kXcds << sh;
            dwgs = uint64_t(ceil_div(d.tiles_total, round)) * round * d.oc_tiles;
        }
    }
    if (dwgs + wwgs > 0x7fffffffull) {
        status = fail(CRB_EINVAL_SHAPE, "crb_conv_bwd: launch grid too large");
        return true;
    }
    hipLaunchKernelGGL((conv_bwd_kernel<DCfg, WCfg>), dim3(u32(dwgs + wwgs)), dim3(kThreads), 0, s, d, w,
                       u32(DGRAD_FIRST ? dwgs : wwgs), DGRAD_FIRST ? 1u : 0u);
    status = check_launch("crb_conv_bwd");
    if (status == CRB_OK && plan.splits > 1 && dW)  // dW == nullptr: the slices stay in ws, unsummed
        status = launch_splitk_reduce(ws, dW, g->OC * g->IC * 9, plan.splits, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, "crb_conv_bwd");
    return true;
}

// Pairs for the layer shapes of CIFAR residual networks. The weight-gradient configuration is the one crb_conv_wgrad picks
// for the shape (same split plan, same workspace); the data-gradient configuration has the chunking of the one
// crb_conv_dgrad picks (only the output-channel tile may differ, which does not enter any element's summation order), so
// results are identical to crb_conv_dgrad followed by crb_conv_wgrad.
static bool bwd_fused(const crb_conv_geom *g, bool run, const float *Wt, const float *dY, const float *X, float *dX, float *dW,
                      float *ws, hipStream_t s, WgradDirectPlan &plan, int &status) {
#define CRB_PAIR(...) bwd_pair<__VA_ARGS__>(g, run, Wt, dY, X, dX, dW, ws, s, plan, status)
    typedef DirectCfg<32, 8, 16, 16, 4, 1, true, 2, 1, 1, 3, 4> D32a;
    typedef DirectCfg<16, 8, 16, 32, 2, 2, true, 2, 2, 1> D16a;             // chunks of 16 channels
    typedef DirectCfg<16, 8, 32, 32, 2, 2, true, 2, 1, 1, 3, 2> D16r;       // one resident chunk of up to 32
    typedef DirectCfg<8, 8, 16, 32, 1, 2, true, 2, 2, 1> D8a;
    typedef DirectCfg<16, 8, 8, 16, 2, 1, true, 2, 2, 2> D16s2;             // chunks of 8
    typedef DirectCfg<16, 8, 16, 16, 2, 1, true, 2, 2, 2> D16s2c;           // chunks of 16
    // growth-12 dense layers (48 -> 12): the data gradient reads 9..12 channels and writes 33..48; the configurations are
    // the ones try_direct<true, 1> picks for these shapes
    typedef DirectCfg<32, 4, 12, 48, 2, 3, true, 2, 1, 1, 3, 2> D32g;
    typedef DirectCfg<16, 4, 12, 48, 1, 3, true, 2, 1, 1> D16g;
    typedef DirectCfg<8, 8, 16, 16, 1, 1, true, 2, 2, 1> D8g;
    typedef WgradCfg<32, 8, 1, 2, 1> W32a;
    typedef WgradCfg<16, 16, 1, 2, 1> W16a;
    typedef WgradCfg<8, 8, 4, 2, 1> W8a;
    typedef WgradCfg<16, 8, 1, 2, 1> W16b;  // what crb_conv_wgrad falls back to when the image height or the batch does not fit
    typedef WgradCfg<8, 8, 2, 2, 1> W8b;
    typedef WgradCfg<16, 4, 1, 2, 2> W16s2;  // 4-row tiles: 51 KB of LDS, so that a workgroup of each kind shares a CU (8-row tiles: 92 KB)
    const u32 ci = g->OC, co = g->IC;  // channels the data gradient reads / writes
    if (direct_shape(g, 1)) {
        if (ci > 8 && ci <= 12 && co > 32 && co <= 48) {
            if (g->OW == 32) return CRB_PAIR(D32g, W32a);
            if (g->OW == 16) return CRB_PAIR(D16g, W16a) || CRB_PAIR(D16g, W16b);
            if (g->OW == 8) return CRB_PAIR(D8g, W8a) || CRB_PAIR(D8g, W8b);
        }
        if (g->OW == 32 && ci <= 16 && ci > 8 && co <= 16) return CRB_PAIR(D32a, W32a);
        if (g->OW == 16 && co > 16 && co <= 64 && ci > 8)
            return one_chunk_w16(g->N, ci, co, g->OH) ? CRB_PAIR(D16r, W16a) : CRB_PAIR(D16a, W16a);
        if (g->OW == 8 && co <= 64 && ci > 8) return CRB_PAIR(D8a, W8a);
    } else if (direct_shape(g, 2)) {
        if (g->OW == 16 && co <= 16) return s2_dgrad_w16_c16(g->N, ci, co, g->OH) ? CRB_PAIR(D16s2c, W16s2) : CRB_PAIR(D16s2, W16s2);
        // 8-wide stride-2 layers (32 -> 64) run the two gradients as two launches: the weight gradient's 8-row tiles of two
        // images need 92 KB of LDS, so a CU held one workgroup of the pair at a time and the one launch took as long as
        // both (15.1 us against 6.8 + 6.4), and tile shapes small enough for two to share a CU were slower still
    }
#undef CRB_PAIR
    return false;
}

__global__ void __launch_bounds__(256) conv_bias_kernel(float *__restrict__ Y, const float *__restrict__ bias,
                                                        u32 total, u32 C, FastDiv hw) {
    const u32 i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const u32 plane = hw.div(i);
    Y[i] += bias[plane % C];
}

// Bias gradient dB[c] += sum over (n, hw) of dY[n,c,hw], in two passes with a fixed association (bit-reproducible).
// Pass 1 views dY as a (N x C*HW) matrix and sums its columns over a slice of the rows: a workgroup covers 64 columns
// (16 lanes x 4 floats, whole 256-byte row segments) with 16 row-lanes, or 32 columns x 8 row-lanes with scalar loads when
// the matrix is not 16-byte friendly; the row-lanes are combined through LDS in lane order. part[slice][column].
template <bool VEC>
__global__ void __launch_bounds__(256) bias_grad_colsum_kernel(const float *__restrict__ in, float *__restrict__ part, u32 rows,
                                                               u32 cols, u32 rows_per_slice) {
    constexpr u32 CL = VEC ? 16 : 32, RL = 256 / CL, W = VEC ? 4 : 1;
    __shared__ float red[RL][CL * W + 4];
    const u32 o = threadIdx.x % CL, g = threadIdx.x / CL;
    const u32 c = (blockIdx.x * CL + o) * W;
    const u32 r0 = blockIdx.y * rows_per_slice, r1 = r0 + rows_per_slice < rows ? r0 + rows_per_slice : rows;
    float acc[2][W];
#pragma unroll
    for (u32 k = 0; k < W; ++k) acc[0][k] = acc[1][k] = 0.f;
    if (c < cols) {
        const float *p = in + c;
        u32 r = r0 + g;
        for (; r + RL < r1; r += 2 * RL) {
            if constexpr (VEC) {
                const v4f a = *reinterpret_cast<const v4f *>(p + size_t(r) * cols);
                const v4f b = *reinterpret_cast<const v4f *>(p + size_t(r + RL) * cols);
                acc[0][0] += a.x, acc[0][1] += a.y, acc[0][2] += a.z, acc[0][3] += a.w;
                acc[1][0] += b.x, acc[1][1] += b.y, acc[1][2] += b.z, acc[1][3] += b.w;
            } else {
                acc[0][0] += p[size_t(r) * cols];
                acc[1][0] += p[size_t(r + RL) * cols];
            }
        }
        if (r < r1) {
            if constexpr (VEC) {
                const v4f a = *reinterpret_cast<const v4f *>(p + size_t(r) * cols);
                acc[0][0] += a.x, acc[0][1] += a.y, acc[0][2] += a.z, acc[0][3] += a.w;
            } else {
                acc[0][0] += p[size_t(r) * cols];
            }
        }
    }
#pragma unroll
    for (u32 k = 0; k < W; ++k) red[g][o * W + k] = acc[0][k] + acc[1][k];
    __syncthreads();
    const u32 j = blockIdx.x * CL * W + threadIdx.x;
    if (threadIdx.x < CL * W && j < cols) {
        float v = red[0][threadIdx.x];
#pragma unroll
        for (u32 k = 1; k < RL; ++k) v += red[k][threadIdx.x];
        part[size_t(blockIdx.y) * cols + j] = v;
    }
}

// Pass 2: one workgroup per channel folds its HW columns of every slice: dB[c] += sum_{slice, hw} part[slice][c*HW + hw].
__global__ void __launch_bounds__(256) bias_grad_fold_kernel(const float *__restrict__ part, float *__restrict__ dB, u32 HW, u32 cols,
                                                             u32 slices) {
    __shared__ float red[256];
    const u32 c = blockIdx.x;
    float s = 0.f;
    for (u32 sl = 0; sl < slices; ++sl) {
        const float *p = part + size_t(sl) * cols + c * HW;
        for (u32 i = threadIdx.x; i < HW; i += 256) s += p[i];
    }
    red[threadIdx.x] = s;
    __syncthreads();
    for (u32 w = 128; w > 0; w >>= 1) {
        if (threadIdx.x < w) red[threadIdx.x] += red[threadIdx.x + w];
        __syncthreads();
    }
    if (threadIdx.x == 0) dB[c] += red[0];
}

// Row slicing of the bias gradient's first pass: rows are cut into slices until the grid covers the chip (at least 16
// rows per slice).
struct BiasGradPlan {
    u32 col_wgs, slices, rows_per_slice;
};
static BiasGradPlan bias_grad_plan(u32 N, u32 cols, bool vec) {
    BiasGradPlan p;
    p.col_wgs = ceil_div(cols, vec ? 64u : 32u);
    u32 slices = p.col_wgs >= 512 ? 1 : ceil_div(512u, p.col_wgs);
    if (slices > ceil_div(N, 16u)) slices = ceil_div(N, 16u);
    p.rows_per_slice = ceil_div(N, slices);
    p.slices = ceil_div(N, p.rows_per_slice);
    return p;
}

// ---- built-in scratch of the entry point that allocates nothing -----------------------------------------------------------
// Device memory that exists as long as the code object is loaded: one copy per GPU, at an address of its own on each. In
// host code the array's name is only a handle for hipGetSymbolAddress; kernels and copies get the address that call
// returns for the current device.
constexpr size_t kStaticScratchBytes = CRB_NOALLOC_SCRATCH_BYTES;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];
constexpr int kMaxDevices = 64;
static std::mutex g_static_mu;
static void *g_static_ptr[kMaxDevices];

// The current device's copy of `scratch` (looked up once per device, with that device current).
static int static_scratch_ptr(const char *what, void **out) {
    int dev = 0;
    if (hipError_t e = hipGetDevice(&dev)) return check_hip(e, what);
    if (dev < 0 || dev >= kMaxDevices) return fail(CRB_EHIP, "%s: device ordinal %d out of range", what, dev);
    std::lock_guard<std::mutex> lk(g_static_mu);
    if (!g_static_ptr[dev]) {
        void *p = nullptr;
        if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) return check_hip(e, what);
        if (!p) return fail(CRB_EHIP, "%s: the built-in scratch buffer has no device address", what);
        g_static_ptr[dev] = p;
    }
    *out = g_static_ptr[dev];
    return CRB_OK;
}

}  // namespace crb

using namespace crb;

extern "C" {

int crb_conv_fwd(const float *W, const float *X, float *Y, const float *bias_or_null, const crb_conv_geom *g,
                 uint32_t flags, void *stream) {
    if (!W || !X || !Y) return fail(CRB_ENULL, "crb_conv_fwd: null operand");
    if (int st = check_geom("crb_conv_fwd", g)) return st;
    const u32 M = g->OC, N = g->N * g->OH * g->OW, K = g->IC * g->FH * g->FW;
    Im2colPixRows b{make_im2col(X, g)};
    NchwEpi e{Y, bias_or_null, g->OC, g->OH * g->OW, (flags & CRB_FLAG_RELU) ? u32(EPI_RELU) : 0u,
              FastDiv(g->OH * g->OW), 0u};
    hipStream_t s = hipStream_t(stream);
    if (pointwise_shape(g) && aligned16(X) && aligned16(Y)) {
        bool done;
        int st = try_pointwise<false>(W, X, Y, bias_or_null, g->N, g->IC, g->OC, g->OH, g->OW, flags & CRB_FLAG_RELU, s,
                                      "crb_conv_fwd", done);
        if (done) return st;
    }
    if (pointwise_shape(g))
        return gemm_nn_rowbias(W, X, Y, g->OC, g->IH * g->IW, g->IC, g->N, bias_or_null,
                               (flags & CRB_FLAG_RELU) ? u32(EPI_RELU) : 0u, s, "crb_conv_fwd");
    if (tiny2x2_shape(g) && aligned16(X) && aligned16(Y))
        return conv2x2_fwd(W, X, Y, bias_or_null, g->N, g->IC, g->OC, (flags & CRB_FLAG_RELU) ? u32(EPI_RELU) : 0u, s, "crb_conv_fwd");
    if (aligned16(X) && aligned16(Y) && (direct_shape(g, 1) || direct_shape(g, 2))) {
        bool done;
        int st = g->sH == 1 ? try_direct<false, 1>(W, X, Y, bias_or_null, g->N, g->IC, g->OC, g->OH, g->OW, g->IH,
                                                   flags & CRB_FLAG_RELU, s, "crb_conv_fwd", done)
                            : try_direct<false, 2>(W, X, Y, bias_or_null, g->N, g->IC, g->OC, g->OH, g->OW, g->IH,
                                                   flags & CRB_FLAG_RELU, s, "crb_conv_fwd", done);
        if (done) return st;
    }
    // any other extent, padding 0 ... F - 1 (and operands that are only 4-byte aligned)
    if (tiled_s1_shape(g, 3) && tiled_pays(g->N, g->IC, g->OC, g->OH, g->OW, 9))
        return launch_tiled_any<false>(W, X, Y, bias_or_null, g->N, g->IC, g->OC, g->OH, g->OW, flags & CRB_FLAG_RELU, s, "crb_conv_fwd",
                                       g->IH, g->IW, int(g->pH));
    if (tiled_s1_shape(g, 5) && tiled_pays(g->N, g->IC, g->OC, g->OH, g->OW, 25))
        return launch_tiled_any<false, 1, 5>(W, X, Y, bias_or_null, g->N, g->IC, g->OC, g->OH, g->OW, flags & CRB_FLAG_RELU, s, "crb_conv_fwd",
                                             g->IH, g->IW, int(g->pH));
    if (tiled_s2_shape(g) && tiled_pays(g->N, g->IC, g->OC, g->OH, g->OW, 9))
        return launch_tiled_any<false, 2>(W, X, Y, bias_or_null, g->N, g->IC, g->OC, g->OH, g->OW, flags & CRB_FLAG_RELU, s, "crb_conv_fwd",
                                          g->IH, g->IW);
    if (K % 4 == 0 && aligned16(W)) {
        MatK<true> a{W, M, K, 0};
        return run_nchw(a, b, e, M, N, K, s, "crb_conv_fwd");
    }
    MatK<false> a{W, M, K, 0};
    return run_nchw(a, b, e, M, N, K, s, "crb_conv_fwd");
}

int crb_conv_dgrad(const float *W, const float *dY, float *dX, const crb_conv_geom *g, void *stream) {
    if (!W || !dY || !dX) return fail(CRB_ENULL, "crb_conv_dgrad: null operand");
    if (int st = check_geom("crb_conv_dgrad", g)) return st;
    if (pointwise_shape(g) && aligned16(dY) && aligned16(dX)) {
        bool done;
        int st = try_pointwise<true>(W, dY, dX, nullptr, g->N, g->OC, g->IC, g->OH, g->OW, 0, hipStream_t(stream),
                                     "crb_conv_dgrad", done);
        if (done) return st;
    }
    if (pointwise_shape(g))
        return gemm_tn_batched(W, dY, dX, g->IC, g->IH * g->IW, g->OC, g->N, hipStream_t(stream), "crb_conv_dgrad");
    if (tiny2x2_shape(g) && aligned16(dY) && aligned16(dX))
        return conv2x2_dgrad(W, dY, dX, g->N, g->IC, g->OC, hipStream_t(stream), "crb_conv_dgrad");
    if (aligned16(dY) && aligned16(dX) && (direct_shape(g, 1) || direct_shape(g, 2))) {
        bool done;
        // the pixel grid and the staged tensor are dY in both cases (at stride 1 dY and dX have the same extent)
        int st = g->sH == 1 ? try_direct<true, 1>(W, dY, dX, nullptr, g->N, g->OC, g->IC, g->OH, g->OW, g->OH, 0,
                                                  hipStream_t(stream), "crb_conv_dgrad", done)
                            : try_direct<true, 2>(W, dY, dX, nullptr, g->N, g->OC, g->IC, g->OH, g->OW, g->OH, 0,
                                                  hipStream_t(stream), "crb_conv_dgrad", done);
        if (done) return st;
    }
    if (shortcut_shape(g) && aligned16(dX))
        return launch_sc_dgrad(W, dY, dX, g->N, g->IC, g->OC, g->OH, g->OW, hipStream_t(stream), "crb_conv_dgrad");
    // any other extent, padding 0 ... F - 1 (and operands that are only 4-byte aligned): the pixel grid is dX, the staged tensor dY
    if (tiled_s1_shape(g, 3) && tiled_pays(g->N, g->OC, g->IC, g->IH, g->IW, 9))
        return launch_tiled_any<true>(W, dY, dX, nullptr, g->N, g->OC, g->IC, g->IH, g->IW, 0, hipStream_t(stream), "crb_conv_dgrad", g->OH,
                                      g->OW, int(2 - g->pH));
    if (tiled_s1_shape(g, 5) && tiled_pays(g->N, g->OC, g->IC, g->IH, g->IW, 25))
        return launch_tiled_any<true, 1, 5>(W, dY, dX, nullptr, g->N, g->OC, g->IC, g->IH, g->IW, 0, hipStream_t(stream), "crb_conv_dgrad",
                                            g->OH, g->OW, int(4 - g->pH));
    const u32 FHW = g->FH * g->FW;
    {
        bool together = false;
        if (tiled_classes_pay(g, &together)) return dgrad_by_tiled_classes(W, dY, dX, g, together, hipStream_t(stream));
    }
    if ((g->sH > 1 || g->sW > 1) && dgrad_classes_pay(g)) return dgrad_by_classes(W, dY, dX, g, hipStream_t(stream));
    const u32 M = g->IC, N = g->N * g->IH * g->IW, K = g->OC * FHW;
    SepK a{W, g->IC, FHW, g->IC * FHW, 1, FastDiv(FHW)};
    DgradGather b;
    b.dY = dY;
    b.npix = N;
    b.OH = g->OH, b.OW = g->OW;
    b.img_stride = g->OC * g->OH * g->OW;
    b.chan_stride = g->OH * g->OW;
    b.pH = g->pH, b.pW = g->pW;
    b.ihw.init(g->IH * g->IW), b.iw.init(g->IW), b.fhw.init(FHW), b.fw.init(g->FW);
    b.sH.init(g->sH), b.sW.init(g->sW);
    b.unit_stride = g->sH == 1 && g->sW == 1;
    NchwEpi e{dX, nullptr, g->IC, g->IH * g->IW, 0u, FastDiv(g->IH * g->IW), 0u};
    return run_nchw(a, b, e, M, N, K, hipStream_t(stream), "crb_conv_dgrad");
}

size_t crb_conv_wgrad_workspace_bytes(const crb_conv_geom *g) {
    if (check_geom("crb_conv_wgrad_workspace_bytes", g)) return 0;
    if (pointwise_shape(g)) {  // pixel-contraction kernel, or (unaligned / wide layers) the accumulate-NT GEMM form
        const size_t gemm = uint64_t(g->IH) * g->IW * g->N > 0x7fffffffull ? 0 : gemm_scratch_bytes(g->OC, g->IC, g->IH * g->IW * g->N, 1);
        if (!pw_wgrad_fits(g->IC, g->OC, g->IH * g->IW)) return gemm;
        return std::max(gemm, pw_wgrad_plan(g->N, g->IC, g->OC, g->IH * g->IW).workspace_bytes);
    }
    if (tiny2x2_shape(g)) return size_t(g->OC) * g->IC * 16 * sizeof(float);  // (oc, p) x (ic, p') product before the tap fold
    if (shortcut_shape(g)) return sc_wgrad_plan(g->N, g->IC, g->OC, g->OH, g->OW).workspace_bytes;
    {
        WgradDirectPlan dp;
        TiledWgradPlan tp;
        int st = 0;
        if (wgrad_direct(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st)) return dp.workspace_bytes;
        if (wgrad_tiled(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, tp, st)) return tp.workspace_bytes;
    }
    const WgradPlan p = wgrad_plan(g);
    return p.splits > 1 ? size_t(p.splits) * p.M * p.Ncols * sizeof(float) : 0;
}

int crb_conv_wgrad(const float *dY, const float *X, float *dW, const crb_conv_geom *g, void *workspace,
                   size_t workspace_bytes, void *stream) {
    if (!dY || !X || !dW) return fail(CRB_ENULL, "crb_conv_wgrad: null operand");
    if (int st = check_geom("crb_conv_wgrad", g)) return st;
    if (workspace && !aligned16(workspace)) return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace is not 16-byte aligned");
    hipStream_t s = hipStream_t(stream);
    if (pointwise_shape(g) && pw_wgrad_fits(g->IC, g->OC, g->IH * g->IW) && aligned16(dY) && aligned16(X)) {
        const PwWgradPlan pp = pw_wgrad_plan(g->N, g->IC, g->OC, g->IH * g->IW);
        float *pws = static_cast<float *>(workspace);
        if (pp.workspace_bytes) {
            if (pws) {
                if (workspace_bytes < pp.workspace_bytes)
                    return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace %zu bytes < required %zu", workspace_bytes, pp.workspace_bytes);
            } else if (int sg = scratch_get(pp.workspace_bytes, s, "crb_conv_wgrad", &pws)) {
                return sg;
            }
        }
        return launch_pw_wgrad(dY, X, dW, pws, pp, g->IC, g->OC, g->IH * g->IW, s, "crb_conv_wgrad");
    }
    if (pointwise_shape(g)) {
        if (!workspace) return crb_sgemm_nta(dY, X, dW, g->OC, g->IC, g->IH * g->IW, g->N, stream);
        ScratchScope scope(workspace, workspace_bytes);  // the GEMM's split scratch comes from the caller's block
        return crb_sgemm_nta(dY, X, dW, g->OC, g->IC, g->IH * g->IW, g->N, stream);
    }
    if (tiny2x2_shape(g) && aligned16(dY) && aligned16(X)) {
        const size_t need = size_t(g->OC) * g->IC * 16 * sizeof(float);
        float *G = static_cast<float *>(workspace);
        if (G) {
            if (workspace_bytes < need || !aligned16(G))
                return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace %zu bytes < required %zu (or not 16-byte aligned)", workspace_bytes, need);
        } else if (int st = scratch_get(need, s, "crb_conv_wgrad", &G)) {
            return st;
        }
        return conv2x2_wgrad(dY, X, dW, G, g->N, g->IC, g->OC, s, "crb_conv_wgrad");
    }
    if (shortcut_shape(g)) {
        const ScWgradPlan sp = sc_wgrad_plan(g->N, g->IC, g->OC, g->OH, g->OW);
        float *part = static_cast<float *>(workspace);
        if (part) {
            if (workspace_bytes < sp.workspace_bytes)
                return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace %zu bytes < required %zu", workspace_bytes, sp.workspace_bytes);
        } else if (int st = scratch_get(sp.workspace_bytes, s, "crb_conv_wgrad", &part)) {
            return st;
        }
        return launch_sc_wgrad(dY, X, dW, part, sp, g->N, g->IC, g->OC, g->OH, g->OW, s, "crb_conv_wgrad");
    }
    if (aligned16(dY) && aligned16(X)) {
        WgradDirectPlan dp;
        int st = CRB_OK;
        if (wgrad_direct(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st)) {
            float *dws = static_cast<float *>(workspace);
            if (dp.workspace_bytes) {
                if (dws) {
                    if (workspace_bytes < dp.workspace_bytes)
                        return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace %zu bytes < required %zu", workspace_bytes,
                                    dp.workspace_bytes);
                } else if (int sg = scratch_get(dp.workspace_bytes, s, "crb_conv_wgrad", &dws)) {
                    return sg;
                }
            }
            wgrad_direct(g, true, dY, X, dW, dws, s, dp, st);
            return st;
        }
    }
    {
        // the shapes no width-specialised kernel takes (those keep their own workspace size, whatever the alignment)
        TiledWgradPlan tp;
        WgradDirectPlan dp;
        int st = CRB_OK;
        if (!wgrad_direct(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st) &&
            wgrad_tiled(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, tp, st)) {
            float *tws = static_cast<float *>(workspace);
            if (tws) {
                if (workspace_bytes < tp.workspace_bytes)
                    return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace %zu bytes < required %zu", workspace_bytes, tp.workspace_bytes);
            } else if (int sg = scratch_get(tp.workspace_bytes, s, "crb_conv_wgrad", &tws)) {
                return sg;
            }
            wgrad_tiled(g, true, dY, X, dW, tws, s, tp, st);
            return st;
        }
    }
    const WgradPlan p = wgrad_plan(g);
    const u32 OHW = g->OH * g->OW;
    SepK a{dY, g->OC, OHW, g->OC * OHW, 1, FastDiv(OHW)};
    Im2colTapRows b{make_im2col(X, g)};
    if (p.splits == 1) {
        RowMajorEpi e{dW, nullptr, p.Ncols, 0, EPI_ACCUM};
        return run_by_m(a, b, e, p.M, p.Ncols, p.K, 1, 0, p.K, s, "crb_conv_wgrad");
    }
    const size_t need = size_t(p.splits) * p.M * p.Ncols * sizeof(float);
    float *ws = static_cast<float *>(workspace);
    if (ws) {
        if (workspace_bytes < need)
            return fail(CRB_EWORKSPACE, "crb_conv_wgrad: workspace %zu bytes < required %zu", workspace_bytes, need);
    } else if (int st = scratch_get(need, s, "crb_conv_wgrad", &ws)) {
        return st;
    }
    RowMajorEpi e{ws, nullptr, p.Ncols, p.M * p.Ncols, 0u};
    if (int st = run_by_m(a, b, e, p.M, p.Ncols, p.K, p.splits, 1, p.k_per_z, s, "crb_conv_wgrad")) return st;
    return launch_splitk_reduce(ws, dW, p.M * p.Ncols, p.splits, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, "crb_conv_wgrad(reduce)");
}

int crb_conv_wgrad_noalloc(const float *dY, const float *X, float *dW, const crb_conv_geom *g, void *stream) {
    if (!dY || !X || !dW) return fail(CRB_ENULL, "crb_conv_wgrad_noalloc: null operand");
    if (int st = check_geom("crb_conv_wgrad_noalloc", g)) return st;
    const size_t need = crb_conv_wgrad_workspace_bytes(g);
    if (need > kStaticScratchBytes)
        return fail(CRB_EWORKSPACE,
                    "crb_conv_wgrad_noalloc: this geometry needs %zu bytes of scratch, the built-in buffer holds %zu; use "
                    "crb_conv_wgrad with a caller workspace", need, kStaticScratchBytes);
    void *ptr = nullptr;
    if (int st = static_scratch_ptr("crb_conv_wgrad_noalloc", &ptr)) return st;
    // every scratch request below this call is served from the built-in buffer or refused: nothing allocates
    // (no explicit workspace is passed down, so the scope is the one owner of the buffer and hands out disjoint blocks)
    ScratchScope scope(ptr, kStaticScratchBytes);
    return crb_conv_wgrad(dY, X, dW, g, nullptr, 0, stream);
}

size_t crb_conv_fwd_workspace_bytes(const crb_conv_geom *g, int operands_aligned16) {
    if (check_geom("crb_conv_fwd_workspace_bytes", g)) return 0;
    bool done = false;
    if (pointwise_shape(g) && operands_aligned16) {
        try_pointwise<false>(nullptr, nullptr, nullptr, nullptr, g->N, g->IC, g->OC, g->OH, g->OW, 0, nullptr, "", done, true);
        if (done) return 0;
    }
    if (pointwise_shape(g)) return gemm_scratch_bytes(g->OC, g->IH * g->IW, g->IC, g->N);
    if (tiny2x2_shape(g) && operands_aligned16) return gemm_scratch_bytes(g->N, g->OC * 4, g->IC * 4, 1, false);
    if (operands_aligned16 && (direct_shape(g, 1) || direct_shape(g, 2))) {
        if (g->sH == 1)
            try_direct<false, 1>(nullptr, nullptr, nullptr, nullptr, g->N, g->IC, g->OC, g->OH, g->OW, g->IH, 0, nullptr, "", done, true);
        else
            try_direct<false, 2>(nullptr, nullptr, nullptr, nullptr, g->N, g->IC, g->OC, g->OH, g->OW, g->IH, 0, nullptr, "", done, true);
        if (done) return 0;
    }
    if (((tiled_s1_shape(g, 3) || tiled_s1_shape(g, 5) || tiled_s2_shape(g)) && tiled_pays(g->N, g->IC, g->OC, g->OH, g->OW, g->FH * g->FW)))
        return 0;  // the tiled kernel
    return nchw_scratch_bytes(g->OC, g->N * g->OH * g->OW, g->IC * g->FH * g->FW);
}

size_t crb_conv_dgrad_workspace_bytes(const crb_conv_geom *g, int operands_aligned16) {
    if (check_geom("crb_conv_dgrad_workspace_bytes", g)) return 0;
    bool done = false;
    if (pointwise_shape(g) && operands_aligned16) {
        try_pointwise<true>(nullptr, nullptr, nullptr, nullptr, g->N, g->OC, g->IC, g->OH, g->OW, 0, nullptr, "", done, true);
        if (done) return 0;
    }
    if (pointwise_shape(g)) return gemm_scratch_bytes(g->IC, g->IH * g->IW, g->OC, g->N);
    if (tiny2x2_shape(g) && operands_aligned16) return gemm_scratch_bytes(g->N, g->IC * 4, g->OC * 4, 1, false);
    if (operands_aligned16 && (direct_shape(g, 1) || direct_shape(g, 2))) {
        if (g->sH == 1)
            try_direct<true, 1>(nullptr, nullptr, nullptr, nullptr, g->N, g->OC, g->IC, g->OH, g->OW, g->OH, 0, nullptr, "", done, true);
        else
            try_direct<true, 2>(nullptr, nullptr, nullptr, nullptr, g->N, g->OC, g->IC, g->OH, g->OW, g->OH, 0, nullptr, "", done, true);
        if (done) return 0;
    }
    if (shortcut_shape(g) && operands_aligned16) return 0;
    if ((tiled_s1_shape(g, 3) || tiled_s1_shape(g, 5)) && tiled_pays(g->N, g->OC, g->IC, g->IH, g->IW, g->FH * g->FW))
        return 0;  // the tiled kernel
    if (tiled_classes_pay(g)) return 0;                              // one tiled launch per residue class
    if ((g->sH > 1 || g->sW > 1) && dgrad_classes_pay(g)) return 0;  // one launch per residue class, none of them cut
    return nchw_scratch_bytes(g->IC, g->N * g->IH * g->IW, g->OC * g->FH * g->FW);
}

int crb_conv_bwd(const float *W, const float *dY, const float *X, float *dX, float *dW, const crb_conv_geom *g, void *workspace,
                 size_t workspace_bytes, void *stream) {
    if (!W || !dY || !X || !dX || !dW) return fail(CRB_ENULL, "crb_conv_bwd: null operand");
    if (int st = check_geom("crb_conv_bwd", g)) return st;
    if (workspace && !aligned16(workspace)) return fail(CRB_EWORKSPACE, "crb_conv_bwd: workspace is not 16-byte aligned");
    if (aligned16(dY) && aligned16(X) && aligned16(dX)) {
        WgradDirectPlan dp;
        int st = CRB_OK;
        if (bwd_fused(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st)) {
            float *dws = static_cast<float *>(workspace);
            if (dp.workspace_bytes) {
                if (dws) {
                    if (workspace_bytes < dp.workspace_bytes)
                        return fail(CRB_EWORKSPACE, "crb_conv_bwd: workspace %zu bytes < required %zu", workspace_bytes, dp.workspace_bytes);
                } else if (int sg = scratch_get(dp.workspace_bytes, hipStream_t(stream), "crb_conv_bwd", &dws)) {
                    return sg;
                }
            }
            bwd_fused(g, true, W, dY, X, dX, dW, dws, hipStream_t(stream), dp, st);
            return st;
        }
    }
    if (int st = crb_conv_dgrad(W, dY, dX, g, stream)) return st;
    return crb_conv_wgrad(dY, X, dW, g, workspace, workspace_bytes, stream);
}

uint32_t crb_conv_bwd_slices(const crb_conv_geom *g) {
    if (check_geom("crb_conv_bwd_slices", g)) return 0;
    WgradDirectPlan dp;
    int st = CRB_OK;
    if (pointwise_shape(g)) {  // the pixel-contraction weight gradient leaves one slice per pixel range
        if (!pw_wgrad_fits(g->IC, g->OC, g->IH * g->IW)) return 0;
        const u32 n = pw_wgrad_plan(g->N, g->IC, g->OC, g->IH * g->IW).splits;
        return n > 1 ? n : 0;
    }
    if (tiny2x2_shape(g)) return 0;
    if (shortcut_shape(g)) {
        const u32 n = sc_wgrad_plan(g->N, g->IC, g->OC, g->OH, g->OW).splits;
        return n > 1 ? n : 0;
    }
    if (!wgrad_direct(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st)) return 0;
    return dp.splits > 1 ? dp.splits : 0;
}

int crb_conv_bwd_sliced(const float *W, const float *dY, const float *X, float *dX, const crb_conv_geom *g, void *workspace,
                        size_t workspace_bytes, void *stream) {
    if (!W || !dY || !X || !dX || !workspace) return fail(CRB_ENULL, "crb_conv_bwd_sliced: null operand");
    if (int st = check_geom("crb_conv_bwd_sliced", g)) return st;
    if (!crb_conv_bwd_slices(g) || !aligned16(dY) || !aligned16(X) || !aligned16(dX) || !aligned16(workspace))
        return fail(CRB_EINVAL_SHAPE, "crb_conv_bwd_sliced: this geometry (or operand alignment) has no sliced form; use crb_conv_bwd");
    WgradDirectPlan dp;
    int st = CRB_OK;
    float *ws = static_cast<float *>(workspace);
    hipStream_t s = hipStream_t(stream);
    if (pointwise_shape(g)) {
        const PwWgradPlan pp = pw_wgrad_plan(g->N, g->IC, g->OC, g->IH * g->IW);
        if (workspace_bytes < pp.workspace_bytes)
            return fail(CRB_EWORKSPACE, "crb_conv_bwd_sliced: workspace %zu bytes < required %zu", workspace_bytes, pp.workspace_bytes);
        if (int sd = crb_conv_dgrad(W, dY, dX, g, stream)) return sd;
        return launch_pw_wgrad(dY, X, nullptr, ws, pp, g->IC, g->OC, g->IH * g->IW, s, "crb_conv_bwd_sliced");
    }
    if (shortcut_shape(g)) {
        const ScWgradPlan sp = sc_wgrad_plan(g->N, g->IC, g->OC, g->OH, g->OW);
        if (workspace_bytes < sp.workspace_bytes)
            return fail(CRB_EWORKSPACE, "crb_conv_bwd_sliced: workspace %zu bytes < required %zu", workspace_bytes, sp.workspace_bytes);
        if (int sd = crb_conv_dgrad(W, dY, dX, g, stream)) return sd;
        return launch_sc_wgrad(dY, X, nullptr, ws, sp, g->N, g->IC, g->OC, g->OH, g->OW, s, "crb_conv_bwd_sliced");
    }
    if (bwd_fused(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st)) {
        if (workspace_bytes < dp.workspace_bytes)
            return fail(CRB_EWORKSPACE, "crb_conv_bwd_sliced: workspace %zu bytes < required %zu", workspace_bytes, dp.workspace_bytes);
        bwd_fused(g, true, W, dY, X, dX, nullptr, ws, s, dp, st);
        return st;
    }
    wgrad_direct(g, false, nullptr, nullptr, nullptr, nullptr, nullptr, dp, st);
    if (workspace_bytes < dp.workspace_bytes)
        return fail(CRB_EWORKSPACE, "crb_conv_bwd_sliced: workspace %zu bytes < required %zu", workspace_bytes, dp.workspace_bytes);
    if (int sd = crb_conv_dgrad(W, dY, dX, g, stream)) return sd;
    wgrad_direct(g, true, dY, X, nullptr, ws, s, dp, st);
    return st;
}

int crb_sum_slices_multi(const crb_slice_sum_item *items, uint32_t n_items, void *stream) {
    if (!items && n_items) return fail(CRB_ENULL, "crb_sum_slices_multi: null item list");
    static_assert(sizeof(crb_slice_sum_item) == sizeof(SliceSumItem), "item layout");
    for (uint32_t i = 0; i < n_items; ++i) {
        if (!items[i].slices || !items[i].dst) return fail(CRB_ENULL, "crb_sum_slices_multi: item %u has a null pointer", i);
        if (!items[i].count || !items[i].n_slices) return fail(CRB_EINVAL_SHAPE, "crb_sum_slices_multi: item %u is empty", i);
        if (uint64_t(items[i].count) * items[i].n_slices > 0x7fffffffull)
            return fail(CRB_EINVAL_SHAPE, "crb_sum_slices_multi: item %u exceeds 2^31 elements", i);
    }
    return launch_slice_sum_multi(reinterpret_cast<const SliceSumItem *>(items), n_items, hipStream_t(stream), "crb_sum_slices_multi");
}

size_t crb_conv_bias_grad_workspace_bytes(uint32_t N, uint32_t C, uint32_t HW) {
    if (!N || !C || !HW || uint64_t(N) * C * HW > 0x7fffffffull) return 0;
    // the scalar form (operands not 16-byte friendly) has the narrower column blocks, hence the most slices
    const BiasGradPlan v = bias_grad_plan(N, C * HW, true), sc = bias_grad_plan(N, C * HW, false);
    return size_t(v.slices > sc.slices ? v.slices : sc.slices) * C * HW * sizeof(float);
}

int crb_conv_bias_grad(const float *dY, float *dB, uint32_t N, uint32_t C, uint32_t HW, void *stream) {
    if (!dY || !dB) return fail(CRB_ENULL, "crb_conv_bias_grad: null operand");
    if (!N || !C || !HW) return fail(CRB_EINVAL_SHAPE, "crb_conv_bias_grad: zero dimension");
    if (uint64_t(N) * C * HW > 0x7fffffffull)
        return fail(CRB_EINVAL_SHAPE, "crb_conv_bias_grad: tensor exceeds 2^31 elements");
    hipStream_t s = hipStream_t(stream);
    const u32 cols = C * HW;
    const bool vec = cols % 4 == 0 && aligned16(dY);
    const BiasGradPlan bp = bias_grad_plan(N, cols, vec);
    const u32 col_wgs = bp.col_wgs, slices = bp.slices, rows_per_slice = bp.rows_per_slice;
    const size_t need = size_t(slices) * cols * sizeof(float);
    float *part = nullptr;
    if (int st = scratch_get(need, s, "crb_conv_bias_grad", &part)) return st;
    if (vec)
        hipLaunchKernelGGL(bias_grad_colsum_kernel<true>, dim3(col_wgs, slices), dim3(256), 0, s, dY, part, N, cols, rows_per_slice);
    else
        hipLaunchKernelGGL(bias_grad_colsum_kernel<false>, dim3(col_wgs, slices), dim3(256), 0, s, dY, part, N, cols, rows_per_slice);
    if (int st = check_launch("crb_conv_bias_grad")) return st;
    hipLaunchKernelGGL(bias_grad_fold_kernel, dim3(C), dim3(256), 0, s, part, dB, HW, cols, slices);
    return check_launch("crb_conv_bias_grad");
}

int crb_conv_bias(float *Y, const float *bias, uint32_t N, uint32_t C, uint32_t HW, void *stream) {
    if (!Y || !bias) return fail(CRB_ENULL, "crb_conv_bias: null operand");
    if (!N || !C || !HW) return fail(CRB_EINVAL_SHAPE, "crb_conv_bias: zero dimension");
    if (uint64_t(N) * C * HW > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "crb_conv_bias: tensor exceeds 2^31 elements");
    const u32 total = N * C * HW;
    hipLaunchKernelGGL(conv_bias_kernel, dim3(ceil_div(total, 256)), dim3(256), 0, hipStream_t(stream), Y, bias, total, C,
                       FastDiv(HW));
    return check_launch("crb_conv_bias");
}

}  // extern "C"
