// Weight gradient of a 3x3 / pad 1 convolution (stride 1 or 2) for gfx950.
//
// dW[oc][ic][fh][fw] = sum over (n, y, x) of dY[n][oc][y][x] * X[n][ic][y+fh-1][x+fw-1]: for each of the 9 taps a
// (OC x IC) matrix product whose contraction index is the pixel. A workgroup owns ONE 16x16 (oc-block, ic-block)
// pair for all 9 taps and a slice of the pixel range (split z). It walks its slice tile by tile (TI images x TR
// rows), staging the 16 dY planes and the 16 X planes (with their one-row halo, zero outside the image) in
// double-buffered LDS. Inside a tile the pixels are a flat run k' = y*W + x, and tap (fh, fw) of X is the same
// run shifted by the constant fh*W + fw - 1, so every fragment read is base + immediate. The wrap-around that
// the shift causes at the left/right image border is removed by zeroing the dY value of the lanes that sit on
// column 0 (taps fw = 0) or column W-1 (taps fw = 2) — a select on one step in W/4, decided at compile time.
//
// Stride 2 (even input extents): X is staged de-interleaved into its four (row parity, column parity) planes, each the
// size of dY plus one halo row above. Input (2oh + fh - 1, 2ow + fw - 1) then lives in plane (fh != 1, fw != 1) at
// (oh - (fh == 0), ow - (fw == 0)): again a constant shift of the flat dY run, so the inner loop is unchanged. Only
// the fw = 0 taps can wrap (at ow = 0) and need the select.
//
// v_mfma_f32_16x16x4_f32 mapping (wave64, lane l): A = dY[oc = l%16][k' = 4s + l/16], B = X[k'][ic = l%16],
// accumulator register r = dW[oc = 4*(l/16) + r][ic = l%16]; 9 accumulator tiles (one per tap) per wave.
// The 4 waves take different rows (or images) of the tile; their accumulators are summed through LDS in fixed
// wave order at the end and written either as this split's partial result or, without splitting, added to dW.
//
// Eight-wave form (WAVES = 8): waves w and w + 4 take the SAME pixels and split the taps (0..4 and 5..8), so every SIMD
// holds two waves that fill each other's issue gaps (a lone wave keeps the matrix pipe about two thirds busy) while each
// accumulator still sees exactly the MFMA sequence of the four-wave form: results are bit-identical.
#pragma once
#include <type_traits>

#include "igemm_engine.h"

namespace crb {

// W_: dY width; TR_: dY rows per image per tile; TI_: images per tile (more than 4: whole small images, TI/4 per wave);
// S_: stride; WAVES_: 4, or 8 (two waves per pixel group, each with half of the taps).
template <int W_, int TR_, int TI_, int OCC_, int S_ = 1, int WAVES_ = 4>
struct WgradCfg {
    static constexpr int W = W_, TR = TR_, TI = TI_, OCC = OCC_, S = S_;
    static constexpr int WAVES = WAVES_, NT = 64 * WAVES_;  // threads per workgroup
    static_assert(WAVES == 4 || WAVES == 8, "waves per workgroup");
    static constexpr bool SPLIT = WAVES == 8;  // a wave multiplies half of the taps
    static constexpr int TAP_SPLIT = 5;  // eight-wave form: waves 0..3 take taps 0..4, waves 4..7 taps 5..8
    static constexpr int WPI = TI >= 4 ? 1 : 4 / TI;  // waves per image of the tile
    static constexpr int IPW = TI >= 4 ? TI / 4 : 1;  // images per wave (small images: TR is the whole image height)
    static constexpr int RW = TR / WPI;        // rows per wave (per image)
    static constexpr int KW = IPW * RW * W;    // pixels per wave per tile
    static constexpr int NSTEP = KW / 4;       // MFMA steps per wave per tile
    static constexpr int YIMG = TR * W;        // dY floats per image per plane
    static constexpr int PL = (TR + 1) * W;    // stride 2: one parity plane (halo row above + TR rows)
    static constexpr int XIMG = S == 1 ? (TR + 2) * W : 4 * PL;  // X floats per image per channel (halo rows included)
    static constexpr int XROWS = S == 1 ? TR + 2 : 2 * (TR + 1);  // input rows staged per image
    static constexpr int XRW = S * W;                             // input row width
    // plane strides == 2 mod 4 (and even): 16 planes x 2 lane groups of a half-wave land on 32 distinct banks
    static constexpr int YP = TI * YIMG + 2;
    static constexpr int XP = TI * XIMG + 8 + 2;  // 4 leading + 4 trailing pad floats (kept zero)
    static constexpr int Y_SIZE = 16 * YP, X_SIZE = 16 * XP;
    static constexpr int BUF = Y_SIZE + X_SIZE;      // one staging buffer (floats)
    static constexpr int RED_SIZE = 4 * 9 * 256 + 2304;  // cross-wave reduction scratch (floats), reuses the staging space
    static constexpr int SMEM = 2 * BUF > RED_SIZE ? 2 * BUF : RED_SIZE;
    static_assert(TI == 1 || TI == 2 || TI == 4 || TI == 8 || TI == 16, "images per tile");
    static_assert(IPW == 1 || S == 1, "several images per wave: stride 1 only");
    // X offset of MFMA step s of a wave's pixel run: the dY run is flat across the wave's images, the X planes of
    // consecutive images are XIMG apart (they carry halo rows)
    static constexpr int x_off(int s) { return IPW == 1 ? 4 * s : (4 * s / YIMG) * XIMG + (4 * s) % YIMG; }
    static_assert(TR % WPI == 0 && KW % 4 == 0, "rows must split evenly over the waves");
    static_assert(S == 1 || S == 2, "stride");
    // LDS offset of tap (fh, fw) relative to the lane's X base (which already carries the 4 leading pad floats)
    static constexpr int tap_off(int tap) {
        const int fh = tap / 3, fw = tap % 3;
        if (S == 1) return fh * W + fw - 1;
        return ((fh != 1 ? 2 : 0) + (fw != 1 ? 1 : 0)) * PL + (fh == 0 ? 0 : 1) * W + (fw == 0 ? -1 : 0);
    }
};

struct WgradArgs {
    const float *dY;  // N x OC x H x W
    const float *X;   // N x IC x (S*H) x (S*W)
    float *out;       // splits > 1: partials [z][OC][IC][9]; splits == 1: dW (accumulated)
    u32 OC, IC, H;
    u32 ic_blocks;        // ceil(IC / 16)
    u32 tiles, tiles_per_z;  // tile count (N/TI * H/TR) and tiles per split
    u32 tiles_per_img;    // H / TR
    u32 pairs, splits;
    u32 accumulate;       // add to `out` instead of overwriting (splits == 1)
};

// The work of workgroup `bid` of the grid launch_wgrad_direct sizes; `smem` = Cfg::SMEM floats of LDS, 16-byte aligned
// (buffer b: dY planes at b*BUF, X planes after them). A device function so that a kernel can run it next to another
// kind of work in one launch.
template <class Cfg>
__device__ __forceinline__ void wgrad3x3_body(const WgradArgs &a, const u32 bid, float *smem) {
    constexpr int W = Cfg::W, TR = Cfg::TR, TI = Cfg::TI, YP = Cfg::YP, XP = Cfg::XP, NSTEP = Cfg::NSTEP;
    constexpr int YIMG = Cfg::YIMG, XIMG = Cfg::XIMG;

    constexpr int NT = Cfg::NT;
    const u32 t = threadIdx.x;
    // The workgroups of one split z read the same tiles (different channel blocks). With ids 8 apart they run on the
    // same XCD and share the tiles through its L2 (workgroups are dealt round-robin to the 8 XCDs).
    // Only done when there are at least 8 splits; with fewer, ids map plainly so every XCD still gets work.
    u32 pair, z;
    if (a.splits >= kXcds) {
        const u32 xcd = bid % kXcds, slot = bid / kXcds;
        pair = slot % a.pairs, z = (slot / a.pairs) * kXcds + xcd;
        if (z >= a.splits) return;
    } else {
        pair = bid % a.pairs, z = bid / a.pairs;
    }
    const u32 ob = pair / a.ic_blocks, ib = pair % a.ic_blocks;
    const u32 HW = a.H * W;                            // dY plane
    const u32 in_H = a.H * Cfg::S, in_HW = in_H * Cfg::XRW;  // X plane
    const u32 t_begin = z * a.tiles_per_z;
    const u32 t_end = t_begin + a.tiles_per_z < a.tiles ? t_begin + a.tiles_per_z : a.tiles;

    // ---- staging: 16-byte global loads, 8-byte LDS stores (plane strides are even, not multiples of 4) ------
    // A thread owns one (image, channel, quad-of-a-row) column of the tile for the whole kernel and walks down its rows,
    // so per tile and item the address arithmetic is one add of a compile-time multiple of the row pitch.
    constexpr int YRQ = W / 4, XRQ = Cfg::XRW / 4;      // quads per dY row / per input row
    constexpr int YC = TI * 16 * YRQ, XC = TI * 16 * XRQ;  // columns
    static_assert(NT % YC == 0 && NT % XC == 0, "columns must divide the workgroup");
    constexpr int YRPP = NT / YC, XRPP = NT / XC;  // rows covered per pass
    constexpr int YNP = (TR + YRPP - 1) / YRPP, XNP = (Cfg::XROWS + XRPP - 1) / XRPP;
    v4f yreg[YNP], xreg[XNP];

    const u32 ycol = t % YC, yrp = t / YC;
    const u32 yq = ycol % YRQ, yc = (ycol / YRQ) % 16, yimg = ycol / (YRQ * 16);
    const bool ychan_ok = ob * 16 + yc < a.OC;  // channels past the tensor's extent are staged as zeros
    const float *ysrc = a.dY + (size_t(yimg) * a.OC + ob * 16 + yc) * HW + yrp * W + 4 * yq;
    const u32 ylds = yc * YP + yimg * YIMG + yrp * W + 4 * yq;

    const u32 xcol = t % XC, xrp = t / XC;
    const u32 xq = xcol % XRQ, xc = (xcol / XRQ) % 16, ximg = xcol / (XRQ * 16);
    const bool xchan_ok = ib * 16 + xc < a.IC;
    const float *xsrc = a.X + (size_t(ximg) * a.IC + ib * 16 + xc) * in_HW + 4 * xq;
    const u32 xlds = xc * XP + 4 + ximg * XIMG + (Cfg::S == 1 ? 4 * xq : 2 * xq);

    auto fetch = [&](u32 tile, v4f *yr, v4f *xr) {
        const u32 n0 = (tile / a.tiles_per_img) * TI;
        const int r0 = int(tile % a.tiles_per_img) * TR;
        const float *yp = ysrc + size_t(n0) * a.OC * HW + u32(r0) * W;
#pragma unroll
        for (int i = 0; i < YNP; ++i) {
            v4f v = {0.f, 0.f, 0.f, 0.f};
            if (ychan_ok && (TR % YRPP == 0 || i * YRPP + int(yrp) < TR)) v = *reinterpret_cast<const v4f *>(yp + i * YRPP * W);
            yr[i] = v;
        }
        // first staged input row: r0 - 1 (stride 1), 2*(r0 - 1) (stride 2: both parities of the halo row pair)
        const int row0 = (Cfg::S == 1 ? r0 - 1 : 2 * (r0 - 1)) + int(xrp);
        const float *xp = xsrc + size_t(n0) * a.IC * in_HW;
#pragma unroll
        for (int i = 0; i < XNP; ++i) {
            v4f v = {0.f, 0.f, 0.f, 0.f};
            const int row = row0 + i * XRPP;
            if (xchan_ok && (Cfg::XROWS % XRPP == 0 || i * XRPP + int(xrp) < Cfg::XROWS) && row >= 0 && row < int(in_H))
                v = *reinterpret_cast<const v4f *>(xp + row * Cfg::XRW);
            xr[i] = v;
        }
    };

    // LDS store of staged item i (dY items first, then X items)
    auto commit_item = [&](int i, const v4f *yr, const v4f *xr, float *dYs, float *dXs) {
        if (i < YNP) {
            if (TR % YRPP == 0 || i * YRPP + int(yrp) < TR) {
                float *p = dYs + ylds + i * YRPP * W;
                *reinterpret_cast<v2f *>(p) = v2f{yr[i].x, yr[i].y};
                *reinterpret_cast<v2f *>(p + 2) = v2f{yr[i].z, yr[i].w};
            }
        } else {
            const int ix = i - YNP;
            if (Cfg::XROWS % XRPP == 0 || ix * XRPP + int(xrp) < Cfg::XROWS) {
                if constexpr (Cfg::S == 1) {
                    float *p = dXs + xlds + (ix * XRPP + xrp) * W;
                    *reinterpret_cast<v2f *>(p) = v2f{xr[ix].x, xr[ix].y};
                    *reinterpret_cast<v2f *>(p + 2) = v2f{xr[ix].z, xr[ix].w};
                } else {
                    // de-interleave: staged row j has row parity j % 2 and plane row j / 2; the quad's even columns go
                    // to the column-parity-0 plane, its odd columns to the column-parity-1 plane
                    const u32 j = ix * XRPP + xrp;
                    float *p = dXs + xlds + (j & 1) * 2 * Cfg::PL + (j >> 1) * W;
                    *reinterpret_cast<v2f *>(p) = v2f{xr[ix].x, xr[ix].z};
                    *reinterpret_cast<v2f *>(p + Cfg::PL) = v2f{xr[ix].y, xr[ix].w};
                }
            }
        }
    };
    constexpr int NITEM = YNP + XNP;

    // leading / trailing pad floats of every X plane stay zero (they are read, multiplied by a zeroed dY value)
    for (u32 e = t; e < 2u * 16 * 8; e += NT) {
        float *plane = smem + (e / 128) * Cfg::BUF + Cfg::Y_SIZE + ((e % 128) / 8) * XP;
        const u32 k = e % 8;
        plane[k < 4 ? k : 4 + TI * XIMG + (k - 4)] = 0.f;
    }

    // ---- per-lane fragment addressing ---------------------------------------------------------------------
    const int lane = t & 63, wave = (t >> 6) & 3;  // wave: the pixel group (eight-wave form: shared by waves w and w + 4)
    const int tap_half = t >> 8;                   // eight-wave form: which part of the taps this wave multiplies
    const int li = lane & 15, kq = lane >> 4;
    const int img_w = (wave / Cfg::WPI) * Cfg::IPW, row_w = (wave % Cfg::WPI) * Cfg::RW;
    const int ybase = li * YP + kq + img_w * YIMG + row_w * W;
    const int xbase = li * XP + kq + 4 + img_w * XIMG + row_w * W;  // +4: leading pad floats

    v4f acc[9];
#pragma unroll
    for (int k = 0; k < 9; ++k) acc[k] = v4f{0.f, 0.f, 0.f, 0.f};

    // One tile: NSTEP MFMA steps. The LDS stores of the next tile's staged data (its global loads were issued before
    // this call) are spread over the last steps, one item per step, so they issue in the shadow of the MFMAs instead
    // of forming a store burst between tiles.
    constexpr int FIRST_STORE_STEP = NSTEP > NITEM ? NSTEP - NITEM : 0;
    // T0, T1 (integral constants): the taps [T0, T1) this wave multiplies.
    auto compute = [&](auto T0c, auto T1c, const float *cy, const float *cx, float *ny, float *nx) {
        constexpr int T0 = decltype(T0c)::value, T1 = decltype(T1c)::value;
        const float *py = cy + ybase, *px = cx + xbase;
        float av[2], bv[2][9];
        auto read_step = [&](int s, int slot) {
            av[slot] = py[4 * s];
#pragma unroll
            for (int k = T0; k < T1; ++k) bv[slot][k] = px[Cfg::x_off(s) + Cfg::tap_off(k)];
        };
        read_step(0, 0);
#pragma unroll
        for (int s = 0; s < NSTEP; ++s) {
            if (s + 1 < NSTEP) read_step(s + 1, (s + 1) & 1);
            const float am = av[s & 1];
            // lanes on dY column 0 contribute nothing to the fw = 0 taps; at stride 1 lanes on column W-1 nothing to fw = 2
            const float a0 = ((4 * s) % W == 0) ? (kq == 0 ? 0.f : am) : am;
            const float a2 = (Cfg::S == 1 && (4 * s + 4) % W == 0) ? (kq == 3 ? 0.f : am) : am;
#pragma unroll
            for (int k = T0; k < T1; ++k)
                acc[k] = __builtin_amdgcn_mfma_f32_16x16x4f32(k % 3 == 0 ? a0 : (k % 3 == 2 ? a2 : am), bv[s & 1][k], acc[k], 0, 0, 0);
            if (s >= FIRST_STORE_STEP) {
                // items per step: all remaining ones on the last step if there are more items than steps
                const int first = s - FIRST_STORE_STEP, last = (s == NSTEP - 1) ? NITEM : first + 1;
#pragma unroll
                for (int i = first; i < last; ++i) commit_item(i, yreg, xreg, ny, nx);
            }
            // issue order inside the step: one MFMA, then one of the next step's LDS reads, and so on, so the matrix
            // pipe never waits for the read burst; the fence keeps the steps themselves in order
#pragma unroll
            for (int k = T0; k < T1; ++k) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // MFMA
                __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // DS read
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // the tap range of this wave
    auto compute_taps = [&](const float *cy, const float *cx, float *ny, float *nx) {
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, 9> I9;
        typedef std::integral_constant<int, Cfg::TAP_SPLIT> IS;
        if constexpr (!Cfg::SPLIT) {
            compute(I0(), I9(), cy, cx, ny, nx);
        } else if (tap_half == 0) {
            compute(I0(), IS(), cy, cx, ny, nx);
        } else {
            compute(IS(), I9(), cy, cx, ny, nx);
        }
    };

    // ---- main loop over this split's tiles (double-buffered) ------------------------------------------------
    fetch(t_begin, yreg, xreg);
#pragma unroll
    for (int i = 0; i < NITEM; ++i) commit_item(i, yreg, xreg, smem, smem + Cfg::Y_SIZE);
    __syncthreads();
    for (u32 tile = t_begin; tile < t_end; ++tile) {
        const u32 b = (tile - t_begin) & 1;
        // After the last tile nothing new was fetched: the stores inside compute() then rewrite stale registers into
        // the idle buffer, which nothing reads before the reduction scratch overwrites it.
        if (tile + 1 < t_end) fetch(tile + 1, yreg, xreg);
        float *cur = smem + b * Cfg::BUF, *nxt = smem + (b ^ 1) * Cfg::BUF;
        compute_taps(cur, cur + Cfg::Y_SIZE, nxt, nxt + Cfg::Y_SIZE);
        __syncthreads();
    }

    // ---- sum the 4 waves' accumulators in wave order, write this (pair, split) block --------------------------
    // Pass 1: every wave parks its 9 tiles in LDS as [wave][tap][lane][4]. Pass 2: thread t sums the 4 waves for
    // element (lane = t/4, r = t%4) of each tap (consecutive threads read consecutive floats: no bank conflicts) and
    // writes the sums back transposed to [oc][ic][tap], the order dW has in memory. Pass 3: coalesced store.
    float *red = smem;                 // [wave][tap][lane][4]  (4*9*256 floats)
    float *tr = smem + 4 * 9 * 256;    // [oc 16][ic 16][tap 9] (2304 floats)
    // (eight-wave form: every wave parks the taps it holds; the threads of the upper half sum the upper taps)
#pragma unroll
    for (int k = 0; k < 9; ++k)
        if (!Cfg::SPLIT || (k < Cfg::TAP_SPLIT) == (tap_half == 0))
            *reinterpret_cast<v4f *>(red + ((wave * 9 + k) * 64 + lane) * 4) = acc[k];
    __syncthreads();
    const size_t count = size_t(a.OC) * a.IC * 9;
    float *out = a.out + size_t(z) * count * (a.accumulate ? 0 : 1);
    {
        const u32 tq = t & 255;
        const u32 l2 = tq >> 2, r = tq & 3;
        const u32 oc = 4 * (l2 >> 4) + r, ic = l2 & 15;
#pragma unroll
        for (int k = 0; k < 9; ++k) {
            if (Cfg::SPLIT && (k < Cfg::TAP_SPLIT) != (tap_half == 0)) continue;
            float sum = red[k * 256 + tq];
#pragma unroll
            for (int w = 1; w < 4; ++w) sum += red[(w * 9 + k) * 256 + tq];
            tr[(oc * 16 + ic) * 9 + k] = sum;
        }
    }
    __syncthreads();
    // whole channel blocks: an output channel's 144 floats are contiguous and 16-byte aligned in dW, so lanes store quads
    if (!a.accumulate && a.OC % 16 == 0 && a.IC % 16 == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0) {
#pragma unroll
        for (int i = 0; i < (576 + NT - 1) / NT; ++i) {
            const u32 q = t + i * NT;  // quad q = oc*36 + j
            if (576 % NT != 0 && q >= 576u) continue;
            const u32 oc = q / 36, j = q % 36;
            *reinterpret_cast<v4f *>(out + (size_t(ob * 16 + oc) * a.IC + ib * 16) * 9 + 4 * j) = *reinterpret_cast<const v4f *>(tr + 4 * q);
        }
        return;
    }
    // (dW's old values are requested together and the stores follow: a read in front of every store would make each store wait
    // for the one before it)
    constexpr int NE = (2304 + NT - 1) / NT;
    float *dst[NE];
    float old[NE];
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const u32 e = t + i * NT;                // e = oc*144 + ic*9 + tap
        const u32 oc = e / 144, rest = e % 144;  // rest = ic*9 + tap: contiguous in dW for one oc
        const bool ok = (2304 % NT == 0 || e < 2304u) && ob * 16 + oc < a.OC && ib * 16 + rest / 9 < a.IC;
        dst[i] = ok ? out + (size_t(ob * 16 + oc) * a.IC + ib * 16) * 9 + rest : nullptr;
        old[i] = 0.f;
    }
    if (a.accumulate) {
#pragma unroll
        for (int i = 0; i < NE; ++i)
            if (dst[i]) old[i] = *dst[i];
#pragma unroll
        for (int i = 0; i < NE; ++i) asm volatile("" : "+v"(old[i]));
    }
#pragma unroll
    for (int i = 0; i < NE; ++i) {
        const u32 e = t + i * NT;
        if (dst[i]) *dst[i] = old[i] + tr[(2304 % NT == 0 || e < 2304u) ? e : 0];
    }
}

template <class Cfg>
__global__ void __launch_bounds__(Cfg::NT, Cfg::OCC) wgrad3x3_kernel(WgradArgs a) {
    __shared__ __attribute__((aligned(16))) float smem[Cfg::SMEM];
    wgrad3x3_body<Cfg>(a, blockIdx.x, smem);
}

struct WgradDirectPlan {
    u32 pairs, tiles, splits, tiles_per_z;
    size_t workspace_bytes;
};

template <class Cfg>
inline bool wgrad_direct_fits(u32 N, u32 IC, u32 OC, u32 H, u32 Wd) {
    (void)IC, (void)OC;  // ragged channel blocks are zero-filled
    if (Cfg::IPW > 1 && H != u32(Cfg::TR)) return false;  // a wave's pixel run must cover whole images
    return Wd == u32(Cfg::W) && H % Cfg::TR == 0 && N % Cfg::TI == 0;
}

template <class Cfg>
inline WgradDirectPlan wgrad_direct_plan(u32 N, u32 IC, u32 OC, u32 H, u32 target_wgs) {
    WgradDirectPlan p;
    p.pairs = ceil_div(OC, 16u) * ceil_div(IC, 16u);
    p.tiles = (N / Cfg::TI) * (H / Cfg::TR);
    // Wide layers (16 or more channel-block pairs) with at least four tiles per slice left: twice the workgroups, so that
    // every SIMD holds two waves (a lone wave issues its MFMAs a third slower and has nobody to hide its loads behind).
    if (p.pairs >= 16 && uint64_t(p.tiles) * p.pairs >= uint64_t(8) * target_wgs) target_wgs *= 2;
    u32 splits = p.pairs >= target_wgs ? 1 : target_wgs / p.pairs;
    if (splits > p.tiles) splits = p.tiles;
    p.tiles_per_z = ceil_div(p.tiles, splits);
    p.splits = ceil_div(p.tiles, p.tiles_per_z);
    p.workspace_bytes = p.splits > 1 ? size_t(p.splits) * OC * IC * 9 * sizeof(float) : 0;
    return p;
}

// Kernel arguments and grid size of one configuration for one call.
template <class Cfg>
inline uint64_t wgrad_direct_args(WgradArgs &a, const float *dY, const float *X, float *dW, float *ws, const WgradDirectPlan &p, u32 IC,
                                  u32 OC, u32 H) {
    a.dY = dY, a.X = X;
    a.out = p.splits > 1 ? ws : dW;
    a.OC = OC, a.IC = IC, a.H = H;
    a.ic_blocks = ceil_div(IC, 16u);
    a.tiles = p.tiles, a.tiles_per_z = p.tiles_per_z;
    a.tiles_per_img = H / Cfg::TR;
    a.accumulate = p.splits > 1 ? 0u : 1u;
    a.pairs = p.pairs, a.splits = p.splits;
    return p.splits >= kXcds ? uint64_t(ceil_div(p.splits, kXcds)) * kXcds * p.pairs  // whole XCD rounds
                             : uint64_t(p.splits) * p.pairs;
}

template <class Cfg>
inline int launch_wgrad_direct(const float *dY, const float *X, float *dW, float *ws, const WgradDirectPlan &p, u32 N, u32 IC,
                               u32 OC, u32 H, hipStream_t s, const char *what) {
    (void)N;
    WgradArgs a;
    const uint64_t wgs = wgrad_direct_args<Cfg>(a, dY, X, dW, ws, p, IC, OC, H);
    if (wgs > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL((wgrad3x3_kernel<Cfg>), dim3(u32(wgs)), dim3(Cfg::NT), 0, s, a);
    if (int st = check_launch(what)) return st;
    if (p.splits > 1 && dW) {  // dW == nullptr: the caller sums the slices later
        return launch_splitk_reduce(ws, dW, OC * IC * 9, p.splits, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, what);
    }
    return CRB_OK;
}

}  // namespace crb
