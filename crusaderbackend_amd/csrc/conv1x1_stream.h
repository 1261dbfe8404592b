// 1x1 / stride 1 convolution (forward and data gradient) for gfx950 with the activations streamed from global memory
// straight into MFMA operands: no LDS round trip and no workgroup barrier in the main loop. These layers (the bottlenecks
// of densely connected networks) read and write tens of megabytes per call for a few hundred MFLOP per megabyte; what a
// staged kernel spends on LDS stores, barriers and the wait for each chunk costs more there than the MFMAs themselves.
//
// v_mfma_f32_16x16x4_f32 (wave64, lane l): A[i = l%16][k = l/16], B[k = l/16][j = l%16], accumulator register r =
// D[i = 4*(l/16) + r][j = l%16]. Here i = output channel, k = contraction channel, j = pixel. A lane loads PV consecutive
// pixels of channel k (PV = 4: 16 bytes, 16 lanes cover a 256-byte run) and uses component b of that vector in MFMA b, whose
// 16 columns are therefore the pixels p0 + PV*j + b: the PV accumulators of a lane hold PV consecutive pixels of one
// output channel again, stored as one vector. The small operand (the filter matrix) sits in LDS, staged once per workgroup.
// A wave owns a run of 16*PV pixels of one image; the summation order per output is the channel order: bit-reproducible.
#pragma once
#include <type_traits>

#include "igemm_engine.h"

namespace crb {

struct PwStreamArgs {
    const float *Wt;    // filters OC x IC of the forward convolution
    const float *X;     // forward: X (N x IC x HW); data gradient: dY (N x OC x HW)
    float *Y;           // forward: Y (N x OC x HW); data gradient: dX (N x IC x HW)
    const float *bias;  // forward only: per output channel or nullptr
    u32 IC, OC, HW;
    u32 tasks;          // N * HW / (16 * PV) pixel runs
    u32 relu;
};

template <int PV>
struct PixVec;
template <>
struct PixVec<4> {
    typedef v4f T;
};
template <>
struct PixVec<2> {
    typedef v2f T;
};
template <int PV>
__device__ __forceinline__ float pv_get(const typename PixVec<PV>::T &v, int b) {
    return v[b];
}
template <int PV>
__device__ __forceinline__ void pv_store(float *p, const float *v) {  // streaming store of PV consecutive floats
    if constexpr (PV == 4)
        __builtin_nontemporal_store(v4f{v[0], v[1], v[2], v[3]}, reinterpret_cast<v4f *>(p));
    else
        __builtin_nontemporal_store(v2f{v[0], v[1]}, reinterpret_cast<v2f *>(p));
}

// ---- forward: Y[oc][p] = sum_ic W[oc][ic] X[ic][p] (+ bias, ReLU); all OC <= 16 * NOB output channels per wave ----------
constexpr int kPwsDepth = 8;  // channel steps (4 channels each) in flight per wave
constexpr int kPwsThreads = 512;  // eight waves: the filter matrix is staged once for eight pixel runs

// Staging of the filter matrix W (OC x IC, rows contiguous) for contraction/input channels [c0, c0 + kc), kc <= 256:
// thread t owns column t % 256 and the rows t / 256, t / 256 + 2, ... of the ROWS staged ones; all of a thread's loads are
// in flight together (one memory round trip), and there is no division in the address arithmetic.
// dst[at(column, row)]; rows or columns past the tensor's extent are staged as zeros.
template <int ROWS, class At>
__device__ __forceinline__ void pws_stage(float *dst, const float *W, u32 OC, u32 IC, u32 c0, u32 kc, u32 cols, At at) {
    static_assert(kPwsThreads == 512 && ROWS % 2 == 0, "two row phases of 256 columns");
    const u32 col = threadIdx.x & 255u, r0 = threadIdx.x >> 8;
    if (col >= cols) return;
    // every load is issued (clamped to a valid element) and the value dropped afterwards: a branch around a load would
    // put a wait for the previous one in front of it
    float v[ROWS / 2];
    const u32 ccol = col < kc ? col : kc - 1;
#pragma unroll
    for (int i = 0; i < ROWS / 2; ++i) {
        const u32 row = r0 + 2 * i;
        v[i] = W[size_t(row < OC ? row : OC - 1) * IC + c0 + ccol];
    }
#pragma unroll
    for (int i = 0; i < ROWS / 2; ++i) dst[at(col, r0 + 2 * i)] = (col < kc && r0 + 2 * i < OC) ? v[i] : 0.f;
}

// The same staging to dst[column * col_stride + row * row_stride].
template <int ROWS>
__device__ __forceinline__ void pws_stage(float *dst, const float *W, u32 OC, u32 IC, u32 c0, u32 kc, u32 cols, u32 row_stride, u32 col_stride) {
    static_assert(kPwsThreads == 512 && ROWS % 2 == 0, "two row phases of 256 columns");
    const u32 col = threadIdx.x & 255u, r0 = threadIdx.x >> 8;
    if (col >= cols) return;
    float v[ROWS / 2];
    const u32 ccol = col < kc ? col : kc - 1;
#pragma unroll
    for (int i = 0; i < ROWS / 2; ++i) {
        const u32 row = r0 + 2 * i;
        v[i] = W[size_t(row < OC ? row : OC - 1) * IC + c0 + ccol];
    }
#pragma unroll
    for (int i = 0; i < ROWS / 2; ++i) dst[col * col_stride + (r0 + 2 * i) * row_stride] = (col < kc && r0 + 2 * i < OC) ? v[i] : 0.f;
}

template <int NOB>
struct PwsFwdLds {
    static constexpr int KC = NOB <= 3 ? 256 : 192;                              // contraction channels staged per pass
    // Ws holds one row of NOB * 16 output channels per contraction channel; channel c sits at (c / 2) * PS + (c % 2) * S1.
    // S1 == 16 mod 32: a fragment read's two lane groups of a half-wave (channels 4s and 4s + 1, or 4s + 2 and 4s + 3,
    // sixteen consecutive output channels each) cover all 32 banks once. PS odd: the staging stores (consecutive lanes on
    // consecutive channels) of a half-wave are sixteen channel pairs whose starts p * PS are distinct mod 32 and never
    // 16 apart, so they cover all 32 banks once as well.
    static constexpr int S1 = NOB <= 1 ? 16 : (NOB <= 3 ? 48 : 80);
    static constexpr int PS = 2 * S1 + 1;
    static constexpr int FLOATS = (KC / 2 + 2) * PS;  // one channel step past the staged rows may be read (never used)
    static __device__ __forceinline__ u32 at(u32 c) { return (c >> 1) * u32(PS) + (c & 1u) * u32(S1); }
};

template <int NOB, int PV>
__global__ void __launch_bounds__(kPwsThreads, 1) pw_fwd_stream_kernel(PwStreamArgs a) {
    typedef typename PixVec<PV>::T XV;
    typedef PwsFwdLds<NOB> LdsW;
    constexpr int KC = LdsW::KC, D = kPwsDepth;
    __shared__ __attribute__((aligned(16))) float Ws[LdsW::FLOATS];  // Ws[ic][oc], see PwsFwdLds
    const u32 t = threadIdx.x, lane = t & 63, wave = t >> 6, j = lane & 15, k = lane >> 4;
    const u32 task = blockIdx.x * (kPwsThreads / 64) + wave;
    const bool on = task < a.tasks;  // idle waves still help staging and meet the barriers
    const u32 pix = (on ? task : 0) * (16 * PV);
    const u32 n = pix / a.HW, p0 = pix % a.HW;
    const float *xrun = a.X + size_t(n) * a.IC * a.HW + p0 + PV * j;  // + channel * HW

    v4f acc[NOB][PV];
#pragma unroll
    for (int o = 0; o < NOB; ++o)
#pragma unroll
        for (int b = 0; b < PV; ++b) acc[o][b] = v4f{0.f, 0.f, 0.f, 0.f};
    // the bias values of this lane's output channels, requested now: a load in the epilogue would wait, through the
    // in-order memory counter, for every store issued before it
    float bias_v[NOB][4];
#pragma unroll
    for (int o = 0; o < NOB; ++o)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const u32 oc = o * 16 + 4 * k + r;
            bias_v[o][r] = (a.bias && oc < a.OC) ? a.bias[oc] : 0.f;
        }

    // Channel step s of a pass that starts at channel c0: this lane's channel is c0 + 4 s + k; past the tensor's extent it
    // reads the last channel and is zeroed at use (its filter values are zero, but 0 * inf is not). Past the pass it reads
    // one dummy line, so that every iteration issues the same loads and the wait in front of a use covers exactly the
    // loads issued before it.
    XV xq[D];
    auto issue_at = [&](u32 c0, u32 steps, u32 s, int slot) {
        const u32 ch = c0 + 4 * s + k;
        const float *p = s < steps ? xrun + size_t(ch < a.IC ? ch : a.IC - 1) * a.HW : a.X;
        xq[slot] = *reinterpret_cast<const XV *>(p);
    };
    // (Requesting the first pass's activations before the filters are staged was measured and is not done: the staging's
    // own loads then queue behind them, 204 -> 48 @ 32x32 at batch 64 took 17.6 instead of 15.3 us.)

    for (u32 c0 = 0; c0 < a.IC; c0 += KC) {
        const u32 kc = a.IC - c0 < u32(KC) ? a.IC - c0 : u32(KC);
        const u32 steps = (kc + 3) / 4, kc4 = steps * 4;
        if (c0) __syncthreads();  // every wave is done with the previous pass's filters
        // consecutive threads take consecutive contraction channels of one filter row (contiguous in memory)
        pws_stage<NOB * 16>(Ws, a.Wt, a.OC, a.IC, c0, kc, kc4, [](u32 col, u32 row) { return LdsW::at(col) + row; });
        __syncthreads();
        if (!on) continue;

        auto issue = [&](u32 s, int slot) { issue_at(c0, steps, s, slot); };
        // this lane's filter values of step s: channel 4 s + k, output channels 16 o + j
        const float *wl = Ws + (k >> 1) * LdsW::PS + (k & 1u) * LdsW::S1 + j;
        float av[2][NOB];
        auto read_a = [&](u32 s, int slot) {
#pragma unroll
            for (int o = 0; o < NOB; ++o) av[slot][o] = wl[(2 * s) * LdsW::PS + o * 16];
        };
#pragma unroll
        for (int i = 0; i < D; ++i) issue(i, i);
        read_a(0, 0);
        // One channel step. The filter values of the next step are requested first (unconditionally — past the last step
        // they come from the spare rows and are dropped — so that the wait in front of the MFMAs leaves them in flight).
        // FAST: the step and the one it requests (s + D) both lie inside the pass and the tensor: no select, and the
        // load address is the running pointer.
        const float *pnext = xrun + (size_t(c0) + 4 * D + k) * a.HW;  // channel of step D
        const size_t pstep = size_t(4) * a.HW;
        auto step = [&](u32 s, int i, auto fast) {
            constexpr bool FAST = decltype(fast)::value;
            read_a(s + 1, (i + 1) & 1);
            const bool live = FAST || c0 + 4 * s + k < a.IC;
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int b = 0; b < PV; ++b) {
                const float xv = live ? pv_get<PV>(xq[i], b) : 0.f;
#pragma unroll
                for (int o = 0; o < NOB; ++o) acc[o][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[i & 1][o], xv, acc[o][b], 0, 0, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (FAST) {
                xq[i] = *reinterpret_cast<const XV *>(pnext);
                pnext += pstep;
            } else {
                issue(s + D, i);
            }
        };
        u32 s0 = 0;
        for (; s0 + 2 * D < steps; s0 += D) {  // every step of the group and the steps it requests are in range
#pragma unroll
            for (int i = 0; i < D; ++i) step(s0 + i, i, std::true_type{});
        }
        for (; s0 < steps; s0 += D) {
#pragma unroll
            for (int i = 0; i < D; ++i)
                if (s0 + i < steps) step(s0 + i, i, std::false_type{});
        }
    }
    if (!on) return;
    // accumulator register r of MFMA b: output channel 16 o + 4 k + r, pixel p0 + PV j + b
    float *yrun = a.Y + size_t(n) * a.OC * a.HW + p0 + PV * j;
#pragma unroll
    for (int o = 0; o < NOB; ++o)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const u32 oc = o * 16 + 4 * k + r;
            if (oc >= a.OC) continue;
            const float bv = bias_v[o][r];
            float v[PV];
#pragma unroll
            for (int b = 0; b < PV; ++b) {
                v[b] = acc[o][b][r] + bv;
                if (a.relu) v[b] = v[b] > 0.f ? v[b] : 0.f;
            }
            pv_store<PV>(yrun + size_t(oc) * a.HW, v);
        }
}

// ---- data gradient: dX[ic][p] = sum_oc W[oc][ic] dY[oc][p]; contraction over OC <= 4 * NS channels ------------------------
// A wave loads its run of dY once (NS vectors per lane) and multiplies it against one block of 16 input channels after
// the other, storing each block as soon as it is complete: the stores drain behind the next block's MFMAs.
constexpr int kPwsIcp = 208;  // filter row stride in LDS (== 16 mod 32) = input channels staged per pass

template <int NS, int PV>
__global__ void __launch_bounds__(kPwsThreads, 1) pw_dgrad_stream_kernel(PwStreamArgs a) {
    typedef typename PixVec<PV>::T XV;
    constexpr int ICP = kPwsIcp;
    __shared__ __attribute__((aligned(16))) float Ws[NS * 4 * ICP];  // Ws[oc][ic - c0]
    const u32 t = threadIdx.x, lane = t & 63, wave = t >> 6, j = lane & 15, k = lane >> 4;
    const u32 task = blockIdx.x * (kPwsThreads / 64) + wave;
    const bool on = task < a.tasks;
    const u32 pix = (on ? task : 0) * (16 * PV);
    const u32 n = pix / a.HW, p0 = pix % a.HW;

    // this lane's dY values: channel 4 s + k (past the extent: the last channel, zeroed), pixels p0 + PV j ..
    XV dy[NS];
    const float *yrun = a.X + size_t(n) * a.OC * a.HW + p0 + PV * j;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        const u32 ch = 4 * s + k;
        dy[s] = *reinterpret_cast<const XV *>(yrun + size_t(ch < a.OC ? ch : a.OC - 1) * a.HW);
    }
    float *xrun = a.Y + size_t(n) * a.IC * a.HW + p0 + PV * j;
    bool dy_clean = false;

    for (u32 c0 = 0; c0 < a.IC; c0 += ICP) {
        const u32 kc = a.IC - c0 < u32(ICP) ? a.IC - c0 : u32(ICP);
        const u32 blocks = (kc + 15) / 16;
        if (c0) __syncthreads();
        pws_stage<NS * 4>(Ws, a.Wt, a.OC, a.IC, c0, kc, blocks * 16, ICP, 1);
        __syncthreads();
        if (!on) continue;
        if (!dy_clean) {  // once, after the staging (the loads have had that long to arrive)
            dy_clean = true;
#pragma unroll
            for (int s = 0; s < NS; ++s)
                if (4 * s + k >= a.OC) dy[s] = XV{};
        }
        const float *wl = Ws + k * ICP + j;
        float av[2][NS];
        auto read_a = [&](u32 ib, int slot) {
#pragma unroll
            for (int s = 0; s < NS; ++s) av[slot][s] = wl[(4 * s) * ICP + ib * 16];
        };
        read_a(0, 0);
        for (u32 ib = 0; ib < blocks; ib += 2) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                if (ib + h >= blocks) break;
                if (ib + h + 1 < blocks) read_a(ib + h + 1, (h + 1) & 1);
                v4f acc[PV];
#pragma unroll
                for (int b = 0; b < PV; ++b) acc[b] = v4f{0.f, 0.f, 0.f, 0.f};
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int s = 0; s < NS; ++s)
#pragma unroll
                    for (int b = 0; b < PV; ++b) acc[b] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[h][s], pv_get<PV>(dy[s], b), acc[b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const u32 ic = c0 + (ib + h) * 16 + 4 * k + r;
                    if (ic >= a.IC) continue;
                    float v[PV];
#pragma unroll
                    for (int b = 0; b < PV; ++b) v[b] = acc[b][r];
                    pv_store<PV>(xrun + size_t(ic) * a.HW, v);
                }
            }
        }
    }
}

// Pixels per lane for a problem: the widest vector that still yields two waves per SIMD (2048 runs), else the narrower
// one if that covers at least half the CUs; 0: not applicable (smaller problems are faster through the staged kernels).
inline int pw_stream_pv(u32 N, u32 HW) {
    const uint64_t px = uint64_t(N) * HW;
    if (HW % 64 == 0 && px / 64 >= 2048) return 4;
    if (HW % 32 == 0 && px / 32 >= 1024) return 2;
    return 0;
}

template <int PV>
inline int launch_pw_fwd_stream(const PwStreamArgs &a, hipStream_t s, const char *what) {
    const dim3 grid(ceil_div(a.tasks, u32(kPwsThreads / 64))), block(kPwsThreads);
    switch (ceil_div(a.OC, 16u)) {
        case 1: hipLaunchKernelGGL((pw_fwd_stream_kernel<1, PV>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((pw_fwd_stream_kernel<2, PV>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((pw_fwd_stream_kernel<3, PV>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((pw_fwd_stream_kernel<4, PV>), grid, block, 0, s, a); break;
    }
    return check_launch(what);
}

template <int PV>
inline int launch_pw_dgrad_stream(const PwStreamArgs &a, hipStream_t s, const char *what) {
    const dim3 grid(ceil_div(a.tasks, u32(kPwsThreads / 64))), block(kPwsThreads);
    switch (ceil_div(a.OC, 16u)) {
        case 1: hipLaunchKernelGGL((pw_dgrad_stream_kernel<4, PV>), grid, block, 0, s, a); break;
        case 2: hipLaunchKernelGGL((pw_dgrad_stream_kernel<8, PV>), grid, block, 0, s, a); break;
        case 3: hipLaunchKernelGGL((pw_dgrad_stream_kernel<12, PV>), grid, block, 0, s, a); break;
        default: hipLaunchKernelGGL((pw_dgrad_stream_kernel<16, PV>), grid, block, 0, s, a); break;
    }
    return check_launch(what);
}

// Both passes need the short side of the layer (OC) to fit one wave: at most 64 channels.
inline bool pw_stream_fits(u32 N, u32 OC, u32 HW) { return OC <= 64 && pw_stream_pv(N, HW) != 0; }

// dgrad = false: Y = W * X (+ bias, ReLU); true: dX = W^T * dY (X: dY, Y: dX).
inline int launch_pw_stream(bool dgrad, const float *Wt, const float *X, float *Y, const float *bias, u32 N, u32 IC, u32 OC, u32 HW,
                            u32 relu, hipStream_t s, const char *what) {
    const int pv = pw_stream_pv(N, HW);
    PwStreamArgs a{Wt, X, Y, bias, IC, OC, HW, u32(uint64_t(N) * HW / (16u * u32(pv))), relu};
    if (dgrad) return pv == 4 ? launch_pw_dgrad_stream<4>(a, s, what) : launch_pw_dgrad_stream<2>(a, s, what);
    return pv == 4 ? launch_pw_fwd_stream<4>(a, s, what) : launch_pw_fwd_stream<2>(a, s, what);
}

}  // namespace crb
