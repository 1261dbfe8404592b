// Generic fp32 MFMA contraction engine for gfx950:  D(M x N) = sum_k A(m,k) * B(k,n).
//
// One 256-thread workgroup (4 wave64) owns a BM x BN macro-tile. Operand panels are staged through
// double-buffered LDS one BK-wide K slab at a time (global -> registers -> LDS prefetch of slab s+1
// overlaps the MFMAs of slab s; one barrier per slab) and fed to v_mfma_f32_32x32x2_f32.
//
// Operands are functors, so the same mainloop serves plain matrices (any transposition), K-concatenated
// batches and the implicit im2col gathers of the convolution passes. Each operand declares which of
// its two indices is contiguous in memory:
//   kKFast = true  : LDS panel is [row][k] (row stride BK+4 floats). A lane reads one 16-byte vector
//                    = the k values of 4 consecutive MFMA steps.
//   kKFast = false : LDS panel is [k][row] (row stride ROWS+4 floats). MFMA block `b` of a wave owns
//                    rows {T*i + b}, so a lane reads its T blocks' values for one step as one vector.
// Either way global->LDS copies are straight (no transposition) and LDS reads are vector reads.
// Within a group of 8 k's, MFMA step s of lane-half h consumes k = 4*h + s for both operands.
//
// MFMA 32x32x2 f32 operand mapping (wave64, lane l): A value = A[i = l%32][k = l/32],
// B value = B[k = l/32][j = l%32], accumulator register r = D[8*(r/4) + 4*(l/32) + r%4][l%32].
#pragma once
#include "crb_common.h"

namespace crb {

typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr u32 kXcds = 8;

enum : u32 { EPI_ACCUM = 1u, EPI_RELU = 2u };

// Workgroup barrier that orders LDS accesses only: global loads requested before it stay in flight across it
// (__syncthreads() fences every address space and so waits for them).
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

struct IgemmDims {
    u32 M, N, K;
    u32 tiles_m, tiles_n;
    u32 k_per_z;  // K range handled per blockIdx.z when split_k != 0 (multiple of BK)
    u32 split_k;  // 0: blockIdx.z is a batch index; 1: blockIdx.z is a K-split index
};

// PF_: how many K slabs ahead of the MFMAs the global loads run (1: the next slab's loads have one slab of MFMAs to
// arrive in; 2: two register sets, two slabs in flight — for grids that leave a CU a single workgroup).
// KG_: wave groups along K. 2: eight waves; both groups own the same macro-tile and each multiplies half of every staged
// slab, so that a grid of one workgroup per CU still puts two waves on every SIMD; the second group's accumulators are
// added to the first's through LDS before the epilogue (fixed order: bit-reproducible).
template <int BM_, int BN_, int BK_, int WM_, int WN_, int OCC_, int PF_ = 1, int KG_ = 1>
struct TileCfg {
    static constexpr int BM = BM_, BN = BN_, BK = BK_, WM = WM_, WN = WN_, OCC = OCC_, PF = PF_, KG = KG_;
    static constexpr int NTH = kThreads * KG_;  // threads per workgroup
    static_assert(KG == 1 || (KG == 2 && BK_ % 16 == 0), "two wave groups split a slab into halves of whole 8-k groups");
    static_assert(PF == 1 || PF == 2, "prefetch distance");
    static constexpr int WTM = BM / WM, WTN = BN / WN;  // wave tile
    static constexpr int TM = WTM / 32, TN = WTN / 32;  // 32x32 MFMA blocks per wave tile
    static_assert(WM * WN == 4, "4 waves per workgroup");
    static_assert(TM >= 1 && TN >= 1 && TM * 32 * WM == BM && TN * 32 * WN == BN, "tile shape");
    static_assert(BK % 8 == 0, "K slab is a multiple of 8");
};

// ---- global -> register -> LDS staging of one operand panel (ROWS x BK) -----------------------------
template <class Op, int ROWS, int BK, int NTH = kThreads>
struct PanelLoader {
    static constexpr bool KF = Op::kKFast;
    static constexpr bool VEC = Op::kVec;
    static constexpr int LD = KF ? BK + 4 : ROWS + 4;
    static constexpr int SIZE = KF ? ROWS * LD : BK * LD;
    // number of register-resident items per thread per slab
    static constexpr int ITEMS = VEC ? ROWS * BK / 4 : ROWS * BK;
    static constexpr int NP = (ITEMS + NTH - 1) / NTH;
    static_assert(ITEMS % NTH == 0 || ITEMS < NTH, "panel must split evenly over 256 threads");
    // panels with fewer items than threads are staged by the first ITEMS threads only
    static __device__ __forceinline__ bool active() { return ITEMS >= NTH || threadIdx.x < ITEMS; }
    static_assert(VEC || KF || ROWS <= NTH, "row-fast scalar staging needs ROWS <= 256");

    // scalar, k-fast: thread owns k lane t%BK and rows t/BK + i*(256/BK): NP row states kept
    // scalar, row-fast: thread owns row t%ROWS and k's t/ROWS + i*(256/ROWS): one row state kept
    static constexpr int NROWSTATE = VEC ? 1 : (KF ? NP : 1);
    typename Op::RowS rs[NROWSTATE];
    float reg[VEC ? NP * 4 : NP];
    u32 row0;

    __device__ __forceinline__ void init(const Op &op, u32 row0_) {
        row0 = row0_;
        const u32 t = threadIdx.x;
        if constexpr (!VEC) {
            if constexpr (KF) {
#pragma unroll
                for (int i = 0; i < NP; ++i) rs[i] = op.prep_row(row0 + t / BK + i * (NTH / BK));
            } else {
                rs[0] = op.prep_row(row0 + t % ROWS);
            }
        }
    }

    __device__ __forceinline__ void fetch(const Op &op, u32 k0, u32 klimit) {
        const u32 t = threadIdx.x;
        if (!active()) return;
        if constexpr (VEC) {
            if constexpr (KF) {
                constexpr int QK = BK / 4, RP = NTH / QK;
#pragma unroll
                for (int i = 0; i < NP; ++i) {
                    v4f v = op.fetch4(row0 + t / QK + i * RP, k0 + 4 * (t % QK), klimit);
                    reg[4 * i + 0] = v.x, reg[4 * i + 1] = v.y, reg[4 * i + 2] = v.z, reg[4 * i + 3] = v.w;
                }
            } else {
                constexpr int QR = ROWS / 4, KP = NTH / QR;
#pragma unroll
                for (int i = 0; i < NP; ++i) {
                    v4f v = op.fetch4(row0 + 4 * (t % QR), k0 + t / QR + i * KP, klimit);
                    reg[4 * i + 0] = v.x, reg[4 * i + 1] = v.y, reg[4 * i + 2] = v.z, reg[4 * i + 3] = v.w;
                }
            }
        } else {
            if constexpr (KF) {
                typename Op::KS ks = op.prep_k(k0 + t % BK, klimit);
#pragma unroll
                for (int i = 0; i < NP; ++i) reg[i] = op.fetch(rs[i], ks);
            } else {
                constexpr int KP = NTH / ROWS;
#pragma unroll
                for (int i = 0; i < NP; ++i) {
                    typename Op::KS ks = op.prep_k(k0 + t / ROWS + i * KP, klimit);
                    reg[i] = op.fetch(rs[0], ks);
                }
            }
        }
    }

    __device__ __forceinline__ void commit(float *lds) const {
        const u32 t = threadIdx.x;
        if (!active()) return;
        if constexpr (VEC) {
            if constexpr (KF) {
                constexpr int QK = BK / 4, RP = NTH / QK;
#pragma unroll
                for (int i = 0; i < NP; ++i) {
                    v4f v = {reg[4 * i], reg[4 * i + 1], reg[4 * i + 2], reg[4 * i + 3]};
                    *reinterpret_cast<v4f *>(lds + (t / QK + i * RP) * LD + 4 * (t % QK)) = v;
                }
            } else {
                constexpr int QR = ROWS / 4, KP = NTH / QR;
#pragma unroll
                for (int i = 0; i < NP; ++i) {
                    v4f v = {reg[4 * i], reg[4 * i + 1], reg[4 * i + 2], reg[4 * i + 3]};
                    *reinterpret_cast<v4f *>(lds + (t / QR + i * KP) * LD + 4 * (t % QR)) = v;
                }
            }
        } else {
            if constexpr (KF) {
#pragma unroll
                for (int i = 0; i < NP; ++i) lds[(t / BK + i * (NTH / BK)) * LD + t % BK] = reg[i];
            } else {
                constexpr int KP = NTH / ROWS;
#pragma unroll
                for (int i = 0; i < NP; ++i) lds[(t / ROWS + i * KP) * LD + t % ROWS] = reg[i];
            }
        }
    }
};

// ---- LDS -> MFMA fragments for one group of 8 k's (4 MFMA steps) ------------------------------------
// frag[s][b]: value this lane feeds to MFMA step s for 32-row block b of the wave tile.
template <bool KF, int T, int LD>
__device__ __forceinline__ void read_frags(const float *lds, int wave_row0, int g, int lane, float (&frag)[4][T]) {
    const int i = lane & 31, h = lane >> 5;
    if constexpr (KF) {
#pragma unroll
        for (int b = 0; b < T; ++b) {
            v4f v = *reinterpret_cast<const v4f *>(lds + (wave_row0 + b * 32 + i) * LD + 8 * g + 4 * h);
            frag[0][b] = v.x, frag[1][b] = v.y, frag[2][b] = v.z, frag[3][b] = v.w;
        }
    } else {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const float *p = lds + (8 * g + 4 * h + s) * LD + wave_row0 + i * T;
            if constexpr (T == 1) {
                frag[s][0] = p[0];
            } else if constexpr (T == 2) {
                v2f v = *reinterpret_cast<const v2f *>(p);
                frag[s][0] = v.x, frag[s][1] = v.y;
            } else {
                static_assert(T % 4 == 0 || T <= 2, "row-fast wave tiles use 1, 2 or 4k blocks");
#pragma unroll
                for (int q = 0; q < T / 4; ++q) {
                    v4f v = *reinterpret_cast<const v4f *>(p + 4 * q);
                    frag[s][4 * q + 0] = v.x, frag[s][4 * q + 1] = v.y, frag[s][4 * q + 2] = v.z,
                                    frag[s][4 * q + 3] = v.w;
                }
            }
        }
    }
}

// Workgroups are dealt round-robin to the 8 XCDs (each with its own L2). Give every XCD a contiguous
// run of the tile sequence, and order that sequence in bands of 8 tile-rows walked column by column,
// so the workgroups resident on one XCD share A and B panels through that XCD's L2.
__device__ __forceinline__ void swizzled_tile(u32 bid, u32 tiles_m, u32 tiles_n, u32 &tm, u32 &tn) {
    const u32 nt = tiles_m * tiles_n;
    const u32 q = nt / kXcds, r = nt % kXcds;
    const u32 xcd = bid % kXcds, loc = bid / kXcds;
    const u32 tile = xcd * q + (xcd < r ? xcd : r) + loc;
    constexpr u32 BAND = 8;
    const u32 per_band = BAND * tiles_n;
    const u32 band = tile / per_band, in_band = tile % per_band;
    const u32 first_m = band * BAND;
    const u32 rows = tiles_m - first_m < BAND ? tiles_m - first_m : BAND;
    tm = first_m + in_band % rows;
    tn = in_band / rows;
}

template <class Cfg, class AOp, class BOp, class Epi>
__global__ void __launch_bounds__(Cfg::NTH, Cfg::OCC) igemm_kernel(AOp a, BOp b, Epi epi, IgemmDims d) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, TM = Cfg::TM, TN = Cfg::TN;
    using LA = PanelLoader<AOp, BM, BK, Cfg::NTH>;
    using LB = PanelLoader<BOp, BN, BK, Cfg::NTH>;
    __shared__ __attribute__((aligned(16))) float sA[2][LA::SIZE];
    __shared__ __attribute__((aligned(16))) float sB[2][LB::SIZE];

    u32 tm, tn;
    swizzled_tile(blockIdx.x, d.tiles_m, d.tiles_n, tm, tn);
    const u32 z = blockIdx.z;
    u32 kbeg = 0, kend = d.K;
    if (d.split_k) {
        kbeg = z * d.k_per_z;
        kend = kbeg + d.k_per_z < d.K ? kbeg + d.k_per_z : d.K;
        a.bind(0), b.bind(0);
    } else {
        a.bind(z), b.bind(z);
    }
    epi.bind(z);

    const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) & 3;  // wave: position in the macro-tile (shared by both K groups)
    const int kgroup = threadIdx.x >> 8;                               // which half of every slab this wave multiplies (KG = 2)
    const int wave_m = wave / Cfg::WN, wave_n = wave % Cfg::WN;
    const u32 row0 = tm * BM, col0 = tn * BN;

    LA la;
    LB lb;
    la.init(a, row0);
    lb.init(b, col0);

    v16f acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int ni = 0; ni < TN; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    // accumulating epilogues on interior tiles read the result's previous values a block (16 per lane, or 16 pairs) at a
    // time, all loads of a block in flight together, instead of one memory round trip per element; a one-block wave
    // tile requests them before the last slab is multiplied, so that they arrive behind its MFMAs
    constexpr bool kPair = !BOp::kKFast && TN == 2 && Epi::kPairStore;
    constexpr bool kOldEarly = Epi::kEarlyOld && TM * TN == 1;
    float oldv[Epi::kPrefetchOld ? (kPair ? 32 : 16) : 1];
    bool have_old = false, old_tried = false;
    // block (mi, ni) of the wave tile (pair form: both ni of row block mi)
    auto fetch_old_block = [&](int mi, int ni) {
        if constexpr (Epi::kPrefetchOld) {
            const int j = lane & 31, h = lane >> 5;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int id = 8 * (r / 4) + 4 * h + (r % 4);
                const u32 row = row0 + wave_m * Cfg::WTM + (AOp::kKFast ? mi * 32 + id : id * TM + mi);
                if constexpr (kPair) {
                    const v2f o = *reinterpret_cast<const v2f *>(epi.at(row, col0 + wave_n * Cfg::WTN + j * 2));
                    oldv[r] = o.x, oldv[16 + r] = o.y;
                } else {
                    oldv[r] = *epi.at(row, col0 + wave_n * Cfg::WTN + (BOp::kKFast ? ni * 32 + j : j * TN + ni));
                }
            }
        }
    };
    const bool old_ok = Epi::kPrefetchOld && kgroup == 0 && epi.accum_interior(row0, col0, BM, BN, d.M, d.N) &&
                        (!kPair || epi.pair_aligned(col0 + wave_n * Cfg::WTN));
    auto fetch_old = [&]() {
        old_tried = true;
        if constexpr (kOldEarly) {
            if (old_ok) fetch_old_block(0, 0), have_old = true;
        }
    };

    // optional second result of epilogues that carry `a_rowsum`: a_rowsum[m] += sum over k of A(m, k), formed by the
    // workgroups of the first tile column from the A panels they stage anyway, in ascending k (bit-reproducible);
    // thread t < BM owns row t of the panel
    bool do_rowsum = false;
    if constexpr (Epi::kRowSum) do_rowsum = epi.a_rowsum && tn == 0 && threadIdx.x < BM;
    float rowsum = 0.f;

    // the MFMAs of the slab held by LDS buffer `buf`
    auto multiply = [&](int buf) {
        const float *pa = sA[buf], *pb = sB[buf];
        if constexpr (Epi::kRowSum) {
            if (do_rowsum) {
#pragma unroll
                for (int k = 0; k < BK; ++k) rowsum += AOp::kKFast ? pa[threadIdx.x * LA::LD + k] : pa[k * LA::LD + threadIdx.x];
            }
        }
        constexpr int GPW = BK / 8 / Cfg::KG;  // 8-k groups per wave per slab
#pragma unroll
        for (int gi = 0; gi < GPW; ++gi) {
            const int g = Cfg::KG == 1 ? gi : kgroup * GPW + gi;
            float fa[4][TM], fb[4][TN];
            read_frags<AOp::kKFast, TM, LA::LD>(pa, wave_m * Cfg::WTM, g, lane, fa);
            read_frags<BOp::kKFast, TN, LB::LD>(pb, wave_n * Cfg::WTN, g, lane, fb);
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int mi = 0; mi < TM; ++mi)
#pragma unroll
                    for (int ni = 0; ni < TN; ++ni)
                        acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s][mi], fb[s][ni], acc[mi][ni], 0, 0, 0);
        }
    };

    if constexpr (Cfg::PF == 2) {
        // Two register sets: slab t travels in set t % 2. While slab s is multiplied, slab s + 1 is already on its way
        // (issued one iteration earlier) and slab s + 2 is issued; slab s + 1 is committed to LDS after the MFMAs.
        LA la2;
        LB lb2;
        la2.init(a, row0);
        lb2.init(b, col0);
        if (kbeg < kend) {
            la.fetch(a, kbeg, kend);
            lb.fetch(b, kbeg, kend);
            if (kbeg + BK < kend) {
                la2.fetch(a, kbeg + BK, kend);
                lb2.fetch(b, kbeg + BK, kend);
            }
            fetch_old();  // (one-block wave tiles of the accumulating dense form) behind the first slabs: they arrive with them
            la.commit(sA[0]);
            lb.commit(sB[0]);
        }
        __syncthreads();
        // one step: multiply slab k0 (buffer `buf`), issue slab k0 + 2 BK into `far` (the set slab k0 arrived in),
        // commit slab k0 + BK from `near`
        auto step = [&](u32 k0, int buf, LA &far_a, LB &far_b, LA &near_a, LB &near_b) {
            if (k0 + 2 * BK < kend) {
                far_a.fetch(a, k0 + 2 * BK, kend);
                far_b.fetch(b, k0 + 2 * BK, kend);
            }
            if (k0 + BK >= kend && !old_tried) fetch_old();
            multiply(buf);
            if (k0 + BK < kend) {
                near_a.commit(sA[buf ^ 1]);
                near_b.commit(sB[buf ^ 1]);
            }
            __syncthreads();
        };
        for (u32 k0 = kbeg; k0 < kend; k0 += 2 * BK) {
            step(k0, 0, la, lb, la2, lb2);
            if (k0 + BK < kend) step(k0 + BK, 1, la2, lb2, la, lb);
        }
    } else {
        if (kbeg < kend) {
            la.fetch(a, kbeg, kend);
            lb.fetch(b, kbeg, kend);
            la.commit(sA[0]);
            lb.commit(sB[0]);
        }
        __syncthreads();

        int buf = 0;
        for (u32 k0 = kbeg; k0 < kend; k0 += BK, buf ^= 1) {
            const bool more = k0 + BK < kend;
            if (more) {
                la.fetch(a, k0 + BK, kend);
                lb.fetch(b, k0 + BK, kend);
            } else {
                fetch_old();
            }
            multiply(buf);
            if (more) {
                la.commit(sA[buf ^ 1]);
                lb.commit(sB[buf ^ 1]);
            }
            __syncthreads();
        }
    }

    if constexpr (Cfg::KG == 2) {
        // the second K group parks its accumulators in the staging space (idle now: the last slab's barrier has passed),
        // the first adds them to its own and runs the epilogue alone
        float *park = &sA[0][0];
        constexpr int PER_WAVE = TM * TN * 16 * 64;
        static_assert(4 * PER_WAVE <= 2 * LA::SIZE, "parking space");
        if (kgroup == 1) {
#pragma unroll
            for (int mi = 0; mi < TM; ++mi)
#pragma unroll
                for (int ni = 0; ni < TN; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r) park[wave * PER_WAVE + ((mi * TN + ni) * 16 + r) * 64 + lane] = acc[mi][ni][r];
        }
        __syncthreads();
        if (kgroup == 1) return;
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int ni = 0; ni < TN; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[mi][ni][r] += park[wave * PER_WAVE + ((mi * TN + ni) * 16 + r) * 64 + lane];
    }
    if constexpr (Epi::kRowSum) {
        if (do_rowsum && row0 + threadIdx.x < d.M) epi.a_rowsum[row0 + threadIdx.x] += rowsum;
    }
    if (!old_tried) fetch_old();  // empty contraction range
    // epilogue: accumulator register r of lane l is D[8*(r/4) + 4*(l/32) + r%4][l%32] of its block
    const int j = lane & 31, h = lane >> 5;
    // the per-row bias of the 16 rows a lane holds of row block mi: requested together (a load in front of every store
    // would be a memory round trip per element), live for that block only
    float rowb[16];
    auto fetch_row_bias = [&](int mi) {
#pragma unroll
        for (int r = 0; r < 16; ++r) rowb[r] = 0.f;
        if (epi.has_row_bias()) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int id = 8 * (r / 4) + 4 * h + (r % 4);
                const u32 row = row0 + wave_m * Cfg::WTM + (AOp::kKFast ? mi * 32 + id : id * TM + mi);
                rowb[r] = epi.row_bias_at(row < d.M ? row : d.M - 1);
            }
        }
    };
    // A whole tile takes stores that test and read nothing: bounds tests and a conditional read of the previous value in
    // front of every store keep each store waiting for the one before it. Previous values (accumulating forms) and row
    // biases are requested a block at a time, then the block's 16 stores follow one another.
    const bool whole = row0 + BM <= d.M && col0 + BN <= d.N;
    if constexpr (!BOp::kKFast && TN == 2 && Epi::kPairStore) {
        if (whole && epi.pair_aligned(col0 + wave_n * Cfg::WTN)) {
            const u32 col = col0 + wave_n * Cfg::WTN + j * 2;
            const typename Epi::ColS c0 = epi.prep_col(col, d.N), c1 = epi.prep_col(col + 1, d.N);
            const bool accumulates = epi.accumulates();
            if constexpr (Epi::kPrefetchOld) {
#pragma unroll
                for (int r = 0; r < (kPair ? 32 : 16); ++r) oldv[r] = 0.f;
            }
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) {
                fetch_row_bias(mi);
                if (accumulates) fetch_old_block(mi, 0);
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int id = 8 * (r / 4) + 4 * h + (r % 4);
                    const u32 row = row0 + wave_m * Cfg::WTM + (AOp::kKFast ? mi * 32 + id : id * TM + mi);
                    epi.put2(row, c0, c1, acc[mi][0][r], acc[mi][1][r], rowb[r], Epi::kPrefetchOld ? oldv[r] : 0.f,
                             Epi::kPrefetchOld ? oldv[kPair ? 16 + r : 0] : 0.f);
                }
            }
            return;
        }
    } else {
        if (whole) {
            const bool accumulates = epi.accumulates();
            if constexpr (Epi::kPrefetchOld) {
                if (!have_old) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) oldv[r] = 0.f;
                }
            }
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
                const typename Epi::ColS cs = epi.prep_col(col0 + wave_n * Cfg::WTN + (BOp::kKFast ? ni * 32 + j : j * TN + ni), d.N);
#pragma unroll
                for (int mi = 0; mi < TM; ++mi) {
                    fetch_row_bias(mi);
                    if (accumulates && !have_old) fetch_old_block(mi, ni);  // have_old: the one block was requested in the main loop
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int id = 8 * (r / 4) + 4 * h + (r % 4);
                        const u32 row = row0 + wave_m * Cfg::WTM + (AOp::kKFast ? mi * 32 + id : id * TM + mi);
                        epi.put(row, cs, acc[mi][ni][r], rowb[r], Epi::kPrefetchOld ? oldv[r] : 0.f);
                    }
                }
            }
            return;
        }
    }
    if constexpr (!BOp::kKFast && TN == 2 && Epi::kPairStore) {
        // row-fast B: a lane's two blocks are neighbouring columns, stored (and, accumulating, loaded) as one 8-byte access,
        // so that a store instruction writes whole 256-byte runs instead of every other float of them
        const u32 col = col0 + wave_n * Cfg::WTN + j * 2;
        const typename Epi::ColS c0 = epi.prep_col(col, d.N), c1 = epi.prep_col(col + 1, d.N);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi) {
            fetch_row_bias(mi);
            if (old_ok) fetch_old_block(mi, 0), have_old = true;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int id = 8 * (r / 4) + 4 * h + (r % 4);
                const u32 row = row0 + wave_m * Cfg::WTM + (AOp::kKFast ? mi * 32 + id : id * TM + mi);
                if (row < d.M && c0.ok) epi.store2(row, c0, c1, acc[mi][0][r], acc[mi][1][r], rowb[r], have_old, oldv[r], oldv[kPair ? 16 + r : 0]);
            }
        }
    } else {
#pragma unroll
        for (int ni = 0; ni < TN; ++ni) {
            const u32 col = col0 + wave_n * Cfg::WTN + (BOp::kKFast ? ni * 32 + j : j * TN + ni);
            const typename Epi::ColS cs = epi.prep_col(col, d.N);
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) {
                fetch_row_bias(mi);
                if constexpr (!kOldEarly) {
                    if (old_ok) fetch_old_block(mi, ni), have_old = true;
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int id = 8 * (r / 4) + 4 * h + (r % 4);
                    const u32 row = row0 + wave_m * Cfg::WTM + (AOp::kKFast ? mi * 32 + id : id * TM + mi);
                    if (row < d.M) epi.store(row, cs, acc[mi][ni][r], rowb[r], have_old, oldv[r]);
                }
            }
        }
    }
}

// ---- split-K second pass --------------------------------------------------------------------------------
// C[i] (+)= sum_z partial[z][i] (+ bias) (ReLU). A workgroup covers OUTS consecutive outputs with 256/OUTS z-lanes per
// output; every z-lane keeps 4 independent running sums over its strided subset of z (loads in flight instead of one
// dependent chain), then the lanes are combined through LDS in lane order. The association is fixed by (splits, OUTS)
// alone, so repeated runs are bit-identical. Bias index of output i: (i / bias_div) % bias_mod
// (row-major result with per-column bias: div 1, mod N; NCHW with per-channel bias: div H*W, mod C).
struct ReduceEpi {
    const float *bias;
    u32 bias_div, bias_mod;
    u32 flags;  // EPI_ACCUM | EPI_RELU
};

template <int OUTS>
static __global__ void __launch_bounds__(256) splitk_reduce_kernel(const float *__restrict__ partial, float *__restrict__ C, u32 count,
                                                                   u32 splits, ReduceEpi e, FastDiv bdiv) {
    constexpr u32 ZL = 256 / OUTS;
    __shared__ float red[ZL][OUTS];
    const u32 o = threadIdx.x % OUTS, g = threadIdx.x / OUTS;
    const u32 i = blockIdx.x * OUTS + o;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (i < count) {
        const float *p = partial + i;
        u32 zz = g;
        for (; zz + 3 * ZL < splits; zz += 4 * ZL) {
            s0 += p[size_t(zz) * count];
            s1 += p[size_t(zz + ZL) * count];
            s2 += p[size_t(zz + 2 * ZL) * count];
            s3 += p[size_t(zz + 3 * ZL) * count];
        }
        for (; zz < splits; zz += ZL) s0 += p[size_t(zz) * count];
    }
    red[g][o] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (g == 0 && i < count) {
        float r = red[0][o];
#pragma unroll
        for (u32 k = 1; k < ZL; ++k) r += red[k][o];
        if (e.bias) r += e.bias[bdiv.div(i) % e.bias_mod];
        if (e.flags & EPI_ACCUM) r += C[i];
        if (e.flags & EPI_RELU) r = r > 0.f ? r : 0.f;
        C[i] = r;
    }
}

// Same reduction with 16-byte loads: OL lanes cover 4 * OL consecutive results of one slice (a full 128-byte line
// or more), 256 / OL lanes walk the slices.  Needs count % 4 == 0 and 16-byte aligned pointers.
// `red` = 256 / OL rows of 4 * OL + 4 floats of LDS; `block` = which group of 4 * OL results this workgroup sums.
template <int OL>
__device__ __forceinline__ void reduce_vec_block(const float *__restrict__ partial, float *__restrict__ C, u32 count, u32 splits,
                                                 const ReduceEpi &e, const FastDiv &bdiv, u32 block, float *red) {
    constexpr u32 ZL = 256 / OL, OUTS = 4 * OL, RS = OUTS + 4;
    const u32 o = threadIdx.x % OL, g = threadIdx.x / OL;
    const u32 i = block * OUTS + 4 * o;
    // the result's previous value (accumulating forms) is requested before the slices, not after their sum, so that it
    // does not cost a memory round trip of its own at the end
    const u32 j = block * OUTS + threadIdx.x;
    float prev = 0.f, bias_v = 0.f;
    if ((e.flags & EPI_ACCUM) && threadIdx.x < OUTS && j < count) prev = C[j];
    if (e.bias && threadIdx.x < OUTS && j < count) bias_v = e.bias[bdiv.div(j) % e.bias_mod];  // likewise: behind the sum it would be a round trip of its own
    float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0;
    auto add = [](float4 &s, const float4 &v) { s.x += v.x, s.y += v.y, s.z += v.z, s.w += v.w; };
    if (i < count) {
        const float *p = partial + i;
        u32 zz = g;
        // A lane's slices are requested eight, then four, then two at a time (all loads of a batch in flight together);
        // the two running sums take them alternately in slice order whatever the batch size, so the association — and
        // with it every bit of the result — depends on (splits, OL) alone.
        for (; zz + 7 * ZL < splits; zz += 8 * ZL) {
            float4 v[8];
#pragma unroll
            for (u32 q = 0; q < 8; ++q) v[q] = *reinterpret_cast<const float4 *>(p + size_t(zz + q * ZL) * count);
#pragma unroll
            for (u32 q = 0; q < 8; q += 2) add(s0, v[q]), add(s1, v[q + 1]);
        }
        if (zz + 3 * ZL < splits) {
            float4 v[4];
#pragma unroll
            for (u32 q = 0; q < 4; ++q) v[q] = *reinterpret_cast<const float4 *>(p + size_t(zz + q * ZL) * count);
#pragma unroll
            for (u32 q = 0; q < 4; q += 2) add(s0, v[q]), add(s1, v[q + 1]);
            zz += 4 * ZL;
        }
        if (zz + ZL < splits) {
            const float4 a = *reinterpret_cast<const float4 *>(p + size_t(zz) * count);
            const float4 b = *reinterpret_cast<const float4 *>(p + size_t(zz + ZL) * count);
            add(s0, a), add(s1, b);
            zz += 2 * ZL;
        }
        if (zz < splits) add(s0, *reinterpret_cast<const float4 *>(p + size_t(zz) * count));
    }
    *reinterpret_cast<float4 *>(&red[g * RS + 4 * o]) = make_float4(s0.x + s1.x, s0.y + s1.y, s0.z + s1.z, s0.w + s1.w);
    __syncthreads();
    if (threadIdx.x < OUTS && j < count) {
        float r = red[threadIdx.x];
#pragma unroll
        for (u32 k = 1; k < ZL; ++k) r += red[k * RS + threadIdx.x];
        if (e.bias) r += bias_v;
        if (e.flags & EPI_ACCUM) r += prev;
        if (e.flags & EPI_RELU) r = r > 0.f ? r : 0.f;
        C[j] = r;
    }
}
constexpr int kReduceVecLds = 1152;  // floats: the largest of (256 / OL) * (4 * OL + 4) over OL = 8, 16, 32, 64

template <int OL>
static __global__ void __launch_bounds__(256) splitk_reduce_vec_kernel(const float *__restrict__ partial, float *__restrict__ C,
                                                                       u32 count, u32 splits, ReduceEpi e, FastDiv bdiv) {
    __shared__ __attribute__((aligned(16))) float red[(256 / OL) * (4 * OL + 4)];
    reduce_vec_block<OL>(partial, C, count, splits, e, bdiv, blockIdx.x, red);
}

// Lanes per result row of the 16-byte form for a given problem: slice lanes ~ splits / 2, so that every lane has at
// least two independent loads in flight. The association of the sum depends on this choice, so every caller asks here.
inline __host__ __device__ u32 reduce_vec_ol(u32 count, u32 splits) {
    return splits >= 64 ? 8u : (splits >= 32 ? 16u : ((splits >= 16 || count < 256u * 512u) ? 32u : 64u));
}
inline bool reduce_vec_ok(const float *partial, u32 count) { return count % 4 == 0 && reinterpret_cast<uintptr_t>(partial) % 16 == 0; }

inline int launch_splitk_reduce(const float *partial, float *C, u32 count, u32 splits, ReduceEpi e, hipStream_t s,
                                const char *what) {
    FastDiv bdiv(e.bias_div ? e.bias_div : 1);
    if (!e.bias_mod) e.bias_mod = 1;
    if (reduce_vec_ok(partial, count)) {
        switch (reduce_vec_ol(count, splits)) {
            case 8: hipLaunchKernelGGL(splitk_reduce_vec_kernel<8>, dim3(ceil_div(count, 32)), dim3(256), 0, s, partial, C, count, splits, e, bdiv); break;
            case 16: hipLaunchKernelGGL(splitk_reduce_vec_kernel<16>, dim3(ceil_div(count, 64)), dim3(256), 0, s, partial, C, count, splits, e, bdiv); break;
            case 32: hipLaunchKernelGGL(splitk_reduce_vec_kernel<32>, dim3(ceil_div(count, 128)), dim3(256), 0, s, partial, C, count, splits, e, bdiv); break;
            default: hipLaunchKernelGGL(splitk_reduce_vec_kernel<64>, dim3(ceil_div(count, 256)), dim3(256), 0, s, partial, C, count, splits, e, bdiv); break;
        }
        return check_launch(what);
    }
    // enough workgroups to cover the chip even when the result is small
    if (count >= 32u * 512u)
        hipLaunchKernelGGL(splitk_reduce_kernel<32>, dim3(ceil_div(count, 32)), dim3(256), 0, s, partial, C, count, splits, e, bdiv);
    else if (count >= 16u * 256u)
        hipLaunchKernelGGL(splitk_reduce_kernel<16>, dim3(ceil_div(count, 16)), dim3(256), 0, s, partial, C, count, splits, e, bdiv);
    else
        hipLaunchKernelGGL(splitk_reduce_kernel<8>, dim3(ceil_div(count, 8)), dim3(256), 0, s, partial, C, count, splits, e, bdiv);
    return check_launch(what);
}

// The same accumulating reduction for many results in one launch: dst += sum over its slices, item by item, each with
// the association launch_splitk_reduce would use for it (bit-identical results). The items travel in the kernel
// arguments; a workgroup finds its item by its first-block table.
struct SliceSumItem {
    const float *slices;
    float *dst;
    u32 count, n_slices;
};
constexpr int kSliceSumItems = 96;
struct SliceSumArgs {
    SliceSumItem item[kSliceSumItems];
    u32 first_block[kSliceSumItems + 1];
    u32 n;
};
static __global__ void __launch_bounds__(256) slice_sum_multi_kernel(SliceSumArgs a) {
    __shared__ __attribute__((aligned(16))) float red[kReduceVecLds];
    u32 lo = 0, hi = a.n;  // last item whose first block is <= blockIdx.x
    while (hi - lo > 1) {
        const u32 mid = (lo + hi) / 2;
        if (a.first_block[mid] <= blockIdx.x) lo = mid; else hi = mid;
    }
    const SliceSumItem it = a.item[lo];
    const u32 block = blockIdx.x - a.first_block[lo];
    const ReduceEpi e{nullptr, 1, 1, EPI_ACCUM};
    const FastDiv bdiv;
    switch (reduce_vec_ol(it.count, it.n_slices)) {
        case 8: reduce_vec_block<8>(it.slices, it.dst, it.count, it.n_slices, e, bdiv, block, red); break;
        case 16: reduce_vec_block<16>(it.slices, it.dst, it.count, it.n_slices, e, bdiv, block, red); break;
        case 32: reduce_vec_block<32>(it.slices, it.dst, it.count, it.n_slices, e, bdiv, block, red); break;
        default: reduce_vec_block<64>(it.slices, it.dst, it.count, it.n_slices, e, bdiv, block, red); break;
    }
}

// items: host memory. Items the 16-byte form cannot take are reduced by launches of their own.
inline int launch_slice_sum_multi(const SliceSumItem *items, u32 n_items, hipStream_t s, const char *what) {
    SliceSumArgs a;
    a.n = 0;
    u32 blocks = 0;
    auto flush = [&]() -> int {
        if (!a.n) return CRB_OK;
        a.first_block[a.n] = blocks;
        hipLaunchKernelGGL(slice_sum_multi_kernel, dim3(blocks), dim3(256), 0, s, a);
        a.n = 0, blocks = 0;
        return check_launch(what);
    };
    for (u32 i = 0; i < n_items; ++i) {
        const SliceSumItem &it = items[i];
        if (!reduce_vec_ok(it.slices, it.count) || reinterpret_cast<uintptr_t>(it.dst) % 4 != 0) {
            if (int st = launch_splitk_reduce(it.slices, it.dst, it.count, it.n_slices, ReduceEpi{nullptr, 1, 1, EPI_ACCUM}, s, what)) return st;
            continue;
        }
        const u32 nb = ceil_div(it.count, 4 * reduce_vec_ol(it.count, it.n_slices));
        if (a.n == u32(kSliceSumItems) || blocks + nb > 0x3fffffffu)
            if (int st = flush()) return st;
        a.item[a.n] = it;
        a.first_block[a.n] = blocks;
        blocks += nb;
        ++a.n;
    }
    return flush();
}

// How to cut K when an M x N result gives too few macro-tiles to occupy 256 CUs.
struct SplitPlan {
    u32 splits, k_per_z;
};
inline SplitPlan plan_split(u32 M, u32 N, u32 K, u32 BM, u32 BN, u32 BK, u32 zdim) {
    SplitPlan p{1, K};
    const uint64_t tiles = uint64_t(ceil_div(M, BM)) * ceil_div(N, BN) * zdim;
    if (zdim != 1 || tiles >= 160) return p;
    u32 want = u32(ceil_div(512u, u32(tiles)));
    const u32 max_by_k = K / (8 * BK) ? K / (8 * BK) : 1;  // keep at least 8 slabs per slice
    if (want > max_by_k) want = max_by_k;
    if (want <= 1) return p;
    p.k_per_z = ceil_div(ceil_div(K, want), BK) * BK;
    p.splits = ceil_div(K, p.k_per_z);
    if (p.splits <= 1) p = SplitPlan{1, K};
    return p;
}

template <class Cfg, class AOp, class BOp, class Epi>
inline int launch_igemm(const AOp &a, const BOp &b, const Epi &epi, u32 M, u32 N, u32 K, u32 zdim, u32 split_k,
                        u32 k_per_z, hipStream_t stream, const char *what) {
    IgemmDims d;
    d.M = M, d.N = N, d.K = K;
    d.tiles_m = ceil_div(M, Cfg::BM);
    d.tiles_n = ceil_div(N, Cfg::BN);
    d.split_k = split_k;
    d.k_per_z = k_per_z;
    const uint64_t tiles = uint64_t(d.tiles_m) * d.tiles_n;
    if (tiles > 0x7fffffffull || zdim > 65535u) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    dim3 grid(u32(tiles), 1, zdim);
    hipLaunchKernelGGL((igemm_kernel<Cfg, AOp, BOp, Epi>), grid, dim3(Cfg::NTH), 0, stream, a, b, epi, d);
    return check_launch(what);
}

}  // namespace crb
