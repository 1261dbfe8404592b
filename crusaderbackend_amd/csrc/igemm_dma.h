// fp32 MFMA product of two plain dense matrices with operand panels loaded from global memory straight into LDS
// (gfx950: 16 bytes per lane per load, no register hop, no LDS store instruction): D(M x N) = sum_k A(m,k) * B(k,n).
//
// A 256-thread workgroup owns a BM x BN macro-tile and walks the contraction in slabs of 32. A slab's two panels live in
// one of S LDS stages; the loads of slab t + S - 1 are issued while slab t is multiplied, so S - 1 slabs are in flight
// without holding a register, and the hand-over between slabs is a counter wait and one LDS-only barrier (no commit phase).
// A load instruction of a wave writes 1 KB of consecutive LDS (lane l's 16 bytes at base + 16 l), which fixes the layouts:
//   operand contiguous along k ("k-fast": A of NN / NT, B of NT): panel [row][32 k], a row is eight 16-byte chunks, and
//     chunk c of row r is stored in slot c ^ (r % 8) — the lane that fills a slot simply fetches the chunk that belongs
//     there. A fragment read (lane = row, one chunk = the k values of four MFMA steps) then touches eight different
//     slots in any eight consecutive rows: no bank conflicts without padding.
//   operand contiguous along its row index ("row-fast": B of NN / TN, A of TN): panel [32 k][rows], read one float per
//     MFMA step by 32 lanes on consecutive addresses.
// Rows (or row chunks) past the matrix are fetched from the last valid one and never stored; the contraction length must
// be a multiple of 32 (other lengths take the register-staged engine).
//
// v_mfma_f32_32x32x2_f32 (wave64, lane l): A value = A[i = l%32][k = l/32], B value = B[k = l/32][j = l%32], accumulator
// register r = D[8*(r/4) + 4*(l/32) + r%4][l%32]. Within a group of 8 k's, step s of lane-half h consumes k = 4h + s.
#pragma once
#include "igemm_engine.h"

namespace crb {

struct DmaOperand {
    const float *base;
    u32 rows;        // extent along the index that is not contracted (M for A, N for B)
    u32 ld;          // k-fast: floats between consecutive rows; row-fast: floats between consecutive k
    u32 zstride;     // floats between batch entries (0: shared by all)
    u32 cat_k;       // k-fast only: contraction index kk = nd * cat_k + k lives at base + nd * cat_stride + row * ld + k (0: plain)
    u32 cat_stride;
};

struct DmaDims {
    u32 M, N, K;
    u32 tiles_m, tiles_n;
    u32 k_per_z;  // 0: blockIdx.z is a batch index; otherwise it names a slice of the contraction, this many long (multiple of 32)
};

// KG_ = 2: an eight-wave workgroup; both groups of four waves own the whole tile and each multiplies half of every slab
// (two waves per SIMD, so one wave's fragment reads hide behind the other's MFMAs even with one workgroup on the CU); the
// second group's accumulators are added to the first's through LDS before the epilogue.
template <int BM_, int BN_, int WM_, int WN_, int S_, int OCC_, int KG_ = 1>
struct DmaCfg {
    static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_, S = S_, OCC = OCC_, BK = 32, KG = KG_, THREADS = 256 * KG_;
    static constexpr int WTM = BM / WM, WTN = BN / WN, TM = WTM / 32, TN = WTN / 32;
    static_assert(WM * WN == 4 && TM >= 1 && TN >= 1 && TM * 32 * WM == BM && TN * 32 * WN == BN, "tile shape");
    static constexpr int A_FLOATS = BM * BK, B_FLOATS = BK * BN, STAGE = A_FLOATS + B_FLOATS;
    static constexpr int A_PW = A_FLOATS / THREADS / 4, B_PW = B_FLOATS / THREADS / 4;  // 1 KB load instructions per wave per slab
    static_assert(A_FLOATS % (4 * THREADS) == 0 && B_FLOATS % (4 * THREADS) == 0 && (KG == 1 || KG == 2), "whole load instructions per wave");
    static_assert(KG == 1 || 4 * TM * TN * 16 * 64 <= S * STAGE, "room to hand over the second group's accumulators");
    static constexpr int LPS = A_PW + B_PW;
    static_assert((S - 2) * LPS <= 63, "the counter wait must fit its field");
};

#define CRB_GPTR(p) ((const __attribute__((address_space(1))) void *)(p))
#define CRB_LPTR(p) ((__attribute__((address_space(3))) void *)(p))

template <int N>
__device__ __forceinline__ void dma_wait() {
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <class Cfg, bool AKF, bool BKF, class Epi>
__global__ void __launch_bounds__(Cfg::THREADS, Cfg::OCC) igemm_dma_kernel(DmaOperand a, DmaOperand b, Epi epi, DmaDims d) {
    constexpr int BM = Cfg::BM, BN = Cfg::BN, BK = Cfg::BK, S = Cfg::S, TM = Cfg::TM, TN = Cfg::TN;
    constexpr int A_PW = Cfg::A_PW, B_PW = Cfg::B_PW;
    __shared__ __attribute__((aligned(1024))) float smem[S * Cfg::STAGE];

    u32 tm, tn;
    swizzled_tile(blockIdx.x, d.tiles_m, d.tiles_n, tm, tn);
    const u32 z = blockIdx.z;
    u32 kbeg = 0, kend = d.K;
    if (d.k_per_z) {
        kbeg = z * d.k_per_z;
        kend = kbeg + d.k_per_z < d.K ? kbeg + d.k_per_z : d.K;
    } else {
        a.base += size_t(z) * a.zstride, b.base += size_t(z) * b.zstride;
    }
    epi.bind(z);

    const u32 t = threadIdx.x, lane = t & 63, wave = t >> 6;  // the loads are shared out over all waves
    const u32 kgroup = wave >> 2;                              // which half of a slab this wave multiplies (KG == 2)
    const int wave_m = (wave & 3) / Cfg::WN, wave_n = (wave & 3) % Cfg::WN;
    const u32 row0 = tm * BM, col0 = tn * BN;

    // ---- where this lane's load instructions fetch from (slab offset added per slab) ---------------------------------
    // k-fast panel [ROWS][32]: instruction q covers rows 8q .. 8q + 7, lane -> row 8q + lane / 8, slot lane % 8
    // row-fast panel [32][ROWS]: instruction q covers floats 256 q .. of the panel in [k][row] order
    auto src_of = [&](const DmaOperand &op, bool kfast, u32 first, u32 ROWS, u32 q) -> const float * {
        if (kfast) {
            const u32 r = 8 * q + lane / 8, slot = lane & 7, c = slot ^ (r & 7);
            const u32 row = first + r < op.rows ? first + r : op.rows - 1;
            return op.base + size_t(row) * op.ld + 4 * c;
        }
        const u32 e = q * 256 + lane * 4, kr = e / ROWS, cc = e % ROWS;
        const u32 col = first + cc < op.rows ? first + cc : op.rows - 4;  // rows % 4 == 0: a whole valid chunk
        return op.base + size_t(kr) * op.ld + col;
    };
    const float *a_src[A_PW], *b_src[B_PW];
#pragma unroll
    for (int i = 0; i < A_PW; ++i) a_src[i] = src_of(a, AKF, row0, BM, wave * A_PW + i);
#pragma unroll
    for (int i = 0; i < B_PW; ++i) b_src[i] = src_of(b, BKF, col0, BN, wave * B_PW + i);
    // offset of contraction index k0 (a multiple of 32) inside an operand
    auto koff = [&](const DmaOperand &op, bool kfast, u32 k0) -> size_t {
        if (!kfast) return size_t(k0) * op.ld;
        if (op.cat_k) return size_t(k0 / op.cat_k) * op.cat_stride + k0 % op.cat_k;
        return k0;
    };
    auto issue = [&](u32 k0, u32 stage) {
        float *sa = smem + stage * Cfg::STAGE, *sb = sa + Cfg::A_FLOATS;
        const size_t ao = koff(a, AKF, k0), bo = koff(b, BKF, k0);
#pragma unroll
        for (int i = 0; i < A_PW; ++i) __builtin_amdgcn_global_load_lds(CRB_GPTR(a_src[i] + ao), CRB_LPTR(sa + (wave * A_PW + i) * 256), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < B_PW; ++i) __builtin_amdgcn_global_load_lds(CRB_GPTR(b_src[i] + bo), CRB_LPTR(sb + (wave * B_PW + i) * 256), 16, 0, 0);
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int mi = 0; mi < TM; ++mi)
#pragma unroll
        for (int ni = 0; ni < TN; ++ni)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.0f;

    // optional second result of epilogues that carry `a_rowsum` (row-fast A only): a_rowsum[m] += sum over k of A(m, k),
    // formed by the workgroups of the first tile column from the A panels they hold anyway, in ascending k; thread t < BM
    // owns row t of the panel
    bool do_rowsum = false;
    if constexpr (Epi::kRowSum && !AKF) do_rowsum = epi.a_rowsum && tn == 0 && t < BM;
    float rowsum = 0.f;

    const u32 nslab = (kend - kbeg) / BK;
#pragma unroll
    for (int s = 0; s < S - 1; ++s)
        if (u32(s) < nslab) issue(kbeg + s * BK, s);

    const int i32 = lane & 31, h = lane >> 5;
    u32 stage = 0;
    for (u32 sl = 0; sl < nslab; ++sl) {
        // slab sl has landed (this wave's own loads) once at most S - 2 later slabs' loads are outstanding; the barrier then
        // says the same for every wave, and that everyone is done reading the stage that is refilled next
        if (sl + S - 1 <= nslab) dma_wait<(S - 2) * Cfg::LPS>(); else dma_wait<0>();
        lds_barrier();
        if (sl + S - 1 < nslab) issue(kbeg + (sl + S - 1) * BK, stage == 0 ? S - 1 : stage - 1);
        const float *sa = smem + stage * Cfg::STAGE, *sb = sa + Cfg::A_FLOATS;
        if constexpr (Epi::kRowSum && !AKF) {
            if (do_rowsum) {
#pragma unroll
                for (int k = 0; k < BK; ++k) rowsum += sa[k * BM + t];
            }
        }
#pragma unroll
        for (int gi = 0; gi < BK / 8 / Cfg::KG; ++gi) {
            const int g = Cfg::KG == 1 ? gi : int(kgroup) * (BK / 8 / Cfg::KG) + gi;
            float fa[4][TM], fb[4][TN];
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) {
                const int r = wave_m * Cfg::WTM + mi * 32 + i32;
                if constexpr (AKF) {
                    const v4f v = *reinterpret_cast<const v4f *>(sa + r * BK + 4 * ((2 * g + h) ^ (r & 7)));
                    fa[0][mi] = v.x, fa[1][mi] = v.y, fa[2][mi] = v.z, fa[3][mi] = v.w;
                } else {
#pragma unroll
                    for (int s = 0; s < 4; ++s) fa[s][mi] = sa[(8 * g + 4 * h + s) * BM + r];
                }
            }
#pragma unroll
            for (int ni = 0; ni < TN; ++ni) {
                const int c = wave_n * Cfg::WTN + ni * 32 + i32;
                if constexpr (BKF) {
                    const v4f v = *reinterpret_cast<const v4f *>(sb + c * BK + 4 * ((2 * g + h) ^ (c & 7)));
                    fb[0][ni] = v.x, fb[1][ni] = v.y, fb[2][ni] = v.z, fb[3][ni] = v.w;
                } else {
#pragma unroll
                    for (int s = 0; s < 4; ++s) fb[s][ni] = sb[(8 * g + 4 * h + s) * BN + c];
                }
            }
#pragma unroll
            for (int s = 0; s < 4; ++s)
#pragma unroll
                for (int mi = 0; mi < TM; ++mi)
#pragma unroll
                    for (int ni = 0; ni < TN; ++ni) acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[s][mi], fb[s][ni], acc[mi][ni], 0, 0, 0);
        }
        stage = stage + 1 == u32(S) ? 0 : stage + 1;
    }

    if constexpr (Epi::kRowSum && !AKF) {
        if (do_rowsum && row0 + t < d.M) epi.a_rowsum[row0 + t] += rowsum;
    }
    if constexpr (Cfg::KG == 2) {
        // the second group hands its accumulators over through the ring (idle now: the barrier says every wave has read the
        // last slab), the first adds them to its own and runs the epilogue alone
        constexpr int PER_WAVE = TM * TN * 16 * 64;
        lds_barrier();
        if (kgroup == 1) {
#pragma unroll
            for (int mi = 0; mi < TM; ++mi)
#pragma unroll
                for (int ni = 0; ni < TN; ++ni)
#pragma unroll
                    for (int r = 0; r < 16; ++r) smem[(wave & 3) * PER_WAVE + ((mi * TN + ni) * 16 + r) * 64 + lane] = acc[mi][ni][r];
        }
        lds_barrier();
        if (kgroup == 1) return;
#pragma unroll
        for (int mi = 0; mi < TM; ++mi)
#pragma unroll
            for (int ni = 0; ni < TN; ++ni)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[mi][ni][r] += smem[wave * PER_WAVE + ((mi * TN + ni) * 16 + r) * 64 + lane];
    }
    // ---- epilogue: accumulator register r of lane l is D[8*(r/4) + 4*(l/32) + r%4][l%32] of its 32 x 32 block -------------
    if (row0 + BM <= d.M && col0 + BN <= d.N) {
        // A whole tile: no bounds tests, and no read between the stores (a conditional read of the previous value in front of
        // every store keeps each store waiting for the one before it; measured 73 instead of 83 us at 4096 x 4096 x 256).
        const bool accumulates = epi.accumulates(), row_biased = epi.has_row_bias();
#pragma unroll
        for (int ni = 0; ni < TN; ++ni) {
            const typename Epi::ColS cs = epi.prep_col(col0 + wave_n * Cfg::WTN + ni * 32 + i32, d.N);
#pragma unroll
            for (int mi = 0; mi < TM; ++mi) {
                const u32 rbase = row0 + wave_m * Cfg::WTM + mi * 32 + 4 * h;
                float rowb[16], oldv[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) rowb[r] = 0.f, oldv[r] = 0.f;
                if (row_biased) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) rowb[r] = epi.row_bias_at(rbase + 8 * (r / 4) + (r % 4));
                }
                if (accumulates) {
#pragma unroll
                    for (int r = 0; r < 16; ++r) oldv[r] = *epi.at(rbase + 8 * (r / 4) + (r % 4), cs.col);
                }
#pragma unroll
                for (int r = 0; r < 16; ++r) epi.put(rbase + 8 * (r / 4) + (r % 4), cs, acc[mi][ni][r], rowb[r], oldv[r]);
            }
        }
        return;
    }
#pragma unroll
    for (int ni = 0; ni < TN; ++ni) {
        const u32 col = col0 + wave_n * Cfg::WTN + ni * 32 + i32;
        const typename Epi::ColS cs = epi.prep_col(col, d.N);
#pragma unroll
        for (int mi = 0; mi < TM; ++mi) {
            const u32 rbase = row0 + wave_m * Cfg::WTM + mi * 32 + 4 * h;
            // edge tiles: bounds tests per element; a lane's 16 per-row bias values are still requested together
            float rowb[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) rowb[r] = 0.f;
            if (epi.has_row_bias()) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const u32 row = rbase + 8 * (r / 4) + (r % 4);
                    rowb[r] = epi.row_bias_at(row < d.M ? row : d.M - 1);
                }
            }
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const u32 row = rbase + 8 * (r / 4) + (r % 4);
                if (row < d.M) epi.store(row, cs, acc[mi][ni][r], rowb[r]);
            }
        }
    }
}

typedef DmaCfg<128, 128, 2, 2, 2, 2> DmaLarge;  // 64 KB of LDS: two workgroups per CU, one slab in flight each
typedef DmaCfg<64, 64, 2, 2, 4, 2> DmaSmall;    // 64 KB of LDS: two workgroups per CU, three slabs in flight each
typedef DmaCfg<64, 64, 2, 2, 4, 2, 2> DmaSmall8;  // the same tile as eight waves, for grids of at most one tile per CU

// Whether an operand can be loaded this way: 16-byte aligned rows (or k rows) and, row-fast, whole 4-float chunks.
inline bool dma_operand_ok(const DmaOperand &op, bool kfast) {
    if (reinterpret_cast<uintptr_t>(op.base) % 16 || op.ld % 4 || op.zstride % 4 || op.cat_stride % 4) return false;
    if (op.cat_k && (!kfast || op.cat_k % 32)) return false;
    return kfast || (op.rows % 4 == 0 && op.rows >= 4);
}

template <class Cfg, bool AKF, bool BKF, class Epi>
inline int launch_igemm_dma(const DmaOperand &a, const DmaOperand &b, const Epi &e, u32 M, u32 N, u32 K, u32 zdim, u32 k_per_z,
                            hipStream_t s, const char *what) {
    DmaDims d;
    d.M = M, d.N = N, d.K = K;
    d.tiles_m = ceil_div(M, u32(Cfg::BM)), d.tiles_n = ceil_div(N, u32(Cfg::BN));
    d.k_per_z = k_per_z;
    const uint64_t tiles = uint64_t(d.tiles_m) * d.tiles_n;
    if (tiles > 0x7fffffffull || zdim > 65535u) return fail(CRB_EINVAL_SHAPE, "%s: launch grid too large", what);
    hipLaunchKernelGGL((igemm_dma_kernel<Cfg, AKF, BKF, Epi>), dim3(u32(tiles), 1, zdim), dim3(Cfg::THREADS), 0, s, a, b, e, d);
    return check_launch(what);
}

}  // namespace crb
