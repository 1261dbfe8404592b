// C-ABI entry points of the GEMM and dense-layer families (fp32, row-major) on the MFMA engine.
#include "gemm_internal.h"
#include "gemm_tiny.h"
#include "igemm_dma.h"
#include "operands.h"

namespace crb {

// Macro-tiles. Large: 128x128, each wave a 64x64 block of four 32x32 MFMA tiles. Small: 64x64 for
// problems that would not fill 256 CUs with large tiles.
typedef TileCfg<128, 128, 16, 2, 2, 2> CfgLarge;
typedef TileCfg<64, 64, 16, 2, 2, 2> CfgSmall;
typedef TileCfg<64, 64, 64, 2, 2, 2> CfgSmallDeep;  // 64-wide K slabs: one workgroup per CU has nobody to hide its loads behind
typedef TileCfg<64, 64, 32, 2, 2, 2, 2> CfgSmallAhead;
typedef TileCfg<64, 64, 64, 2, 2, 1, 1, 2> CfgSmallDeep8;  // eight waves: two K groups per macro-tile, for grids of one workgroup per CU  // loads run two slabs ahead: small tiles finish a slab faster than a load takes

static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// Tile choice by how many workgroups the grid gives a CU; when neither tile size fills the chip, K is split — with
// large tiles only when each slice keeps a long contraction (the split costs a second pass over the result).
// `dense` = the result rows are contiguous (ld == N), which the partial results of a split assume.
enum GemmTile { TILE_LARGE, TILE_SMALL, TILE_SMALL_DEEP, TILE_SMALL_AHEAD, TILE_SMALL_DEEP8 };
struct GemmChoice {
    GemmTile tile;
    u32 want_splits;  // > 1: cut K this many times although the tile grid covers the chip
};
static GemmChoice choose_tiles(u32 M, u32 N, u32 K, u32 zdim, bool dense) {
    const uint64_t tiles_l = uint64_t(ceil_div(M, 128)) * ceil_div(N, 128) * zdim;
    const uint64_t tiles_s = uint64_t(ceil_div(M, 64)) * ceil_div(N, 64) * zdim;
    if (M > 64 && N > 64) {
        // measured on square and skinny-K problems: large tiles win once they give a CU three or more workgroups; below
        // that, small tiles with loads two slabs ahead win as soon as there are two of them per CU
        // a short contraction (16 large slabs or fewer) is mostly prologue and epilogue for a large tile
        if (tiles_l >= 800 && K <= 256) return {TILE_SMALL_AHEAD, 0};
        if (tiles_l >= 800) return {TILE_LARGE, 0};
        if (tiles_s >= 512) return {TILE_SMALL_AHEAD, 0};
        // at most one small tile per CU: a contraction long enough is cut in two, so that two workgroups per CU hide each
        // other's loads (measured: pays from K = 1280, from 1024 when the tiles do not cover the CUs evenly) ...
        if (tiles_s >= 160 && K < 2048 && (K >= 1280 || (K >= 1024 && tiles_s > 256)) && zdim == 1 && dense) return {TILE_SMALL_AHEAD, 2};
        // ... a shorter one gets longer slabs, so that a slab's loads have a whole slab of MFMAs (2048 clocks) to arrive in
        // ... with at most one tile per CU as eight waves (two K groups), so that every SIMD still holds two waves
        // (1024^3: 32.0 -> 29.7 us, 1000^3: 30.7 -> 28.6; slabs of 32 or 128 and loads two slabs ahead measured the same)
        if (tiles_s >= 160 && tiles_s <= 256 && K >= 512 && K < 2048) return {TILE_SMALL_DEEP8, 0};
        if (tiles_s >= 160 && K >= 512 && K < 2048) return {TILE_SMALL_DEEP, 0};
        if (tiles_s >= 160 && K < 2048) return {TILE_SMALL_AHEAD, 0};
        // one small tile per CU at most but a long contraction: two K slices per tile put two workgroups on every CU
        if (tiles_s >= 160 && K >= 2048 && zdim == 1 && dense) return {TILE_SMALL_AHEAD, 2};
        if (tiles_l >= 160) return {TILE_LARGE, 0};
        // A grid of small tiles somewhat short of the chip, cut over K by plan_split, beats large tiles cut deeper.
        if (tiles_s >= 100 && K >= 512 && K < 2048) return {TILE_SMALL_AHEAD, 0};
        const SplitPlan sp = plan_split(M, N, K, 128, 128, 16, zdim);
        if (sp.splits > 1 && sp.k_per_z >= 512) return {TILE_LARGE, 0};
    }
    if (K >= 32768) return {TILE_SMALL_AHEAD, 0};  // very long contraction: slices stay long after the split
    // tall and skinny (the im2col shape of a 64-channel layer): one column of 64x64 tiles, two per CU; with 64-wide slabs and
    // eight waves a tile's nine slabs are nine hand-overs instead of 36 (32768 x 64 x 576: 29.3 -> 27.7 us)
    if (M >= 8192 && N > 32 && N <= 64 && K >= 512 && K < 2048 && zdim == 1) return {TILE_SMALL_DEEP8, 0};
    return {TILE_SMALL, 0};
}

// The K split of a tile configuration for a problem (splits == 1: none).
template <class Cfg>
static SplitPlan split_for(u32 M, u32 N, u32 K, u32 zdim, u32 want_splits, bool dense) {
    SplitPlan sp = plan_split(M, N, K, Cfg::BM, Cfg::BN, Cfg::BK, zdim);
    if (want_splits > 1 && zdim == 1 && sp.splits == 1) {  // the caller wants K cut although the tile grid covers the chip
        sp.k_per_z = ceil_div(ceil_div(K, want_splits), u32(Cfg::BK)) * Cfg::BK;
        sp.splits = ceil_div(K, sp.k_per_z);
    }
    if (!dense) sp = SplitPlan{1, K};  // partials assume a dense result
    return sp;
}

// Runs C = A*B through the engine. `e` describes the final result; when the M x N tile grid is too small to occupy the
// chip (and there is no batch), K is cut into slices whose partial results go to scratch and a second kernel combines
// them in fixed order and applies the epilogue (bias / accumulate / ReLU).
template <class Cfg, class AOp, class BOp, class E>
static int run_cfg(const AOp &a, const BOp &b, const E &e, u32 M, u32 N, u32 K, u32 zdim, hipStream_t s, const char *what,
                   u32 want_splits = 0, bool *rowsum_done = nullptr) {
    const SplitPlan sp = split_for<Cfg>(M, N, K, zdim, want_splits, e.ld == N);
    if (sp.splits == 1) {
        if constexpr (E::kRowSum) {
            // the row sums of A ride along only with one unsplit, unbatched launch; otherwise the caller forms them itself
            E e1 = e;
            if (zdim != 1) e1.a_rowsum = nullptr;
            if (rowsum_done) *rowsum_done = e1.a_rowsum != nullptr;
            return launch_igemm<Cfg>(a, b, e1, M, N, K, zdim, 0, K, s, what);
        } else {
            return launch_igemm<Cfg>(a, b, e, M, N, K, zdim, 0, K, s, what);
        }
    }
    const size_t need = size_t(sp.splits) * M * N * sizeof(float);
    float *ws = nullptr;
    if (int st = scratch_get(need, s, what, &ws)) return st;
    RowMajorEpi pe{ws, nullptr, N, M * N, 0u};
    if (int st = launch_igemm<Cfg>(a, b, pe, M, N, K, sp.splits, 1, sp.k_per_z, s, what)) return st;
    if (e.row_bias) return launch_splitk_reduce(ws, e.C, M * N, sp.splits, ReduceEpi{e.row_bias, N, M, e.flags}, s, what);
    return launch_splitk_reduce(ws, e.C, M * N, sp.splits, ReduceEpi{e.col_bias, 1u << e.col_bias_shift, N >> e.col_bias_shift, e.flags},
                                s, what);
}

template <class AOp, class BOp, class E>
static int run_tiles(const AOp &a, const BOp &b, const E &e, u32 M, u32 N, u32 K, u32 zdim, hipStream_t s, const char *what,
                     bool *rowsum_done = nullptr) {
    const GemmChoice c = choose_tiles(M, N, K, zdim, e.ld == N);
    switch (c.tile) {
        case TILE_LARGE: return run_cfg<CfgLarge>(a, b, e, M, N, K, zdim, s, what, c.want_splits, rowsum_done);
        case TILE_SMALL_DEEP: return run_cfg<CfgSmallDeep>(a, b, e, M, N, K, zdim, s, what, c.want_splits, rowsum_done);
        case TILE_SMALL_DEEP8: return run_cfg<CfgSmallDeep8>(a, b, e, M, N, K, zdim, s, what, c.want_splits, rowsum_done);
        case TILE_SMALL_AHEAD: return run_cfg<CfgSmallAhead>(a, b, e, M, N, K, zdim, s, what, c.want_splits, rowsum_done);
        default: return run_cfg<CfgSmall>(a, b, e, M, N, K, zdim, s, what, c.want_splits, rowsum_done);
    }
}

// ---- products of plain dense matrices on the direct-to-LDS kernel (igemm_dma.h) ---------------------------------------------
// Taken when the contraction is a multiple of 32, the operands are 16-byte friendly and the tile grid fills the chip in
// whole rounds; everything else stays on the register-staged engine. Returns 0: not taken; 1: 128 x 128 tiles; 2: 64 x 64.
struct DmaChoice {
    int tile;    // 0: not taken; 1: 128 x 128 tiles; 2: 64 x 64; 3: 64 x 64 as eight waves
    u32 splits;  // > 1: the contraction is cut into this many slices (dense, unbatched results only)
};
static DmaChoice choose_dma(u32 M, u32 N, u32 K, u32 zdim) {
    if (K % 32 || K < 256) return {0, 1};  // whole 32-deep slabs; a short contraction is mostly prologue and epilogue
    const uint64_t tiles_l = uint64_t(ceil_div(M, 128)) * ceil_div(N, 128) * zdim;
    const uint64_t tiles_s = uint64_t(ceil_div(M, 64)) * ceil_div(N, 64) * zdim;
    // One 128 x 128 tile per CU already runs close to the MFMA rate, so the time goes by whole rounds of 256 tiles: taken
    // when the last round is (nearly) full. Measured against the register-staged engine, NN / NT / TN alike:
    // 2048^3 138 vs 150 us, 4096 x 4096 x 256 76 vs 83, 4096^3 1025 vs 1070; 3072^3 (2.25 rounds) 583 vs 494.
    if (M >= 128 && N >= 128 && tiles_l >= 256 && tiles_l * 10 >= ceil_div(tiles_l, 256) * 256 * 9) return {1, 1};
    // 64 x 64 tiles, two per CU: rounds of 512 (512 x 4096 x 1024 40.3 vs 42.8 us, 32768 x 64 x 576 25.3 vs 26.4;
    // 1024^3 the same as the engine, 1536^3 and 1280 x 1024 x 1024 slower)
    if (M >= 64 && N >= 64 && K >= 512 && tiles_s >= 512 && tiles_s * 20 >= ceil_div(tiles_s, 512) * 512 * 19) return {2, 1};
    // At most one 64 x 64 tile per CU: the same tile as an eight-wave workgroup, two waves per SIMD (1024^3 24.0-24.8 us
    // against the engine's eight-wave tiles at 24.1-25.9, 1024 x 1024 x 2048 44.6-46.1 against 45.6-47.5, 896^3 21.4-21.8
    // against 21.4-22.8); longer contractions are better cut (below)
    if (M >= 64 && N >= 64 && K >= 512 && K <= 2048 && tiles_s >= 160 && tiles_s <= 256) return {3, 1};
    // Few tiles and a long contraction: K is cut so that tiles x slices make one round (partial results to scratch, summed
    // in fixed order by the split reduction). Measured against the engine's own split plans, M x N x K: 256 x 4096 x 4096
    // 78 vs 85 us, 512 x 512 x 4096 26.4 vs 29.5, 128 x 2048 x 2048 15.6 vs 17.4, 256 x 1024 x 8192 43.9 vs 50.9; with fewer
    // than 16 tiles the engine's deeper cuts win (128 x 128 x 8192: 10.5 vs 15.8).
    if (zdim == 1 && K >= 1024) {
        if (M >= 128 && N >= 128 && tiles_l >= 64 && tiles_l <= 128 && K / u32(256 / tiles_l) >= 1024) return {1, u32(256 / tiles_l)};
        if (M >= 64 && N >= 64 && tiles_s >= 16 && tiles_s <= 128) {
            u32 splits = u32(512 / tiles_s);
            if (splits > 16) splits = 16;
            if (K / splits >= 256) return {2, splits};
        }
    }
    return {0, 1};
}

// Runs the product through the direct-to-LDS kernel when the operands allow it and the shape is one it wins on. Returns
// false when it did not take the problem (the caller goes on to the engine); `status` is the launch status otherwise.
template <bool AKF, bool BKF, class E>
static bool try_dma(const DmaOperand &a, const DmaOperand &b, const E &e, u32 M, u32 N, u32 K, u32 zdim, hipStream_t s, const char *what,
                    int &status, bool *rowsum_done = nullptr) {
    if (K % 32 || !dma_operand_ok(a, AKF) || !dma_operand_ok(b, BKF)) return false;
    const DmaChoice c = choose_dma(M, N, K, zdim);
    if (!c.tile) return false;
    if (c.splits > 1) {
        if (zdim != 1 || e.ld != N || a.cat_k || b.cat_k) return false;
        const u32 k_per_z = ceil_div(ceil_div(K, c.splits), 32u) * 32u, splits = ceil_div(K, k_per_z);
        float *ws = nullptr;
        if ((status = scratch_get(size_t(splits) * M * N * sizeof(float), s, what, &ws))) return true;
        RowMajorEpi pe{ws, nullptr, N, M * N, 0u};
        status = c.tile == 1   ? launch_igemm_dma<DmaLarge, AKF, BKF>(a, b, pe, M, N, K, splits, k_per_z, s, what)
                 : c.tile == 2 ? launch_igemm_dma<DmaSmall, AKF, BKF>(a, b, pe, M, N, K, splits, k_per_z, s, what)
                               : launch_igemm_dma<DmaSmall8, AKF, BKF>(a, b, pe, M, N, K, splits, k_per_z, s, what);
        if (status) return true;
        status = e.row_bias ? launch_splitk_reduce(ws, e.C, M * N, splits, ReduceEpi{e.row_bias, N, M, e.flags}, s, what)
                            : launch_splitk_reduce(ws, e.C, M * N, splits, ReduceEpi{e.col_bias, 1u << e.col_bias_shift, N >> e.col_bias_shift, e.flags}, s, what);
        return true;
    }
    E e1 = e;
    if constexpr (E::kRowSum) {
        if (zdim != 1 || AKF) e1.a_rowsum = nullptr;  // the row sums ride along with one unbatched launch on a row-fast A only
        if (rowsum_done) *rowsum_done = e1.a_rowsum != nullptr;
    }
    status = c.tile == 1   ? launch_igemm_dma<DmaLarge, AKF, BKF>(a, b, e1, M, N, K, zdim, 0, s, what)
             : c.tile == 2 ? launch_igemm_dma<DmaSmall, AKF, BKF>(a, b, e1, M, N, K, zdim, 0, s, what)
                           : launch_igemm_dma<DmaSmall8, AKF, BKF>(a, b, e1, M, N, K, zdim, 0, s, what);
    return true;
}

// Scratch bytes run_tiles asks for on a dense M x N result with contraction length K (0: the contraction is not cut).
size_t gemm_scratch_bytes(u32 M, u32 N, u32 K, u32 zdim, bool one_launch_form) {
    if (one_launch_form && tiny_gemm_fits(M, N, K, zdim)) return 0;  // one launch, no partial results
    // the direct-to-LDS kernel needs friendly operands, which a size query cannot see: the larger of its need and the engine's
    size_t dma_need = 0;
    if (one_launch_form) {  // (callers that name the tiled engine directly never take the direct-to-LDS kernel)
        const DmaChoice dc = choose_dma(M, N, K, zdim);
        if (dc.tile && dc.splits > 1) {
            const u32 k_per_z = ceil_div(ceil_div(K, dc.splits), 32u) * 32u;
            dma_need = size_t(ceil_div(K, k_per_z)) * M * N * sizeof(float);
        }
    }
    const GemmChoice c = choose_tiles(M, N, K, zdim, true);
    SplitPlan sp;
    switch (c.tile) {
        case TILE_LARGE: sp = split_for<CfgLarge>(M, N, K, zdim, c.want_splits, true); break;
        case TILE_SMALL_DEEP: sp = split_for<CfgSmallDeep>(M, N, K, zdim, c.want_splits, true); break;
        case TILE_SMALL_DEEP8: sp = split_for<CfgSmallDeep8>(M, N, K, zdim, c.want_splits, true); break;
        case TILE_SMALL_AHEAD: sp = split_for<CfgSmallAhead>(M, N, K, zdim, c.want_splits, true); break;
        default: sp = split_for<CfgSmall>(M, N, K, zdim, c.want_splits, true); break;
    }
    const size_t eng = sp.splits > 1 ? size_t(sp.splits) * M * N * sizeof(float) : 0;
    return eng > dma_need ? eng : dma_need;
}

static int check_dims(const char *what, u32 M, u32 N, u32 K, u32 batch) {
    if (M == 0 || N == 0 || K == 0 || batch == 0) return fail(CRB_EINVAL_SHAPE, "%s: zero dimension", what);
    const uint64_t lim = 0x7fffffffull;
    if (uint64_t(M) * K * batch > lim || uint64_t(K) * N * batch > lim || uint64_t(M) * N * batch > lim)
        return fail(CRB_EINVAL_SHAPE, "%s: operand exceeds 2^31 elements", what);
    return CRB_OK;
}

// column sums of a (rows x cols) row-major matrix: out[c] += sum_r in[r*cols + c]. 32 columns x 8 row-lanes per
// workgroup; a row-lane sums rows lane, lane+8, ... with 4 independent running sums, the 8 lanes are combined through
// LDS in lane order (fixed association: bit-reproducible).
__global__ void __launch_bounds__(256) colsum_accum_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                           u32 rows, u32 cols) {
    __shared__ float red[8][32];
    const u32 o = threadIdx.x % 32, g = threadIdx.x / 32;
    const u32 c = blockIdx.x * 32 + o;
    float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
    if (c < cols) {
        const float *p = in + c;
        u32 r = g;
        for (; r + 24 < rows; r += 32) {
            s0 += p[size_t(r) * cols];
            s1 += p[size_t(r + 8) * cols];
            s2 += p[size_t(r + 16) * cols];
            s3 += p[size_t(r + 24) * cols];
        }
        for (; r < rows; r += 8) s0 += p[size_t(r) * cols];
    }
    red[g][o] = (s0 + s1) + (s2 + s3);
    __syncthreads();
    if (g == 0 && c < cols) {
        float r = red[0][o];
#pragma unroll
        for (int k = 1; k < 8; ++k) r += red[k][o];
        out[c] += r;
    }
}

static int gemm_nn(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, u32 batch, const float *col_bias,
                   u32 flags, hipStream_t s, const char *what, const float *row_bias = nullptr) {
    if (tiny_gemm_fits(M, N, K, batch))  // A (M x K) row-major, B (K x N) row-major
        return launch_tiny_gemm(TinyGemmArgs{A, B, C, col_bias, row_bias, M, N, K, K, 1, N, 1, N, flags}, K, 0, 0, s, what);
    RowMajorEpi e{C, col_bias, N, M * N, flags};
    e.row_bias = row_bias;
    if (K % 4 == 0 && N % 4 == 0 && aligned16(A) && aligned16(B)) {
        int st = CRB_OK;
        if (try_dma<true, false>(DmaOperand{A, M, K, 0, 0, 0}, DmaOperand{B, N, N, K * N, 0, 0}, e, M, N, K, batch, s, what, st)) return st;
        MatK<true> a{A, M, K, 0};
        MatR<true> b{B, N, N, K * N};
        return run_tiles(a, b, e, M, N, K, batch, s, what);
    }
    MatK<false> a{A, M, K, 0};
    MatR<false> b{B, N, N, K * N};
    return run_tiles(a, b, e, M, N, K, batch, s, what);
}

static int gemm_tn(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, u32 batch, u32 flags,
                   hipStream_t s, const char *what, float *a_rowsum = nullptr, bool *rowsum_done = nullptr) {
    if (rowsum_done) *rowsum_done = false;
    if (tiny_gemm_fits(M, N, K, batch)) {  // A stored K x M, B (K x N) row-major
        TinyGemmArgs t{A, B, C, nullptr, nullptr, M, N, K, 1, M, N, 1, N, flags};
        t.a_rowsum = a_rowsum;
        if (rowsum_done) *rowsum_done = a_rowsum != nullptr;
        return launch_tiny_gemm(t, K, 0, 0, s, what);
    }
    RowMajorEpi e{C, nullptr, N, M * N, flags};
    if (M % 4 == 0 && N % 4 == 0 && aligned16(A) && aligned16(B)) {
        MatR<true> a{A, M, M, 0};
        MatR<true> b{B, N, N, K * N};
        int st = CRB_OK;
        const DmaOperand da{A, M, M, 0, 0, 0}, db{B, N, N, K * N, 0, 0};
        if (flags & EPI_ACCUM) {  // the dense layers' weight gradient
            RowMajorAccEpi ea;
            static_cast<RowMajorEpi &>(ea) = e;
            ea.a_rowsum = a_rowsum;
            if (try_dma<false, false>(da, db, ea, M, N, K, batch, s, what, st, rowsum_done)) return st;
            return run_tiles(a, b, ea, M, N, K, batch, s, what, rowsum_done);
        }
        if (try_dma<false, false>(da, db, e, M, N, K, batch, s, what, st)) return st;
        return run_tiles(a, b, e, M, N, K, batch, s, what);
    }
    MatR<false> a{A, M, M, 0};
    MatR<false> b{B, N, N, K * N};
    return run_tiles(a, b, e, M, N, K, batch, s, what);
}

static int gemm_nt(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, const float *col_bias, u32 flags,
                   hipStream_t s, const char *what) {
    if (tiny_gemm_fits(M, N, K, 1, true))  // A (M x K) row-major, B stored N x K
        return launch_tiny_gemm(TinyGemmArgs{A, B, C, col_bias, nullptr, M, N, K, K, 1, 1, K, N, flags}, K, 0, 0, s, what);
    RowMajorEpi e{C, col_bias, N, 0, flags};
    if (K % 4 == 0 && aligned16(A) && aligned16(B)) {
        int st = CRB_OK;
        if (try_dma<true, true>(DmaOperand{A, M, K, 0, 0, 0}, DmaOperand{B, N, K, 0, 0, 0}, e, M, N, K, 1, s, what, st)) return st;
        MatK<true> a{A, M, K, 0};
        MatK<true> b{B, N, K, 0};
        return run_tiles(a, b, e, M, N, K, 1, s, what);
    }
    MatK<false> a{A, M, K, 0};
    MatK<false> b{B, N, K, 0};
    return run_tiles(a, b, e, M, N, K, 1, s, what);
}

// ---- 3x3 / pad 1 / stride 1 convolution of 2x2 images as dense products over (channel, pixel) pairs -------------------
// X, Y, dY, dX are then plain row-major matrices: N x (C*4).

int conv2x2_fwd(const float *W, const float *X, float *Y, const float *bias, u32 N, u32 IC, u32 OC, u32 flags, hipStream_t s,
                const char *what) {
    // Y (N x OC*4) = X (N x IC*4) * Wp^T, bias per group of 4 columns
    RowMajorEpi e{Y, bias, OC * 4, 0, flags};
    e.col_bias_shift = 2;
    MatK<true> a{X, N, IC * 4, 0};
    TapPairs b{W, OC * 4, IC, true};
    return run_tiles(a, b, e, N, OC * 4, IC * 4, 1, s, what);
}

int conv2x2_dgrad(const float *W, const float *dY, float *dX, u32 N, u32 IC, u32 OC, hipStream_t s, const char *what) {
    // dX (N x IC*4) = dY (N x OC*4) * Wp
    RowMajorEpi e{dX, nullptr, IC * 4, 0, 0u};
    MatK<true> a{dY, N, OC * 4, 0};
    TapPairs b{W, IC * 4, IC, false};
    return run_tiles(a, b, e, N, IC * 4, OC * 4, 1, s, what);
}

// dW[oc][ic][tap] += sum over the (p, p') pairs that meet in that tap of G[oc*4 + p][ic*4 + p'] (1, 2 or 4 pairs per tap)
__global__ void __launch_bounds__(256) conv2x2_fold_kernel(const float *__restrict__ G, float *__restrict__ dW, u32 OC, u32 IC) {
    const u32 i = blockIdx.x * 256 + threadIdx.x;  // (oc, ic) pair
    if (i >= OC * IC) return;
    const u32 oc = i / IC, ic = i % IC;
    float acc[9];
#pragma unroll
    for (int t = 0; t < 9; ++t) acc[t] = 0.f;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const v4f g = *reinterpret_cast<const v4f *>(G + (size_t(oc) * 4 + p) * (IC * 4) + ic * 4);
        const int o = 4 - 3 * (p >> 1) - (p & 1);
        acc[o + 0] += g.x, acc[o + 1] += g.y, acc[o + 3] += g.z, acc[o + 4] += g.w;
    }
    float *dst = dW + size_t(i) * 9;
#pragma unroll
    for (int t = 0; t < 9; ++t) dst[t] += acc[t];
}

int conv2x2_wgrad(const float *dY, const float *X, float *dW, float *G, u32 N, u32 IC, u32 OC, hipStream_t s, const char *what) {
    // G (OC*4 x IC*4, caller's scratch) = dY^T * X over the batch, then folded into the 9 taps
    const u32 M = OC * 4, Nc = IC * 4;
    RowMajorEpi e{G, nullptr, Nc, 0, 0u};
    MatR<true> a{dY, M, M, 0};
    MatR<true> b{X, Nc, Nc, 0};
    // G may be the library's scratch arena, so the contraction is never split here
    const uint64_t tiles_l = uint64_t(ceil_div(M, 128)) * ceil_div(Nc, 128);
    const uint64_t tiles_s = uint64_t(ceil_div(M, 64)) * ceil_div(Nc, 64);
    int st = tiles_l >= 800   ? launch_igemm<CfgLarge>(a, b, e, M, Nc, N, 1, 0, N, s, what)
             : tiles_s >= 512 ? launch_igemm<CfgSmallAhead>(a, b, e, M, Nc, N, 1, 0, N, s, what)
             : tiles_l >= 128 ? launch_igemm<CfgLarge>(a, b, e, M, Nc, N, 1, 0, N, s, what)
                              : launch_igemm<CfgSmall>(a, b, e, M, Nc, N, 1, 0, N, s, what);
    if (st) return st;
    hipLaunchKernelGGL(conv2x2_fold_kernel, dim3(ceil_div(OC * IC, 256)), dim3(256), 0, s, G, dW, OC, IC);
    return check_launch(what);
}

int gemm_nn_rowbias(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, u32 batch, const float *row_bias, u32 flags,
                    hipStream_t s, const char *what) {
    return gemm_nn(A, B, C, M, N, K, batch, nullptr, flags, s, what, row_bias);
}

int gemm_tn_batched(const float *A, const float *B, float *C, u32 M, u32 N, u32 K, u32 batch, hipStream_t s, const char *what) {
    return gemm_tn(A, B, C, M, N, K, batch, 0, s, what);
}

}  // namespace crb

using namespace crb;

extern "C" {

size_t crb_gemm_workspace_bytes(uint32_t M, uint32_t N, uint32_t K, uint32_t batch) {
    if (check_dims("crb_gemm_workspace_bytes", M, N, K, batch)) return 0;
    return gemm_scratch_bytes(M, N, K, batch);
}

int crb_sgemm_nn(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                 void *stream) {
    if (!A || !B || !C) return fail(CRB_ENULL, "crb_sgemm_nn: null operand");
    if (int st = check_dims("crb_sgemm_nn", M, N, K, batch)) return st;
    return gemm_nn(A, B, C, M, N, K, batch, nullptr, 0, hipStream_t(stream), "crb_sgemm_nn");
}

int crb_sgemm_tn(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                 void *stream) {
    if (!A || !B || !C) return fail(CRB_ENULL, "crb_sgemm_tn: null operand");
    if (int st = check_dims("crb_sgemm_tn", M, N, K, batch)) return st;
    return gemm_tn(A, B, C, M, N, K, batch, 0, hipStream_t(stream), "crb_sgemm_tn");
}

int crb_sgemm_nt(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, void *stream) {
    if (!A || !B || !C) return fail(CRB_ENULL, "crb_sgemm_nt: null operand");
    if (int st = check_dims("crb_sgemm_nt", M, N, K, 1)) return st;
    return gemm_nt(A, B, C, M, N, K, nullptr, 0, hipStream_t(stream), "crb_sgemm_nt");
}

int crb_sgemm_nta(const float *A, const float *B, float *C, uint32_t M, uint32_t N, uint32_t K, uint32_t batch,
                  void *stream) {
    if (!A || !B || !C) return fail(CRB_ENULL, "crb_sgemm_nta: null operand");
    if (int st = check_dims("crb_sgemm_nta", M, N, K, batch)) return st;
    if (uint64_t(K) * batch > 0x7fffffffull) return fail(CRB_EINVAL_SHAPE, "crb_sgemm_nta: K*batch too large");
    const u32 KK = K * batch;
    RowMajorEpi e{C, nullptr, N, 0, EPI_ACCUM};
    hipStream_t s = hipStream_t(stream);
    if (tiny_gemm_fits(M, N, KK, 1))  // the batch concatenated along the contraction
        return launch_tiny_gemm(TinyGemmArgs{A, B, C, nullptr, nullptr, M, N, KK, K, 1, 1, K, N, EPI_ACCUM}, K, M * K, N * K, s, "crb_sgemm_nta");
    if (K % 4 == 0 && aligned16(A) && aligned16(B)) {
        int st = CRB_OK;
        if (K % 32 == 0 && try_dma<true, true>(DmaOperand{A, M, K, 0, K, M * K}, DmaOperand{B, N, K, 0, K, N * K}, e, M, N, KK, 1, s, "crb_sgemm_nta", st))
            return st;
        MatKCat<true> a{A, M, K, M * K, FastDiv(K)};
        MatKCat<true> b{B, N, K, N * K, FastDiv(K)};
        return run_tiles(a, b, e, M, N, KK, 1, s, "crb_sgemm_nta");
    }
    MatKCat<false> a{A, M, K, M * K, FastDiv(K)};
    MatKCat<false> b{B, N, K, N * K, FastDiv(K)};
    return run_tiles(a, b, e, M, N, KK, 1, s, "crb_sgemm_nta");
}

int crb_linear_fwd(const float *X, const float *W, const float *bias, float *Y, uint32_t batch, uint32_t IN,
                   uint32_t OUT, uint32_t flags, void *stream) {
    if (!X || !W || !bias || !Y) return fail(CRB_ENULL, "crb_linear_fwd: null operand");
    if (int st = check_dims("crb_linear_fwd", batch, OUT, IN, 1)) return st;
    // Y (batch x OUT) = X (batch x IN) * W^T, bias broadcast along rows
    return gemm_nt(X, W, Y, batch, OUT, IN, bias, (flags & CRB_FLAG_RELU) ? EPI_RELU : 0u, hipStream_t(stream),
                   "crb_linear_fwd");
}

int crb_linear_dgrad(const float *dY, const float *W, float *dX, uint32_t batch, uint32_t IN, uint32_t OUT,
                     void *stream) {
    if (!dY || !W || !dX) return fail(CRB_ENULL, "crb_linear_dgrad: null operand");
    if (int st = check_dims("crb_linear_dgrad", batch, IN, OUT, 1)) return st;
    // dX (batch x IN) = dY (batch x OUT) * W (OUT x IN)
    return gemm_nn(dY, W, dX, batch, IN, OUT, 1, nullptr, 0, hipStream_t(stream), "crb_linear_dgrad");
}

int crb_linear_wgrad(const float *dY, const float *X, float *dW, float *dB, uint32_t batch, uint32_t IN,
                     uint32_t OUT, void *stream) {
    if (!dY || !X || !dW) return fail(CRB_ENULL, "crb_linear_wgrad: null operand");
    if (int st = check_dims("crb_linear_wgrad", OUT, IN, batch, 1)) return st;
    hipStream_t s = hipStream_t(stream);
    // dW (OUT x IN) += dY^T (dY stored batch x OUT) * X (batch x IN)
    // the bias gradient (column sums of dY = row sums of the A operand) rides along with an unsplit product
    bool db_done = false;
    if (int st = gemm_tn(dY, X, dW, OUT, IN, batch, 1, EPI_ACCUM, s, "crb_linear_wgrad", dB, &db_done)) return st;
    if (dB && !db_done) {
        hipLaunchKernelGGL(colsum_accum_kernel, dim3(ceil_div(OUT, 32)), dim3(256), 0, s, dY, dB, batch, OUT);
        return check_launch("crb_linear_wgrad(dB)");
    }
    return CRB_OK;
}

}  // extern "C"
