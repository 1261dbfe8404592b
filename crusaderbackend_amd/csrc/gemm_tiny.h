// Small dense products in ONE launch: C (M x N) = A * B with a result of at most a few hundred thousand elements and a
// contraction too short to be worth a split over workgroups plus a second reduction launch (the dense layers of the CIFAR
// networks: 128 x 512 x 512, 128 x 10 x 512 and their gradients). A workgroup owns one 16 x 16 block of C; its four waves
// each take a quarter of the contraction, fed straight from global memory (the operands are L2-resident at these sizes,
// so there is no LDS staging), and their accumulators are summed through LDS in wave order: bit-reproducible.
//
// v_mfma_f32_16x16x4_f32 (wave64, lane l): A value = A[i = l%16][k = l/16], B value = B[k = l/16][j = l%16], accumulator
// register r = C[4*(l/16) + r][l%16]. When both operands are contiguous along k, a lane loads 16 bytes — the k values
// 16 s + 4 (l/16) + t, t = 0..3 — and feeds them to four MFMAs in turn (A and B agree on the order, which is all the
// contraction needs).
#pragma once
#include "igemm_engine.h"

namespace crb {

struct TinyGemmArgs {
    const float *A, *B;
    float *C;
    const float *col_bias;  // per column, or nullptr
    const float *row_bias;  // per row, or nullptr
    u32 M, N, K;
    u32 a_rs, a_ks;  // element (i, k) of A at A[i * a_rs + k * a_ks]
    u32 b_ks, b_cs;  // element (k, j) of B at B[k * b_ks + j * b_cs]
    u32 ldc, flags;  // EPI_ACCUM | EPI_RELU
    u32 k_per_wave;  // multiple of 16
    u32 tiles_n;
    // K-concatenated batch (the accumulate-NT form): contraction index kk = nd * kb_len + k addresses A + nd * a_bs, B + nd * b_bs;
    // K is then batch * kb_len. Without a batch kb_len = K.
    u32 a_bs, b_bs;
    FastDiv kb_len;
    // optional second result: a_rowsum[i] += sum over k of A(i, k), formed by the workgroups of the first block column
    // (lanes, then waves, in fixed order: bit-reproducible)
    float *a_rowsum = nullptr;
};

template <bool KVEC>
__global__ void __launch_bounds__(256) tiny_gemm_kernel(TinyGemmArgs a) {
    __shared__ __attribute__((aligned(16))) float red[4 * 256];
    __shared__ float rsum[256];
    const u32 t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const u32 li = lane & 15, g = lane >> 4;
    const u32 row0 = (blockIdx.x / a.tiles_n) * 16, col0 = (blockIdx.x % a.tiles_n) * 16;
    const u32 kb = wave * a.k_per_wave;
    const u32 ke = kb + a.k_per_wave < a.K ? kb + a.k_per_wave : a.K;
    const bool row_ok = row0 + li < a.M, col_ok = col0 + li < a.N;
    // What the epilogue adds to the element this thread finishes (row t / 16, column t % 16) is requested now: loaded at
    // the end, bias and previous value would each cost a memory round trip of their own.
    const u32 er = t >> 4, ec = t & 15;
    const u32 erow = row0 + er, ecol = col0 + ec;
    const bool e_ok = erow < a.M && ecol < a.N;
    float *ep = a.C + size_t(e_ok ? erow : 0) * a.ldc + (e_ok ? ecol : 0);
    const float e_cb = (a.col_bias && e_ok) ? a.col_bias[ecol] : 0.f;
    const float e_rb = (a.row_bias && e_ok) ? a.row_bias[erow] : 0.f;
    const float e_old = ((a.flags & EPI_ACCUM) && e_ok) ? *ep : 0.f;
    v4f acc = {0.f, 0.f, 0.f, 0.f};
    float asum = 0.f;  // this lane's share of row li's sum of A
    if constexpr (KVEC) {
        // both operands contiguous along k, K % 4 == 0, 16-byte aligned rows
        const float *pa = a.A + size_t(row0 + li) * a.a_rs;
        const float *pb = a.B + size_t(col0 + li) * a.b_cs;
        constexpr int U = 4;  // 16-k groups requested together
        for (u32 k = kb; k < ke; k += 16 * U) {
            v4f va[U], vb[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const u32 kk = k + 16 * u + 4 * g;
                const bool in = kk < ke;  // ke, kk and the batch length are multiples of 4: a quad is inside or outside as a whole
                u32 nd, kr;
                a.kb_len.divmod(kk, nd, kr);
                va[u] = (in && row_ok) ? *reinterpret_cast<const v4f *>(pa + size_t(nd) * a.a_bs + kr) : v4f{0.f, 0.f, 0.f, 0.f};
                vb[u] = (in && col_ok) ? *reinterpret_cast<const v4f *>(pb + size_t(nd) * a.b_bs + kr) : v4f{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                asum += (va[u].x + va[u].y) + (va[u].z + va[u].w);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(va[u].x, vb[u].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(va[u].y, vb[u].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(va[u].z, vb[u].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(va[u].w, vb[u].w, acc, 0, 0, 0);
            }
        }
    } else {
        const float *pa = a.A + size_t(row0 + li) * a.a_rs;
        const float *pb = a.B + size_t(col0 + li) * a.b_cs;
        constexpr int U = 16;  // MFMA steps requested together
        for (u32 k = kb; k < ke; k += 4 * U) {
            float va[U], vb[U];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const u32 kk = k + 4 * u + g;
                const bool in = kk < ke;
                u32 nd, kr;
                a.kb_len.divmod(kk, nd, kr);
                va[u] = (in && row_ok) ? pa[size_t(nd) * a.a_bs + size_t(kr) * a.a_ks] : 0.f;
                vb[u] = (in && col_ok) ? pb[size_t(nd) * a.b_bs + size_t(kr) * a.b_ks] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                asum += va[u];
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(va[u], vb[u], acc, 0, 0, 0);
            }
        }
    }
    *reinterpret_cast<v4f *>(red + wave * 256 + lane * 4) = acc;
    const bool do_rowsum = a.a_rowsum && col0 == 0;
    if (do_rowsum) rsum[t] = asum;
    __syncthreads();
    if (do_rowsum && t < 16 && row0 + t < a.M) {
        float v = 0.f;
#pragma unroll
        for (int q = 0; q < 16; ++q) v += rsum[q * 16 + t];  // wave q / 4, k lane group q % 4
        a.a_rowsum[row0 + t] += v;
    }
    // thread t finishes element (row t / 16, column t % 16): register row % 4 of lane (row / 4) * 16 + column
    if (!e_ok) return;
    const u32 e = ((er >> 2) * 16 + ec) * 4 + (er & 3);
    float v = red[e];
#pragma unroll
    for (int w = 1; w < 4; ++w) v += red[w * 256 + e];
    if (a.col_bias) v += e_cb;
    if (a.row_bias) v += e_rb;
    if (a.flags & EPI_ACCUM) v += e_old;
    if (a.flags & EPI_RELU) v = v > 0.f ? v : 0.f;
    *ep = v;
}

// Whether the one-launch form takes a product: a small result, a contraction short enough that a quarter of it per wave is
// a few dozen MFMA steps, and enough 16 x 16 blocks (or little enough work) that the chip is not left idle for long.
// K: the whole contraction (batch * K for the K-concatenated accumulate-NT form); batch: independent products (must be 1).
// kfast: both operands are contiguous along k (the NT forms: 16-byte loads). Every block re-reads its operand rows from L2,
// so beyond 2^27 multiply-adds (2^26 with scalar loads) the staged engine wins again (measured, batch 128: 1024 x 1024 one
// launch 9.6 us against 12.9, 1024 x 4096 32.4 against 22.6; data-gradient form 1024 x 512 9.6 against 11.4, 1024 x 1024
// 17.7 against 12.8).
inline bool tiny_gemm_fits(u32 M, u32 N, u32 K, u32 batch, bool kfast = false) {
    if (batch != 1 || uint64_t(M) * N > 512u * 512u || K > 4096u) return false;
    if (uint64_t(M) * N * K > (uint64_t(1) << (kfast ? 27 : 26))) return false;
    const u32 blocks = ceil_div(M, 16u) * ceil_div(N, 16u);
    return blocks >= 64u || uint64_t(M) * N * K <= (1u << 22);
}

// kb_len: length of one batch entry's contraction (a.K for a plain product); a.K = the whole contraction.
inline int launch_tiny_gemm(TinyGemmArgs a, u32 kb_len, u32 a_bs, u32 b_bs, hipStream_t s, const char *what) {
    a.kb_len = FastDiv(kb_len), a.a_bs = a_bs, a.b_bs = b_bs;
    a.tiles_n = ceil_div(a.N, 16u);
    a.k_per_wave = ceil_div(ceil_div(a.K, 4u), 16u) * 16u;
    const u32 blocks = ceil_div(a.M, 16u) * a.tiles_n;
    const bool kvec = a.a_ks == 1 && a.b_ks == 1 && kb_len % 4 == 0 && a_bs % 4 == 0 && b_bs % 4 == 0 && a.a_rs % 4 == 0 && a.b_cs % 4 == 0 &&
                      (reinterpret_cast<uintptr_t>(a.A) & 15u) == 0 && (reinterpret_cast<uintptr_t>(a.B) & 15u) == 0;
    if (kvec)
        hipLaunchKernelGGL(tiny_gemm_kernel<true>, dim3(blocks), dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL(tiny_gemm_kernel<false>, dim3(blocks), dim3(256), 0, s, a);
    return check_launch(what);
}

}  // namespace crb
