// Operand and epilogue functors for the contraction engine. An operand maps (row, k) of its panel to
// a global-memory value (or 0 outside its extent); an epilogue maps (row, col, value) of the result to
// a store. All offsets are uint32 element offsets (each tensor holds fewer than 2^31 elements).
#pragma once
#include "igemm_engine.h"

namespace crb {

// ---- plain matrices -----------------------------------------------------------------------------------
// element(row, k) = base[row*ld + k]  (k contiguous): A of NN/NT, B of NT.
template <bool VEC>
struct MatK {
    static constexpr bool kKFast = true, kVec = VEC;
    const float *base;
    u32 rows, ld, zstride;
    struct RowS {
        u32 off;
        bool ok;
    };
    struct KS {
        u32 k;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32 z) { base += size_t(z) * zstride; }
    __device__ __forceinline__ RowS prep_row(u32 row) const { return {row * ld, row < rows}; }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const { return {k, k < klimit}; }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        return (r.ok && k.ok) ? base[r.off + k.k] : 0.0f;
    }
    __device__ __forceinline__ v4f fetch4(u32 row, u32 k, u32 klimit) const {
        if (row < rows && k < klimit) return *reinterpret_cast<const v4f *>(base + size_t(row) * ld + k);
        return v4f{0.f, 0.f, 0.f, 0.f};
    }
};

// element(row, k) = base[k*ld + row]  (row contiguous): B of NN/TN, A of TN.
template <bool VEC>
struct MatR {
    static constexpr bool kKFast = false, kVec = VEC;
    const float *base;
    u32 rows, ld, zstride;
    struct RowS {
        u32 row;
        bool ok;
    };
    struct KS {
        u32 off;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32 z) { base += size_t(z) * zstride; }
    __device__ __forceinline__ RowS prep_row(u32 row) const { return {row, row < rows}; }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const { return {k * ld, k < klimit}; }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        return (r.ok && k.ok) ? base[k.off + r.row] : 0.0f;
    }
    __device__ __forceinline__ v4f fetch4(u32 row, u32 k, u32 klimit) const {
        if (row < rows && k < klimit) return *reinterpret_cast<const v4f *>(base + size_t(k) * ld + row);
        return v4f{0.f, 0.f, 0.f, 0.f};
    }
};

// K-concatenated batch of k-contiguous matrices: kk -> (nd = kk / Kb, k = kk % Kb),
// element(row, kk) = base[nd*bstride + row*ld + k]. Operands of the accumulate-NT form.
template <bool VEC>
struct MatKCat {
    static constexpr bool kKFast = true, kVec = VEC;
    const float *base;
    u32 rows, ld, bstride;
    FastDiv kb;
    struct RowS {
        u32 off;
        bool ok;
    };
    struct KS {
        u32 off;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ u32 koff(u32 kk) const {
        u32 nd, k;
        kb.divmod(kk, nd, k);
        return nd * bstride + k;
    }
    __device__ __forceinline__ RowS prep_row(u32 row) const { return {row * ld, row < rows}; }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const { return {koff(k), k < klimit}; }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        return (r.ok && k.ok) ? base[r.off + k.off] : 0.0f;
    }
    __device__ __forceinline__ v4f fetch4(u32 row, u32 k, u32 klimit) const {
        if (row < rows && k < klimit) return *reinterpret_cast<const v4f *>(base + size_t(row) * ld + koff(k));
        return v4f{0.f, 0.f, 0.f, 0.f};
    }
};

// element(row, k) = base[roff(row) + koff(k)] with roff = row*rstride and
// koff(k) = (k / kdiv)*kouter + (k % kdiv)*kinner. Scalar only. Used for
//   dgrad filters  A(ic, (oc,fh,fw)) = W[oc*IC*FHW + ic*FHW + r]      (kdiv = FHW, kouter = IC*FHW, kinner = 1)
//   wgrad dY       A(oc, (n,oh,ow))  = dY[n*OC*OHW + oc*OHW + p]      (kdiv = OHW, kouter = OC*OHW, kinner = 1)
struct SepK {
    static constexpr bool kKFast = true, kVec = false;
    const float *base;
    u32 rows, rstride, kouter, kinner;
    FastDiv kdiv;
    struct RowS {
        u32 off;
        bool ok;
    };
    struct KS {
        u32 off;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ RowS prep_row(u32 row) const { return {row * rstride, row < rows}; }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const {
        u32 q, r;
        kdiv.divmod(k, q, r);
        return {q * kouter + r * kinner, k < klimit};
    }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        return (r.ok && k.ok) ? base[r.off + k.off] : 0.0f;
    }
};

// ---- 3x3 / pad 1 / stride 1 filters seen from a 2x2 image --------------------------------------------------------
// On a 2x2 image every input pixel p' = (y', x') reaches every output pixel p = (y, x) through exactly one tap,
// (fh, fw) = (y' - y + 1, x' - x + 1), so the convolution is a dense product over (channel, pixel) pairs with
//   Wp[oc*4 + p][ic*4 + p'] = W[oc][ic][tap],  tap = 3*fh + fw = (4 - 3y - x) + (3y' + x'):
// the filter offset separates into an output-side and an input-side part. This operand presents W in that form.
// element(row, k) = base[side(row) + side(k)], side(i) = (i / 4)*stride + (out ? 4 - 3*((i/2)%2) - i%2 : 3*((i/2)%2) + i%2).
// rows_out = true: rows are (oc, p) pairs and k runs over (ic, p') (forward); false: the roles are swapped (data gradient).
struct TapPairs {
    static constexpr bool kKFast = true, kVec = false;
    const float *base;
    u32 rows;
    u32 IC;  // input channels of the forward convolution
    bool rows_out;
    struct RowS {
        u32 off;
        bool ok;
    };
    struct KS {
        u32 off;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ u32 side(u32 i, bool out) const {
        const u32 y = (i >> 1) & 1, x = i & 1;
        return out ? (i >> 2) * IC * 9 + 4 - 3 * y - x : (i >> 2) * 9 + 3 * y + x;
    }
    __device__ __forceinline__ RowS prep_row(u32 row) const { return {side(row, rows_out), row < rows}; }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const { return {side(k, !rows_out), k < klimit}; }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        return (r.ok && k.ok) ? base[r.off + k.off] : 0.0f;
    }
};

// ---- implicit im2col gather ---------------------------------------------------------------------------
// value(pixel j = (n, oh, ow), tap t = (ic, fh, fw)) = X[n, ic, oh*sH - pH + fh, ow*sW - pW + fw], 0 outside.
struct Im2col {
    const float *X;
    u32 npix, ntap;  // N*OH*OW, IC*FH*FW
    u32 IH, IW, img_stride /* IC*IH*IW */, chan_stride /* IH*IW */;
    u32 sH, sW, pH, pW;
    FastDiv ohw, ow, fhw, fw;
    struct Pix {
        u32 off;
        int ih0, iw0;
        bool ok;
    };
    struct Tap {
        u32 off;
        int fh, fw;
        bool ok;
    };
    __device__ __forceinline__ Pix pixel(u32 j, u32 limit) const {
        u32 n, p, oh, owi;
        ohw.divmod(j, n, p);
        ow.divmod(p, oh, owi);
        return {n * img_stride, int(oh * sH) - int(pH), int(owi * sW) - int(pW), j < limit};
    }
    __device__ __forceinline__ Tap tap(u32 t, u32 limit) const {
        u32 ic, r, fhi, fwi;
        fhw.divmod(t, ic, r);
        fw.divmod(r, fhi, fwi);
        return {ic * chan_stride, int(fhi), int(fwi), t < limit};
    }
    __device__ __forceinline__ float fetch(const Pix &p, const Tap &t) const {
        const int ih = p.ih0 + t.fh, iw = p.iw0 + t.fw;
        const bool in = p.ok && t.ok && u32(ih) < IH && u32(iw) < IW;
        return in ? X[p.off + t.off + u32(ih) * IW + u32(iw)] : 0.0f;
    }
};

// conv forward B operand: rows are output pixels (contiguous in memory for a fixed tap), k are taps.
struct Im2colPixRows {
    static constexpr bool kKFast = false, kVec = false;
    Im2col g;
    typedef Im2col::Pix RowS;
    typedef Im2col::Tap KS;
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ RowS prep_row(u32 row) const { return g.pixel(row, g.npix); }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const { return g.tap(k, klimit); }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const { return g.fetch(r, k); }
};

// conv wgrad B operand: rows are taps (ic,fh,fw), k are output pixels (contiguous for a fixed tap).
struct Im2colTapRows {
    static constexpr bool kKFast = true, kVec = false;
    Im2col g;
    typedef Im2col::Tap RowS;
    typedef Im2col::Pix KS;
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ RowS prep_row(u32 row) const { return g.tap(row, g.ntap); }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const { return g.pixel(k, klimit); }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const { return g.fetch(k, r); }
};

// conv dgrad B operand: rows are input pixels j = (n, y, x); k = (oc, fh, fw);
// value = dY[n, oc, (y+pH-fh)/sH, (x+pW-fw)/sW] where both divisions are exact and in range, else 0.
struct DgradGather {
    static constexpr bool kKFast = false, kVec = false;
    const float *dY;
    u32 npix;  // N*IH*IW
    u32 OH, OW, img_stride /* OC*OH*OW */, chan_stride /* OH*OW */;
    u32 pH, pW;
    FastDiv ihw, iw, fhw, fw, sH, sW;
    bool unit_stride = false;  // sH == sW == 1: no division per element
    struct RowS {
        u32 off;
        int yp, xp;
        bool ok;
    };
    struct KS {
        u32 off;
        int fh, fw;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ RowS prep_row(u32 j) const {
        u32 n, p, y, x;
        ihw.divmod(j, n, p);
        iw.divmod(p, y, x);
        return {n * img_stride, int(y + pH), int(x + pW), j < npix};
    }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const {
        u32 oc, r, fhi, fwi;
        fhw.divmod(k, oc, r);
        fw.divmod(r, fhi, fwi);
        return {oc * chan_stride, int(fhi), int(fwi), k < klimit};
    }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        const int th = r.yp - k.fh, tw = r.xp - k.fw;
        u32 oh, rh, ow, rw;
        if (unit_stride) {
            oh = u32(th), ow = u32(tw), rh = rw = 0;
        } else {
            sH.divmod(u32(th < 0 ? 0 : th), oh, rh);
            sW.divmod(u32(tw < 0 ? 0 : tw), ow, rw);
        }
        const bool in = r.ok && k.ok && th >= 0 && tw >= 0 && rh == 0 && rw == 0 && oh < OH && ow < OW;
        // the load is issued whatever `in` says (from element 0 when no output pixel feeds this tap): with a branch around
        // it the loads of a staging pass are not in flight together
        const float v = dY[in ? r.off + k.off + oh * OW + ow : 0u];
        return in ? v : 0.0f;
    }
};

// ---- strided data gradient, one residue class of input pixels at a time -----------------------------------------
// At stride (sH, sW) the input pixel (y, x) is reached only through the taps fh = (y + pH) mod sH + i sH,
// fw = (x + pW) mod sW + j sW. All pixels of one residue class (y mod sH, x mod sW) = (py, px) therefore share one tap
// subset, and their gradient is a unit-stride correlation of dY with that subset:
//   dX[n, ic, sH y'' + py, sW x'' + px] = sum over (oc, i, j) of dY[n, oc, y'' + qh - i, x'' + qw - j] W[oc, ic, fh0 + i sH, fw0 + j sW]
// with fh0 = (py + pH) mod sH, qh = (py + pH) / sH (likewise fw0, qw). The gather over all taps multiplies
// (sH sW - 1) / (sH sW) structural zeros; the classes multiply none.
// A operand: rows = input channels, k = (oc, i, j) over the class's taps.
struct ClassTaps {
    static constexpr bool kKFast = true, kVec = false;
    const float *W;
    u32 rows /* IC */, rstride /* FH*FW */, oc_stride /* IC*FH*FW */;
    u32 tap0 /* fh0*FW + fw0 */, tap_i /* sH*FW */, tap_j /* sW */;
    FastDiv ntap /* nfh*nfw */, nfw;
    struct RowS {
        u32 off;
        bool ok;
    };
    struct KS {
        u32 off;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ RowS prep_row(u32 row) const { return {row * rstride, row < rows}; }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const {
        u32 oc, r, i, j;
        ntap.divmod(k, oc, r);
        nfw.divmod(r, i, j);
        return {oc * oc_stride + tap0 + i * tap_i + j * tap_j, k < klimit};
    }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const { return (r.ok && k.ok) ? W[r.off + k.off] : 0.0f; }
};

// B operand: columns are the class's pixels (n, y'', x''); k = (oc, i, j).
struct ClassGather {
    static constexpr bool kKFast = false, kVec = false;
    const float *dY;
    u32 npix;  // N * CH * CW pixels of the class
    u32 OH, OW, img_stride /* OC*OH*OW */, chan_stride /* OH*OW */;
    int qh, qw;
    FastDiv chw, cw, ntap, nfw;
    struct RowS {
        u32 off;
        int y, x;  // y'' + qh, x'' + qw
        bool ok;
    };
    struct KS {
        u32 off;
        int i, j;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ RowS prep_row(u32 col) const {
        u32 n, p, y, x;
        chw.divmod(col, n, p);
        cw.divmod(p, y, x);
        return {n * img_stride, int(y) + qh, int(x) + qw, col < npix};
    }
    __device__ __forceinline__ KS prep_k(u32 k, u32 klimit) const {
        u32 oc, r, i, j;
        ntap.divmod(k, oc, r);
        nfw.divmod(r, i, j);
        return {oc * chan_stride, int(i), int(j), k < klimit};
    }
    __device__ __forceinline__ float fetch(const RowS &r, const KS &k) const {
        const int oh = r.y - k.i, ow = r.x - k.j;
        const bool in = r.ok && k.ok && oh >= 0 && ow >= 0 && oh < int(OH) && ow < int(OW);
        const float v = dY[in ? r.off + k.off + u32(oh) * OW + u32(ow) : 0u];  // issued regardless: no branch around a load
        return in ? v : 0.0f;
    }
};

// ---- epilogues ----------------------------------------------------------------------------------------
// Row-major result C[z*zstride + row*ld + col], optional per-column bias (dense layer) or per-row bias (1x1
// convolution as a batched GEMM), optional accumulate (C += v) and ReLU.
struct RowMajorEpi {
    float *C;
    const float *col_bias;
    u32 ld, zstride, flags;
    const float *row_bias = nullptr;
    u32 col_bias_shift = 0;  // column c takes col_bias[c >> shift] (groups of 2^shift columns share a bias)
    struct ColS {
        u32 col;
        float bias;
        bool ok;
    };
    __device__ __forceinline__ void bind(u32 z) { C += size_t(z) * zstride; }
    __device__ __forceinline__ ColS prep_col(u32 col, u32 ncols) const {
        const bool ok = col < ncols;
        return {col, (ok && col_bias) ? col_bias[col >> col_bias_shift] : 0.0f, ok};
    }
    // accumulating forms may hand in the previous value (`old`, requested a block at a time) instead of having it read here
    static constexpr bool kPrefetchOld = true;
    static constexpr bool kEarlyOld = false;  // the request does not move into the main loop
    static constexpr bool kRowSum = false;
    __device__ __forceinline__ bool accum_interior(u32 row0, u32 col0, u32 bm, u32 bn, u32 M, u32 N) const {
        return (flags & EPI_ACCUM) && row0 + bm <= M && col0 + bn <= N;
    }
    __device__ __forceinline__ const float *at(u32 row, u32 col) const { return C + size_t(row) * ld + col; }
    __device__ __forceinline__ bool accumulates() const { return (flags & EPI_ACCUM) != 0u; }
    // A store that tests and reads nothing: the caller has checked the bounds and hands in the previous value (0 when the
    // form does not accumulate). Same order of additions as store().
    __device__ __forceinline__ void put(u32 row, const ColS &c, float v, float rowb, float old) const {
        v += c.bias;
        v += rowb;
        v += old;
        if (flags & EPI_RELU) v = v > 0.0f ? v : 0.0f;
        C[size_t(row) * ld + c.col] = v;
    }
    __device__ __forceinline__ bool pair_aligned(u32 col) const { return ld % 2 == 0 && (reinterpret_cast<uintptr_t>(C + col) & 7u) == 0; }
    // The per-row bias of a lane's rows is loaded by the caller in one batch (row_bias_at) and handed in as `rowb`: a load
    // in front of every store would be a memory round trip per element.
    __device__ __forceinline__ bool has_row_bias() const { return row_bias != nullptr; }
    __device__ __forceinline__ float row_bias_at(u32 row) const { return row_bias[row]; }
    __device__ __forceinline__ void store(u32 row, const ColS &c, float v, float rowb, bool have_old = false, float old = 0.f) const {
        if (!c.ok) return;
        float *p = C + size_t(row) * ld + c.col;
        v += c.bias;
        v += rowb;
        if (have_old)
            v += old;
        else if (flags & EPI_ACCUM)
            v += *p;
        if (flags & EPI_RELU) v = v > 0.0f ? v : 0.0f;
        *p = v;
    }
    // the same for two neighbouring columns at an 8-byte aligned address
    __device__ __forceinline__ void put2(u32 row, const ColS &c0, const ColS &c1, float v0, float v1, float rowb, float old0, float old1) const {
        v0 += c0.bias, v1 += c1.bias;
        v0 += rowb, v1 += rowb;
        v0 += old0, v1 += old1;
        if (flags & EPI_RELU) v0 = v0 > 0.0f ? v0 : 0.0f, v1 = v1 > 0.0f ? v1 : 0.0f;
        *reinterpret_cast<v2f *>(C + size_t(row) * ld + c0.col) = v2f{v0, v1};
    }
    // Two neighbouring columns of one row (c1.col == c0.col + 1) as one 8-byte access where the address allows it.
    static constexpr bool kPairStore = true;
    __device__ __forceinline__ void store2(u32 row, const ColS &c0, const ColS &c1, float v0, float v1, float rowb, bool have_old = false,
                                           float old0 = 0.f, float old1 = 0.f) const {
        float *p = C + size_t(row) * ld + c0.col;
        if (!c1.ok || (reinterpret_cast<uintptr_t>(p) & 7u)) {
            store(row, c0, v0, rowb, have_old, old0);
            store(row, c1, v1, rowb, have_old, old1);
            return;
        }
        v0 += c0.bias, v1 += c1.bias;
        v0 += rowb, v1 += rowb;
        if (have_old) {
            v0 += old0, v1 += old1;
        } else if (flags & EPI_ACCUM) {
            const v2f old = *reinterpret_cast<const v2f *>(p);
            v0 += old.x, v1 += old.y;
        }
        if (flags & EPI_RELU) v0 = v0 > 0.0f ? v0 : 0.0f, v1 = v1 > 0.0f ? v1 : 0.0f;
        *reinterpret_cast<v2f *>(p) = v2f{v0, v1};
    }
};

// The accumulating dense form (C += A*B with a short contraction, where the epilogue weighs as much as the product):
// previous values of one-block wave tiles are requested before the last slab is multiplied, and the row sums of A can ride
// along (a_rowsum[m] += sum_k A(m, k); null: not wanted; only for one unsplit, unbatched launch).
struct RowMajorAccEpi : RowMajorEpi {
    static constexpr bool kEarlyOld = true;
    static constexpr bool kRowSum = true;
    float *a_rowsum = nullptr;
};

// NCHW scatter: row = channel, col = n*HW + p  ->  T[(n*C + row)*HW + p], optional per-row bias, ReLU.
struct NchwEpi {
    float *T;
    const float *row_bias;
    u32 C, HW, flags;
    FastDiv hw;
    u32 zstride;  // elements between split-K partial results (0 when not splitting)
    struct ColS {
        u32 off;
        bool ok;
    };
    static constexpr bool kPairStore = false;
    static constexpr bool kPrefetchOld = false;
    static constexpr bool kEarlyOld = false;
    static constexpr bool kRowSum = false;
    __device__ __forceinline__ void store2(u32, const ColS &, const ColS &, float, float, float, bool, float, float) const {}
    __device__ __forceinline__ bool has_row_bias() const { return row_bias != nullptr; }
    __device__ __forceinline__ float row_bias_at(u32 row) const { return row_bias[row]; }
    __device__ __forceinline__ void bind(u32 z) { T += size_t(z) * zstride; }
    __device__ __forceinline__ ColS prep_col(u32 col, u32 ncols) const {
        u32 n, p;
        hw.divmod(col, n, p);
        return {n * C * HW + p, col < ncols};
    }
    __device__ __forceinline__ bool accum_interior(u32, u32, u32, u32, u32, u32) const { return false; }
    __device__ __forceinline__ const float *at(u32, u32) const { return nullptr; }
    __device__ __forceinline__ bool pair_aligned(u32) const { return false; }
    __device__ __forceinline__ void store(u32 row, const ColS &c, float v, float rowb, bool = false, float = 0.f) const {
        if (!c.ok) return;
        v += rowb;
        if (flags & EPI_RELU) v = v > 0.0f ? v : 0.0f;
        T[c.off + row * HW] = v;
    }
    __device__ __forceinline__ bool accumulates() const { return false; }
    __device__ __forceinline__ void put(u32 row, const ColS &c, float v, float rowb, float) const {  // bounds checked by the caller
        v += rowb;
        if (flags & EPI_RELU) v = v > 0.0f ? v : 0.0f;
        T[c.off + row * HW] = v;
    }
    __device__ __forceinline__ void put2(u32, const ColS &, const ColS &, float, float, float, float, float) const {}
};

// NCHW scatter of one residue class: row = channel, col = (n, y'', x'') -> T[(n*C + row)*H*W + (sH y'' + py)*W + sW x'' + px].
struct NchwClassEpi {
    float *T;
    u32 C, HW, W;          // channels, pixels per plane, row length of the full tensor
    u32 sH, sW, py, px;
    FastDiv chw, cw;       // pixels per image and per row of the class
    struct ColS {
        u32 off;
        bool ok;
    };
    static constexpr bool kPairStore = false;
    static constexpr bool kPrefetchOld = false;
    static constexpr bool kEarlyOld = false;
    static constexpr bool kRowSum = false;
    __device__ __forceinline__ void store2(u32, const ColS &, const ColS &, float, float, float, bool, float, float) const {}
    __device__ __forceinline__ void put2(u32, const ColS &, const ColS &, float, float, float, float, float) const {}
    __device__ __forceinline__ bool has_row_bias() const { return false; }
    __device__ __forceinline__ float row_bias_at(u32) const { return 0.f; }
    __device__ __forceinline__ void bind(u32) {}
    __device__ __forceinline__ ColS prep_col(u32 col, u32 ncols) const {
        u32 n, p, y, x;
        chw.divmod(col, n, p);
        cw.divmod(p, y, x);
        return {n * C * HW + (sH * y + py) * W + sW * x + px, col < ncols};
    }
    __device__ __forceinline__ bool accum_interior(u32, u32, u32, u32, u32, u32) const { return false; }
    __device__ __forceinline__ const float *at(u32, u32) const { return nullptr; }
    __device__ __forceinline__ bool pair_aligned(u32) const { return false; }
    __device__ __forceinline__ bool accumulates() const { return false; }
    __device__ __forceinline__ void store(u32 row, const ColS &c, float v, float, bool = false, float = 0.f) const {
        if (c.ok) T[c.off + row * HW] = v;
    }
    __device__ __forceinline__ void put(u32 row, const ColS &c, float v, float, float) const { T[c.off + row * HW] = v; }
};

}  // namespace crb
