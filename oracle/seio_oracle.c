/*
 * seio_oracle.c — CPU restatement of the per-image data preparation between a dataset file and the network input:
 * byte pixels to float, the two normalising transforms, and the crop / mirror augmentations.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE (same rule as seblas_oracle.c): only the test-suite, the smoke check
 * and the benchmark's cpu_baseline leg may load it.
 *
 * Each function follows the reference's arithmetic in plain scalar loops, in the reference's order of operations, and
 * cites the lines it restates. The reference cannot be built here and ships no dataset file or expected output; the
 * functions are pinned in tests/test_oracle_seio.py by independent checks:
 *   bytesToFloat    numpy astype
 *   uniformNorm     numpy float64 min/max formula per channel with the running (not per-channel) extrema computed by
 *                   numpy minimum.accumulate / maximum.accumulate; output range is [min, max] exactly for channel 0; a
 *                   hand-written 2-channel case showing that channel 1 is scaled by the extrema of channels 0 and 1 together
 *   distribNorm     numpy float64 mean / biased variance; the result has mean desiredMean and standard deviation
 *                   desiredVar per channel
 *   randCrop        numpy slicing of a zero-padded copy, with row 0 and column 0 of the source treated as outside (the
 *                   reference compares with '> 0'); hand-written 3x3 case
 *   mirrorW         numpy [..., ::-1]
 * No function here is "parity unpinned"; mirrorW restates the mirror the reference's flip intends, not its index
 * arithmetic, which writes one element past each row (seio/data/DataAugmentor.cu:78-80: it stores to column `W - w` with w counted from 0).
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

typedef uint32_t u32;

/* X[i] = (float) bytes[i] (seio/data/DataLoader.cu:34-36). */
void oracle_bytesToFloat(const uint8_t *bytes, float *X, u32 n) {
    for (u32 i = 0; i < n; ++i) X[i] = (float)bytes[i];
}

/* UniformNorm::apply on one image of c channels with `step` values each (seio/data/DataTransform.cu:29-44): the
 * extrema are started once, before the channel loop, so channel k is scaled by the extrema of channels 0..k. */
void oracle_uniformNorm(float *X, u32 c, u32 step, float desiredMin, float desiredMax) {
    float max = -1e10f, min = 1e10f;
    for (u32 ch = 0; ch < c; ++ch) {
        for (u32 i = 0; i < step; ++i) {
            if (X[ch * step + i] > max) max = X[ch * step + i];
            if (X[ch * step + i] < min) min = X[ch * step + i];
        }
        for (u32 i = 0; i < step; ++i) {
            volatile float d = X[ch * step + i] - min; /* volatile: each step rounded to float, no fused multiply-add */
            volatile float q = d / (max - min);
            volatile float s = q * (desiredMax - desiredMin);
            X[ch * step + i] = s + desiredMin;
        }
    }
}

/* DistribNorm::apply on one image (DataTransform.cu:7-27): per channel, mean and biased variance accumulated in float
 * in element order, then (x - mean) * desiredVar / (float) sqrt(var + 1e-8) + desiredMean. */
void oracle_distribNorm(float *X, u32 c, u32 step, float desiredMean, float desiredVar) {
    for (u32 ch = 0; ch < c; ++ch) {
        volatile float srcMean = 0, srcVar = 0;
        for (u32 i = 0; i < step; ++i) srcMean += X[ch * step + i];
        srcMean /= (float)step;
        for (u32 i = 0; i < step; ++i) {
            volatile float d = X[ch * step + i] - srcMean;
            volatile float sq = d * d;
            srcVar += sq;
        }
        srcVar /= (float)step;
        const float sd = (float)sqrt((double)srcVar + 1e-8);
        for (u32 i = 0; i < step; ++i) {
            volatile float d = X[ch * step + i] - srcMean;
            volatile float s = d * desiredVar;
            volatile float q = s / sd;
            X[ch * step + i] = q + desiredMean;
        }
    }
}

/* RandCorp::apply for given per-image offsets (seio/data/DataAugmentor.cu:26-62; the offsets are drawn there from
 * [-pad, pad]): dst(h, w) = src(h + hOffset, w + wOffset) when 0 < h + hOffset < H and 0 < w + wOffset < W, else 0. */
void oracle_randCrop(const float *src, float *dst, u32 n, u32 c, u32 H, u32 W, const int32_t *hOffset, const int32_t *wOffset) {
    for (u32 i = 0; i < n; ++i)
        for (u32 ch = 0; ch < c; ++ch)
            for (int h = 0; h < (int)H; ++h)
                for (int w = 0; w < (int)W; ++w) {
                    const int sh = h + hOffset[i], sw = w + wOffset[i];
                    const int inside = sh > 0 && sh < (int)H && sw > 0 && sw < (int)W;
                    const size_t base = ((size_t)i * c + ch) * H * W;
                    dst[base + (size_t)h * W + w] = inside ? src[base + (size_t)sh * W + sw] : 0.0f;
                }
}

/* Mirror along the width for the images whose flag is set, copy for the others (the effect RandFlipW::apply is written
 * for, DataAugmentor.cu:64-104). */
void oracle_mirrorW(const float *src, float *dst, u32 n, u32 c, u32 H, u32 W, const uint8_t *flip) {
    for (u32 i = 0; i < n; ++i)
        for (size_t row = 0; row < (size_t)c * H; ++row)
            for (u32 w = 0; w < W; ++w) {
                const size_t base = ((size_t)i * c * H + row) * W;
                dst[base + w] = src[base + (flip[i] ? W - 1 - w : w)];
            }
}
