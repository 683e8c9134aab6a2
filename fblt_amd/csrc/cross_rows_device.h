/*
 * Cross attention of one new decoder row for one head by one wave: the row
 * sees the few sub-tokens [lo, hi) of its latent patch in the tier-2 cache
 * (csrc/infer/kv_cache.c:240-251, 303-324), so the keys are walked one after
 * the other, lanes over the head's columns.  Softmax as
 * blt_softmax_masked_row_inplace: maximum over finite scores, non-finite
 * scores weigh nothing, an empty or all-dead row gives zeros.  Shared by the
 * stand-alone kernel and by the projection kernels that run it in their
 * epilogue, so that both give the same bits.
 */
#ifndef FBLT_AMD_CROSS_ROWS_DEVICE_H
#define FBLT_AMD_CROSS_ROWS_DEVICE_H

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

/* q: the head's xhd query values; kb / vb: the sequence's slab at the head's first column (row
 * stride E); out: the head's xhd output columns of the row.  xhd <= 256. */
__device__ __forceinline__ void cross_row_head(const float *q, const float *__restrict__ kb,
                                               const float *__restrict__ vb, uint32_t lo, uint32_t hi, uint32_t E,
                                               uint32_t xhd, float scale, float *out, uint32_t lane) {
    auto score = [&](uint32_t j) {
        float p = 0.f;
        for (uint32_t d = lane; d < xhd; d += 64u) p += q[d] * kb[(size_t)j * E + d];
#pragma unroll
        for (int off = 32; off > 0; off >>= 1) p += __shfl_xor(p, off, 64);
        return p * scale;
    };
    float mx = -INFINITY;
    for (uint32_t j = lo; j < hi; j++) {
        const float s = score(j);
        if (isfinite(s)) mx = fmaxf(mx, s);
    }
    float sum = 0.f;
    float acc[4] = {0.f, 0.f, 0.f, 0.f}; /* head widths up to 256 columns */
    for (uint32_t j = lo; j < hi; j++) {
        const float s = score(j);
        const float e = isfinite(s) ? expf(s - mx) : 0.f;
        if (e == 0.f) continue;
        sum += e;
#pragma unroll
        for (int t = 0; t < 4; t++) {
            const uint32_t d = lane + 64u * t;
            if (d < xhd) acc[t] += e * vb[(size_t)j * E + d];
        }
    }
    const float inv = sum > 0.f ? 1.0f / sum : 0.f;
#pragma unroll
    for (int t = 0; t < 4; t++) {
        const uint32_t d = lane + 64u * t;
        if (d < xhd) out[d] = acc[t] * inv;
    }
}

#endif
