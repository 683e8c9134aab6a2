/*
 * Device-side view of one attention problem and the helpers every attention
 * kernel shares.  gfx950 only: 64-lane wavefronts are assumed throughout.
 */
#ifndef FBLT_AMD_ATTN_DEVICE_H
#define FBLT_AMD_ATTN_DEVICE_H

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

enum : uint32_t {
    ATTN_VIS_ALL = 0,    /* every key below nk                                  */
    ATTN_VIS_CAUSAL = 1, /* j <= i + causal_off, optional back window           */
    ATTN_VIS_DENSE = 2,  /* additive fp32 matrix [nq, nk]                       */
    ATTN_VIS_RANGE = 3   /* row_lo[i] <= j < row_hi[i]                          */
};

enum : uint32_t {
    ATTN_FLAG_VEC4 = 1u /* q/k/v/out pointers and strides are 16-byte aligned, head_dim % 4 == 0 */
};

/* One (sequence, head) problem as the kernels read it.  `out` already points
 * at the head's first output column. */
struct AttnProb {
    const float *q;
    const float *k;
    const float *v;
    float *out;
    float *weights;      /* optional [nq, nk]          */
    float *lse;          /* optional [nq, 2]           */
    const float *mask;   /* ATTN_VIS_DENSE             */
    const uint32_t *row_lo;
    const uint32_t *row_hi;
    uint32_t q_stride, k_stride, v_stride, out_stride; /* elements */
    uint32_t nq, nk, hd;
    uint32_t vis;
    uint32_t causal_off, window;
    float scale;
    uint32_t flags;
    uint32_t range_span; /* ATTN_VIS_RANGE: longest range of a row if the caller said so, else 0 */
    uint32_t reserved1;
};

static_assert(sizeof(AttnProb) == 128, "AttnProb is staged to the device as raw bytes");

__device__ __forceinline__ float neg_inf() { return -__builtin_huge_valf(); }

/* Key range [lo, hi) outside of which row i sees nothing.  Inside the range
 * every key is visible, except for ATTN_VIS_DENSE where the matrix decides. */
__device__ __forceinline__ void row_key_range(const AttnProb &p, uint32_t i, uint32_t &lo, uint32_t &hi) {
    lo = 0;
    hi = p.nk;
    if (p.vis == ATTN_VIS_CAUSAL) {
        const uint64_t diag = (uint64_t)i + p.causal_off;
        if (diag + 1 < hi) hi = (uint32_t)(diag + 1);
        if (p.window > 0 && diag + 1 > p.window) {
            const uint64_t l = diag + 1 - p.window;
            lo = l < p.nk ? (uint32_t)l : p.nk;
        }
    } else if (p.vis == ATTN_VIS_RANGE) {
        lo = p.row_lo[i];
        hi = p.row_hi[i];
        if (hi > p.nk) hi = p.nk;
    }
    if (lo > hi) lo = hi;
}

/* exp for softmax weights: argument is <= 0 (or -inf). */
__device__ __forceinline__ float softmax_exp(float x) { return __expf(x); }

#endif /* FBLT_AMD_ATTN_DEVICE_H */
