/*
 * Device helpers shared by the matrix-core attention kernels: the 32x32
 * accumulator layout of v_mfma_f32_32x32x2_f32, log2-domain softmax
 * constants, problem lookup for strided batches and key-tile bounds.
 */
#ifndef FBLT_AMD_ATTN_TILE_H
#define FBLT_AMD_ATTN_TILE_H

#include "attn_device.h"
#include "attn_launch.h"

typedef float floatx16 __attribute__((ext_vector_type(16)));

/* key (within a 32-key tile) that accumulator register r of lane half h holds */
__device__ __forceinline__ constexpr uint32_t acc_key(uint32_t r, uint32_t h) { return 8u * (r >> 2) + 4u * h + (r & 3u); }

constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;

/* 2^x on the transcendental unit; 2^(-inf) = 0 */
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

/* where a workgroup finds its problem */
enum : int {
    SRC_TILES = 0,  /* device arrays: tiles[blockIdx.x] -> probs[tile.prob]           */
    SRC_SINGLE = 1, /* one problem in the kernel arguments                            */
    SRC_AFFINE = 2  /* kernel arguments: first problem + (sequence, head) strides     */
};

/* Problem `prob` of a strided batch.  Field by field: a whole-struct copy
 * that is then edited ends up in scratch memory. */
__device__ __forceinline__ void affine_problem(AttnProb &p, const AttnAffine &aff, uint32_t prob, bool dense) {
    const int64_t sq = prob / aff.heads, hh = prob % aff.heads;
    const AttnProb &f = aff.first;
    p.q = f.q + (sq * aff.q_seq + hh * aff.q_head);
    p.k = f.k + (sq * aff.k_seq + hh * aff.k_head);
    p.v = f.v + (sq * aff.v_seq + hh * aff.v_head);
    p.out = f.out + (sq * aff.o_seq + hh * aff.o_head);
    p.weights = f.weights ? f.weights + (sq * aff.w_seq + hh * aff.w_head) : nullptr;
    p.lse = f.lse ? f.lse + (sq * aff.lse_seq + hh * aff.lse_head) : nullptr;
    p.mask = dense ? f.mask + (sq * aff.mask_seq + hh * aff.mask_head) : nullptr;
    const bool ranged = f.vis == ATTN_VIS_RANGE;
    p.row_lo = ranged ? f.row_lo + (sq * aff.range_seq + hh * aff.range_head) : nullptr;
    p.row_hi = ranged ? f.row_hi + (sq * aff.range_seq + hh * aff.range_head) : nullptr;
    p.q_stride = f.q_stride, p.k_stride = f.k_stride, p.v_stride = f.v_stride, p.out_stride = f.out_stride;
    p.nq = f.nq, p.nk = f.nk, p.hd = f.hd, p.vis = f.vis;
    p.causal_off = f.causal_off, p.window = f.window, p.scale = f.scale, p.flags = f.flags;
    p.range_span = f.range_span;
    p.reserved1 = 0;
}

/* Keys any of the query rows [first, last] can see, [tlo, thi), and keys all
 * of them see, [flo, fhi), for problems whose row ranges are closed-form
 * (everything but ATTN_VIS_RANGE).  Both ends of a row's range grow with the
 * row index and an empty row is followed by empty rows only, so the first
 * and the last row bound the span.  thi <= tlo: no row sees anything. */
__device__ __forceinline__ void span_key_bounds(const AttnProb &p, uint32_t first, uint32_t last, uint32_t &tlo,
                                                uint32_t &thi, uint32_t &flo, uint32_t &fhi) {
    uint32_t lo_a, hi_a, lo_b, hi_b;
    row_key_range(p, first, lo_a, hi_a);
    row_key_range(p, last, lo_b, hi_b);
    if (hi_a > lo_a) tlo = lo_a, thi = hi_b;
    else tlo = 0xFFFFFFFFu, thi = 0u;
    flo = lo_b, fhi = hi_a;
}

#endif /* FBLT_AMD_ATTN_TILE_H */
