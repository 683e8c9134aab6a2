/* Launch interface of the fp32 matrix product kernels (matmul.hip). */
#ifndef FBLT_AMD_MATMUL_H
#define FBLT_AMD_MATMUL_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "rope_device.h"

/* out[m, n] = a[m, k] * b[k, n], leading dimensions in elements.  With
 * rope_cos / rope_sin set ([m, head_dim/2] tables, row r = position of output
 * row r), pairs (2i, 2i+1) of every head_dim-wide block of the first
 * rope_cols output columns are rotated before they are stored; head_dim and
 * rope_cols must be multiples of 4. */
struct MatmulArgs {
    const float *a;
    const float *b;
    const float *b2;       /* optional second weight matrix [k, n] (same ldb): out = silu(a*b2) .* (a*b), the gated
                              feed-forward activation (csrc/ops/elementwise_cpu.c:86-99) in one pass          */
    float *out2;           /* with b2: store a*b2 here (same ldo) instead of gating the first product with it  */
    const float *residual; /* optional [m, n] (leading dimension ldo) added to the result                     */
    const float *norm_w;   /* optional [k]: the rows of a are RMS-normalised with this weight first, i.e. the
                              product is taken of blt_rmsnorm_forward(a, norm_w) (csrc/ops/reductions_cpu.c:
                              327-352) without materialising it; the row statistic is accumulated from the
                              same loads (fp32 tolerance: the scale is applied after the product)              */
    float *out;
    const float *rope_cos;
    const float *rope_sin;
    uint32_t m, k, n;
    uint32_t lda, ldb, ldo;
    uint32_t rope_cols, head_dim;
    /* Optional cross-attention epilogue (matmul_takes_cross): the product is the query projection
     * of a cross block with heads cross_head_dim wide; instead of being stored, each projected row
     * attends, head by head, over the sub-tokens [cross_lo[row], cross_hi[row]) of its sequence's
     * tier-2 slab (sequence = row / cross_rows_per_seq) and the weighted V row goes to
     * cross_out[row, head columns] (csrc/infer/kv_cache.c:303-324).  More than 32 rows: split-K
     * kernel, 32-wide heads (a 32x32 output tile is one head of 32 rows).  Up to 32 rows: the exact
     * kernel with n <= 256, whose single workgroup per row group holds whole projected rows.
     * out may be null. */
    const float *cross_k;
    const float *cross_v;
    float *cross_out;
    const uint32_t *cross_lo;
    const uint32_t *cross_hi;
    uint32_t cross_rows_per_seq, cross_slab_rows, cross_head_dim;
    float cross_scale;
    /* Products of up to 32 rows normally run on the thread-per-column kernel, whose sums follow the
     * reference's order (bit-identical results) at the price of a serial chain of k additions.
     * tolerant != 0: the caller accepts fp32-tolerance results for such shapes too, and they go to
     * the matrix cores with K split over the waves (the whole decoder step sets it: a one-row
     * step takes 72 us instead of 112). */
    uint32_t tolerant;
    /* Set by the launcher, never by callers.  slices > 1: the K range is also split over slices
     * workgroups per output tile (grid z); each leaves its 32x32 sums in slice_sums
     * [tile][slice][1024] and the one that draws the last of the tile's tickets adds them in slice
     * order and runs the epilogue. */
    uint32_t slices;
    float *slice_sums;
    uint32_t *slice_tickets;
};

void matmul_f32_launch(const MatmulArgs &g, hipStream_t s);
/* g0 (plain) and g1 (two weight matrices, two outputs) in one launch; only when matmul_pair_ok says so */
bool matmul_pair_ok(const MatmulArgs &g0, const MatmulArgs &g1);
void matmul_f32_launch_pair(const MatmulArgs &g0, const MatmulArgs &g1, hipStream_t s);
/* b2 is only implemented by the kernels for small outputs; false = run the two products and the activation apart */
bool matmul_takes_gated(const MatmulArgs &g);
/* the cross-attention epilogue for this shape and g.cross_head_dim, no other epilogue set */
bool matmul_takes_cross(const MatmulArgs &g);
/* norm_w likewise */
bool matmul_takes_norm(const MatmulArgs &g);

#endif
