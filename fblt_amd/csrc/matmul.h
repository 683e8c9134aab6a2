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
    float *out;
    const float *rope_cos;
    const float *rope_sin;
    uint32_t m, k, n;
    uint32_t lda, ldb, ldo;
    uint32_t rope_cols, head_dim;
};

void matmul_f32_launch(const MatmulArgs &g, hipStream_t s);

#endif
