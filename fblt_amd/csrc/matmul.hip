/*
 * fp32 matrix product out[M,N] = a[M,K] * b[K,N] (row-major), the projection
 * GEMMs either side of the attention core (reference contract:
 * csrc/ops/matmul.h, CPU loop csrc/ops/linalg_cpu.c:8-18, device twin
 * csrc/ops/linalg.cu:48-134).
 *
 * Three kernels:
 *
 *  - "skinny" (M <= 32: the n new rows of a decode / verify step): one thread
 *    per output column, the column of b read coalesced across the wave, the
 *    rows of a through the scalar cache; every output is the reference's own
 *    sum -- k ascending, product and sum rounded separately -- so this path
 *    is bit-identical to blt_matmul_cpu.
 *
 *  - "mfma" (everything else): 64x64 output tiles per workgroup of four
 *    wavefronts, K in steps of 32 through double-buffered LDS tiles,
 *    v_mfma_f32_32x32x2_f32 accumulation.  The product is accumulated
 *    TRANSPOSED (MFMA A operand = b tile, B operand = a tile), which puts one
 *    output ROW in each lane with four consecutive columns per register
 *    group: rows are stored with 16-byte stores, and an optional epilogue can
 *    rotate (column 2i, column 2i+1) pairs lane-locally -- the rotary position
 *    embedding of the Q and K blocks of a packed QKV projection
 *    (csrc/models/attention.c:76-90) -- without a second pass over the
 *    result.  Summation order differs from the reference's (fp32 tolerance).
 *
 *  - "splitk" (outputs too small to give every compute unit a 64x64 tile,
 *    e.g. 512x128 * 128x384): one 32x32 output tile per workgroup, its four
 *    wavefronts take the 32-wide K chunks round-robin straight from global
 *    memory (no LDS staging, no barrier in the loop) and add their partial
 *    tiles through LDS at the end.  Same accumulator layout and epilogue as
 *    the mfma kernel; the serial MFMA chain per wave is a quarter as long and
 *    there are four times as many workgroups.
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "launch.h"
#include "matmul.h"

#include <stdint.h>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TM = 64, TN = 64, TK = 32;
constexpr int A_PITCH = TK + 4; /* floats per LDS row of the a tile: 16-byte fragment reads of 32 rows hit all banks */
constexpr int B_PITCH = TN + 4;

/* VEC: a, b 16-byte aligned with lda, ldb, K, N multiples of 4, so a 16-byte
 * piece is either entirely inside or entirely outside the matrices.
 * ROPE: rotate pairs of the first g.rope_cols columns in the epilogue. */
template <bool VEC, bool ROPE>
__global__ __launch_bounds__(256, 2) void matmul_mfma_kernel(MatmulArgs g) {
    __shared__ __attribute__((aligned(16))) float sa[2][TM * A_PITCH];
    __shared__ __attribute__((aligned(16))) float sb[2][TK * B_PITCH];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5, c = lane & 31u;
    const uint32_t wr = wave >> 1, wc = wave & 1u; /* wave's 32x32 quadrant of the tile */
    const uint32_t row0 = blockIdx.y * TM, col0 = blockIdx.x * TN;

    /* pieces of 4 floats this thread moves per K step: two of the a tile, two of the b tile */
    float pa[2][4], pb[2][4];
    auto request = [&](uint32_t k0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const uint32_t e = threadIdx.x + 256u * u;
            {
                const uint32_t r = row0 + e / (TK / 4), k = k0 + 4u * (e % (TK / 4));
                const float *src = g.a + (size_t)min(r, g.m - 1u) * g.lda + k;
                if (VEC) {
                    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (k < g.k) t = *reinterpret_cast<const float4 *>(src);
                    pa[u][0] = t.x, pa[u][1] = t.y, pa[u][2] = t.z, pa[u][3] = t.w;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) pa[u][i] = k + i < g.k ? src[i] : 0.f;
                }
            }
            {
                const uint32_t k = k0 + e / (TN / 4), col = col0 + 4u * (e % (TN / 4));
                const float *src = g.b + (size_t)min(k, g.k - 1u) * g.ldb + col;
                if (VEC) {
                    float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                    if (k < g.k && col < g.n) t = *reinterpret_cast<const float4 *>(src);
                    pb[u][0] = t.x, pb[u][1] = t.y, pb[u][2] = t.z, pb[u][3] = t.w;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) pb[u][i] = (k < g.k && col + i < g.n) ? src[i] : 0.f;
                }
            }
        }
    };
    auto park = [&](uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < 2; u++) {
            const uint32_t e = threadIdx.x + 256u * u;
            *reinterpret_cast<float4 *>(&sa[buf][(e / (TK / 4)) * A_PITCH + 4u * (e % (TK / 4))]) =
                make_float4(pa[u][0], pa[u][1], pa[u][2], pa[u][3]);
            *reinterpret_cast<float4 *>(&sb[buf][(e / (TN / 4)) * B_PITCH + 4u * (e % (TN / 4))]) =
                make_float4(pb[u][0], pb[u][1], pb[u][2], pb[u][3]);
        }
    };

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;

    const uint32_t steps = (g.k + TK - 1u) / TK;
    request(0);
    park(0);
    __syncthreads();
    for (uint32_t s = 0; s < steps; s++) {
        const uint32_t buf = s & 1u;
        if (s + 1u < steps) request((s + 1u) * TK);
        /* MFMA A operand (rows of D = output columns): b[k][col], k = 16*h + t
         * MFMA B operand (columns of D = output rows):  a[row][k]            */
        const float *ar = &sa[buf][(wr * 32u + c) * A_PITCH + 16u * h];
        const float *bc = &sb[buf][(16u * h) * B_PITCH + wc * 32u + c];
#pragma unroll
        for (int t4 = 0; t4 < 16; t4 += 4) {
            const float4 av = *reinterpret_cast<const float4 *>(ar + t4);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bc[(t4 + 0) * B_PITCH], av.x, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bc[(t4 + 1) * B_PITCH], av.y, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bc[(t4 + 2) * B_PITCH], av.z, acc, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(bc[(t4 + 3) * B_PITCH], av.w, acc, 0, 0, 0);
        }
        if (s + 1u < steps) park(buf ^ 1u);
        __syncthreads();
    }

    /* lane (h, c) holds out[row0 + 32*wr + c][col0 + 32*wc + 8*q + 4*h + 0..3] in acc[4q..4q+3] */
    const uint32_t row = row0 + wr * 32u + c;
    if (row >= g.m) return;
    float *orow = g.out + (size_t)row * g.ldo;
    const bool vst = VEC && (g.ldo % 4u == 0u) && ((reinterpret_cast<uintptr_t>(g.out) & 15u) == 0u);
#pragma unroll
    for (int q = 0; q < 4; q++) {
        const uint32_t col = col0 + wc * 32u + 8u * q + 4u * h;
        float4 v = make_float4(acc[4 * q + 0], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3]);
        if (ROPE && col < g.rope_cols) {
            /* columns col..col+3 are pairs (col % head_dim)/2 and the next one of the row's position */
            const size_t at = (size_t)row * (g.head_dim / 2u) + (col % g.head_dim) / 2u;
            v = rope_rotate4(v, g.rope_cos + at, g.rope_sin + at);
        }
        if (vst) {
            if (col < g.n) *reinterpret_cast<float4 *>(orow + col) = v;
        } else {
            if (col + 0 < g.n) orow[col + 0] = v.x;
            if (col + 1 < g.n) orow[col + 1] = v.y;
            if (col + 2 < g.n) orow[col + 2] = v.z;
            if (col + 3 < g.n) orow[col + 3] = v.w;
        }
    }
}

/* 32x32 output tile per workgroup, K split over the four waves. */
template <bool VEC, bool ROPE>
__global__ __launch_bounds__(256, 2) void matmul_splitk_kernel(MatmulArgs g) {
    __shared__ float part[4][16][64];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5, c = lane & 31u;
    const uint32_t row = blockIdx.y * 32u + c, col = blockIdx.x * 32u + c;
    const float *arow = g.a + (size_t)min(row, g.m - 1u) * g.lda;
    const float *bcol = g.b + min(col, g.n - 1u);

    /* fragments of one 32-wide K chunk: lane (h, c) holds a[row][k0 + 16h + t] and b[k0 + 16h + t][col] */
    auto fetch = [&](uint32_t k0, float (&fa)[16], float (&fb)[16]) __attribute__((always_inline)) {
        const uint32_t kb = k0 + 16u * h;
        if (VEC) {
#pragma unroll
            for (int t = 0; t < 16; t += 4) {
                float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
                if (kb + t < g.k) v = *reinterpret_cast<const float4 *>(arow + kb + t);
                fa[t + 0] = v.x, fa[t + 1] = v.y, fa[t + 2] = v.z, fa[t + 3] = v.w;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 16; t++) fa[t] = kb + t < g.k ? arow[kb + t] : 0.f;
        }
#pragma unroll
        for (int t = 0; t < 16; t++) fb[t] = kb + t < g.k ? bcol[(size_t)(kb + t) * g.ldb] : 0.f;
    };

    floatx16 acc;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f;
    const uint32_t chunks = (g.k + 31u) / 32u;
    float fa[16], fb[16];
    uint32_t ch = wave;
    if (ch < chunks) fetch(ch * 32u, fa, fb);
    while (ch < chunks) {
        const uint32_t nx = ch + 4u;
        float na[16], nb[16];
        if (nx < chunks) fetch(nx * 32u, na, nb);
#pragma unroll
        for (int t = 0; t < 16; t++) acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[t], fa[t], acc, 0, 0, 0);
#pragma unroll
        for (int t = 0; t < 16; t++) fa[t] = na[t], fb[t] = nb[t];
        ch = nx;
    }

#pragma unroll
    for (int r = 0; r < 16; r++) part[wave][r][lane] = acc[r];
    __syncthreads();
    /* wave w finishes register group w: out[row][col0 + 8w + 4h + 0..3] */
    float v4[4];
#pragma unroll
    for (int i = 0; i < 4; i++)
        v4[i] = (part[0][4 * wave + i][lane] + part[1][4 * wave + i][lane]) +
                (part[2][4 * wave + i][lane] + part[3][4 * wave + i][lane]);
    if (row >= g.m) return;
    const uint32_t oc = blockIdx.x * 32u + 8u * wave + 4u * h;
    float4 v = make_float4(v4[0], v4[1], v4[2], v4[3]);
    if (ROPE && oc < g.rope_cols) {
        const size_t at = (size_t)row * (g.head_dim / 2u) + (oc % g.head_dim) / 2u;
        v = rope_rotate4(v, g.rope_cos + at, g.rope_sin + at);
    }
    float *orow = g.out + (size_t)row * g.ldo;
    if (VEC && (g.ldo % 4u == 0u) && ((reinterpret_cast<uintptr_t>(g.out) & 15u) == 0u)) {
        if (oc < g.n) *reinterpret_cast<float4 *>(orow + oc) = v;
    } else {
        if (oc + 0 < g.n) orow[oc + 0] = v.x;
        if (oc + 1 < g.n) orow[oc + 1] = v.y;
        if (oc + 2 < g.n) orow[oc + 2] = v.z;
        if (oc + 3 < g.n) orow[oc + 3] = v.w;
    }
}

/* R rows of a per thread, one output column per thread. */
template <int R>
__global__ __launch_bounds__(256) void matmul_skinny_kernel(MatmulArgs g) {
#pragma clang fp contract(off) /* product and sum rounded separately, as the reference's loop */
    const uint32_t j = blockIdx.x * 256u + threadIdx.x;
    const uint32_t r0 = blockIdx.y * R;
    if (j >= g.n) return;
    float acc[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f;
    for (uint32_t k = 0; k < g.k; k++) {
        const float bj = g.b[(size_t)k * g.ldb + j];
#pragma unroll
        for (int r = 0; r < R; r++) {
            const uint32_t row = min(r0 + r, g.m - 1u);
            acc[r] = acc[r] + g.a[(size_t)row * g.lda + k] * bj;
        }
    }
#pragma unroll
    for (int r = 0; r < R; r++)
        if (r0 + r < g.m) g.out[(size_t)(r0 + r) * g.ldo + j] = acc[r];
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

} // namespace

void matmul_f32_launch(const MatmulArgs &g, hipStream_t s) {
    if (g.m == 0 || g.n == 0) return;
    const bool rope = g.rope_cos != nullptr && g.rope_cols > 0;
    if (g.m <= 32u && !rope) {
        const dim3 block(256);
        if (g.m <= 4u) {
            blt_launch("matmul_skinny", matmul_skinny_kernel<4>, dim3((g.n + 255u) / 256u, 1), block, 0, s, g);
        } else {
            blt_launch("matmul_skinny", matmul_skinny_kernel<8>, dim3((g.n + 255u) / 256u, (g.m + 7u) / 8u), block, 0,
                       s, g);
        }
        return;
    }
    const dim3 grid((g.n + TN - 1) / TN, (g.m + TM - 1) / TM), block(256);
    const bool vec = aligned16(g.a) && aligned16(g.b) && g.lda % 4u == 0 && g.ldb % 4u == 0 && g.k % 4u == 0 &&
                     g.n % 4u == 0;
    if ((uint64_t)grid.x * grid.y < 128u) {
        /* fewer 64x64 tiles than half the compute units: quarter tiles, K split over the waves */
        const dim3 sgrid((g.n + 31u) / 32u, (g.m + 31u) / 32u);
        if (rope) {
            if (vec) blt_launch("matmul_splitk", matmul_splitk_kernel<true, true>, sgrid, block, 0, s, g);
            else blt_launch("matmul_splitk", matmul_splitk_kernel<false, true>, sgrid, block, 0, s, g);
        } else {
            if (vec) blt_launch("matmul_splitk", matmul_splitk_kernel<true, false>, sgrid, block, 0, s, g);
            else blt_launch("matmul_splitk", matmul_splitk_kernel<false, false>, sgrid, block, 0, s, g);
        }
        return;
    }
    if (rope) {
        if (vec) blt_launch("matmul_mfma", matmul_mfma_kernel<true, true>, grid, block, 0, s, g);
        else blt_launch("matmul_mfma", matmul_mfma_kernel<false, true>, grid, block, 0, s, g);
    } else {
        if (vec) blt_launch("matmul_mfma", matmul_mfma_kernel<true, false>, grid, block, 0, s, g);
        else blt_launch("matmul_mfma", matmul_mfma_kernel<false, false>, grid, block, 0, s, g);
    }
}

extern "C" void blt_matmul_hip(const blt_tensor *a, const blt_tensor *b, blt_tensor *out) {
    BLT_REQUIRE(a != NULL && b != NULL && out != NULL, "matmul: inputs must not be NULL");
    BLT_REQUIRE(a->ndim == 2 && b->ndim == 2 && out->ndim == 2, "matmul: all tensors must be 2D");
    BLT_REQUIRE(a->backend == BLT_BACKEND_HIP && b->backend == BLT_BACKEND_HIP && out->backend == BLT_BACKEND_HIP,
                "matmul: HIP implementation called with a non-HIP tensor");
    BLT_REQUIRE(a->dtype == BLT_DTYPE_FP32 && b->dtype == BLT_DTYPE_FP32,
                "matmul: the HIP backend takes FP32 operands only (BF16 weights are not supported)");
    BLT_REQUIRE(out->dtype == BLT_DTYPE_FP32, "matmul: output must be FP32");
    BLT_REQUIRE(a->shape[1] == b->shape[0], "matmul inner dimensions do not match");
    BLT_REQUIRE(out->shape[0] == a->shape[0] && out->shape[1] == b->shape[1], "matmul output shape is incorrect");
    const size_t m = a->shape[0], k = a->shape[1], n = b->shape[1];
    if (m == 0 || k == 0 || n == 0) return;
    BLT_REQUIRE(m <= 0x7FFFFFFFu && k <= 0x7FFFFFFFu && n <= 0x7FFFFFFFu, "matmul: dimensions exceed 2^31-1");
    MatmulArgs g;
    __builtin_memset(&g, 0, sizeof(g));
    g.a = (const float *)a->data;
    g.b = (const float *)b->data;
    g.out = (float *)out->data;
    g.m = (uint32_t)m, g.k = (uint32_t)k, g.n = (uint32_t)n;
    g.lda = (uint32_t)k, g.ldb = (uint32_t)n, g.ldo = (uint32_t)n;
    matmul_f32_launch(g, 0);
    HIP_CHECK_LAUNCH("blt_matmul");
}
