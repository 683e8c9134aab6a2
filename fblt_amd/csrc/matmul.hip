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
 *    wavefronts (128x128, four MFMA tiles per wavefront, once there are 512
 *    such tiles), K in steps of 32 (16) through double-buffered LDS tiles,
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
#include "cross_rows_device.h"

#include <stdint.h>
#include <stdlib.h>

#include <algorithm>
#include <map>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int TM = 64, TN = 64, TK = 32; /* smallest workgroup tile of the mfma kernel */

__device__ __forceinline__ float silu_times(float gate, float up) {
    const float silu = gate / (1.0f + expf(-gate));
    return silu * up;
}

/* Four consecutive results of output row `row` starting at column `col`:
 * optional rotation, optional residual, store with bounds. */
template <bool ROPE>
__device__ __forceinline__ void store4(const MatmulArgs &g, uint32_t row, uint32_t col, float4 v, bool vec_ok) {
    if (ROPE && col < g.rope_cols) {
        /* columns col..col+3 are pairs (col % head_dim)/2 and the next one of the row's position */
        const size_t at = (size_t)row * (g.head_dim / 2u) + (col % g.head_dim) / 2u;
        v = rope_rotate4(v, g.rope_cos + at, g.rope_sin + at);
    }
    float *orow = g.out + (size_t)row * g.ldo;
    const float *rrow = g.residual ? g.residual + (size_t)row * g.ldo : nullptr;
    if (vec_ok) {
        if (col < g.n) {
            if (rrow) {
                const float4 r = *reinterpret_cast<const float4 *>(rrow + col);
                v.x = r.x + v.x, v.y = r.y + v.y, v.z = r.z + v.z, v.w = r.w + v.w;
            }
            *reinterpret_cast<float4 *>(orow + col) = v;
        }
    } else {
        const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; i++)
            if (col + i < g.n) orow[col + i] = rrow ? rrow[col + i] + e[i] : e[i];
    }
}

/* One (64*WT)x(64*WT) output tile per workgroup of four wavefronts; each wave owns a quadrant of
 * WT x WT MFMA tiles.  WT = 2 is for products large enough to give every compute unit several
 * 128x128 tiles: a fragment read from LDS then feeds two matrix instructions, the four
 * accumulators of a wave are independent, and operands come from L2 half as often.
 * K in steps of 32/WT through double-buffered LDS tiles.
 * VEC: a, b 16-byte aligned with lda, ldb, K, N multiples of 4, so a 16-byte
 * piece is either entirely inside or entirely outside the matrices.
 * ROPE: rotate pairs of the first g.rope_cols columns in the epilogue. */
template <int WT, int NW>
struct MfmaShape {
    static constexpr int BM = TM * WT, BN = TN * WT, BK = TK / WT, THREADS = 64 * NW;
    static constexpr int AP = BK + 4; /* floats per LDS row of the a tile: 16-byte fragment reads of 32 rows hit all banks */
    static constexpr int BP = BN + 4;
    static constexpr int NP = BM * BK / 4 / THREADS; /* 16-byte pieces of each tile a thread moves per step */
    static constexpr int KW = BK / 2 / (NW / 4);     /* k values of a step per half of a wave */
    static constexpr size_t LDS_BYTES = (2 * BM * AP + 2 * BK * BP) * sizeof(float);
    static_assert(BM * BK == BK * BN && NP * 4 * THREADS == BM * BK, "a thread moves the same number of pieces of both tiles");
    static_assert(NW == 4 || (NW == 8 && WT == 1), "eight waves: the small tile only");
    static_assert(NW == 4 || 4 * 16 * 64 * sizeof(float) <= LDS_BYTES, "the second group's sums pass through the tile buffers");
};

/* NW = 8 (small tile): a second group of four waves takes the other half of every K step, so each
 * SIMD holds two waves of the workgroup and one's waits (LDS, memory, barrier) fall into the
 * other's matrix instructions; with one workgroup per compute unit and four waves those waits
 * left the matrix cores idle 46 % of the time.  The groups' sums meet in LDS at the end. */
template <bool VEC, bool ROPE, int WT, int NW = 4>
__global__ __launch_bounds__(64 * NW, 2) void matmul_mfma_kernel(MatmulArgs g) {
    using Shape = MfmaShape<WT, NW>;
    constexpr int BM = Shape::BM, BN = Shape::BN, BK = Shape::BK, KW = Shape::KW, NP = Shape::NP;
    constexpr int AP = Shape::AP, BP = Shape::BP, THREADS = Shape::THREADS;
    extern __shared__ __attribute__((aligned(16))) float mm_lds[];
    float (*sa)[BM * AP] = reinterpret_cast<float (*)[BM * AP]>(mm_lds);
    float (*sb)[BK * BP] = reinterpret_cast<float (*)[BK * BP]>(mm_lds + 2 * BM * AP);

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5, c = lane & 31u;
    const uint32_t wr = (wave & 3u) >> 1, wc = wave & 1u; /* wave's quadrant of the tile */
    const uint32_t kg = wave >> 2;                         /* its half of a K step (eight waves) */
    const uint32_t row0 = blockIdx.y * BM, col0 = blockIdx.x * BN;

    /* pieces of 4 floats this thread moves per K step: NP of the a tile, NP of the b tile.
     * Loads go to clamped addresses and land in registers untouched; pieces outside the matrices
     * are zeroed only when they are parked in LDS, after the step's matrix instructions, so that
     * nothing between the requests and those instructions waits for memory. */
    auto request = [&](float (&pa)[NP][4], float (&pb)[NP][4], uint32_t k0) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NP; u++) {
            const uint32_t e = threadIdx.x + (uint32_t)THREADS * u;
            {
                const uint32_t r = row0 + e / (BK / 4), k = k0 + 4u * (e % (BK / 4));
                const float *src = g.a + (size_t)min(r, g.m - 1u) * g.lda;
                if (VEC) {
                    const float4 t = *reinterpret_cast<const float4 *>(src + min(k, g.k - 4u));
                    pa[u][0] = t.x, pa[u][1] = t.y, pa[u][2] = t.z, pa[u][3] = t.w;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) pa[u][i] = src[min(k + i, g.k - 1u)];
                }
            }
            {
                const uint32_t k = k0 + e / (BN / 4), col = col0 + 4u * (e % (BN / 4));
                const float *src = g.b + (size_t)min(k, g.k - 1u) * g.ldb;
                if (VEC) {
                    const float4 t = *reinterpret_cast<const float4 *>(src + min(col, g.n - 4u));
                    pb[u][0] = t.x, pb[u][1] = t.y, pb[u][2] = t.z, pb[u][3] = t.w;
                } else {
#pragma unroll
                    for (int i = 0; i < 4; i++) pb[u][i] = src[min(col + i, g.n - 1u)];
                }
            }
        }
    };
    auto park = [&](const float (&pa)[NP][4], const float (&pb)[NP][4], uint32_t buf, uint32_t k0)
                    __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < NP; u++) {
            const uint32_t e = threadIdx.x + (uint32_t)THREADS * u;
            const uint32_t ka = k0 + 4u * (e % (BK / 4));
            const uint32_t kb = k0 + e / (BN / 4), col = col0 + 4u * (e % (BN / 4));
            float va[4], vb[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                va[i] = (VEC ? ka : ka + i) < g.k ? pa[u][i] : 0.f;
                vb[i] = (kb < g.k && (VEC ? col : col + i) < g.n) ? pb[u][i] : 0.f;
            }
            *reinterpret_cast<float4 *>(&sa[buf][(e / (BK / 4)) * AP + 4u * (e % (BK / 4))]) =
                make_float4(va[0], va[1], va[2], va[3]);
            *reinterpret_cast<float4 *>(&sb[buf][(e / (BN / 4)) * BP + 4u * (e % (BN / 4))]) =
                make_float4(vb[0], vb[1], vb[2], vb[3]);
        }
    };

    floatx16 acc[WT][WT];
#pragma unroll
    for (int i = 0; i < WT; i++)
#pragma unroll
        for (int j = 0; j < WT; j++)
#pragma unroll
            for (int r = 0; r < 16; r++) acc[i][j][r] = 0.f;

    /* Two register sets take turns: the pieces of step s+1 and s+2 are on their way while step s
     * runs, so a request has two steps of matrix work to arrive in (one step is less than the
     * memory latency when a wave is alone on its SIMD).  Requests and parks are unconditional --
     * addresses are clamped, pieces past K parked as zeros -- so that no load sits behind a branch
     * and no wait has to assume the worst at a join. */
    const uint32_t steps = (g.k + BK - 1u) / BK;
    float pa0[NP][4], pb0[NP][4], pa1[NP][4], pb1[NP][4];
    request(pa0, pb0, 0);
    request(pa1, pb1, BK);
    /* the requests keep the order they have in the loop (one whole set after the other): the wait
     * counts inside the loop are the worst case of both ways into it */
    __builtin_amdgcn_sched_barrier(0);
    park(pa0, pb0, 0, 0);
    request(pa0, pb0, 2u * BK);
    __syncthreads();
    auto step = [&](uint32_t s, float (&pa)[NP][4], float (&pb)[NP][4]) __attribute__((always_inline)) {
        /* (pa, pb) hold the pieces of step s+1 */
        const uint32_t buf = s & 1u;
        /* MFMA A operand (rows of D = output columns): b[k][col], k = KW*(2*kg + h) + t
         * MFMA B operand (columns of D = output rows):  a[row][k]                       */
        const float *ar = &sa[buf][(wr * (32u * WT) + c) * AP + KW * (2u * kg + h)];
        const float *bc = &sb[buf][(KW * (2u * kg + h)) * BP + wc * (32u * WT) + c];
        /* every fragment of the step is requested from LDS before its first matrix instruction:
         * read just in time, each pair of instructions waited for the next read */
        float av[WT][KW], bv[WT][KW];
#pragma unroll
        for (int t4 = 0; t4 < KW; t4 += 4) {
#pragma unroll
            for (int i = 0; i < WT; i++) {
                const float4 t = *reinterpret_cast<const float4 *>(ar + 32 * i * AP + t4);
                av[i][t4 + 0] = t.x, av[i][t4 + 1] = t.y, av[i][t4 + 2] = t.z, av[i][t4 + 3] = t.w;
            }
#pragma unroll
            for (int t = 0; t < 4; t++)
#pragma unroll
                for (int j = 0; j < WT; j++) bv[j][t4 + t] = bc[(t4 + t) * BP + 32 * j];
        }
        __builtin_amdgcn_sched_barrier(0); /* the compiler would sink the reads back between the instructions */
#pragma unroll
        for (int t = 0; t < KW; t++)
#pragma unroll
            for (int i = 0; i < WT; i++)
#pragma unroll
                for (int j = 0; j < WT; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j][t], av[i][t], acc[i][j], 0, 0, 0);
        park(pa, pb, buf ^ 1u, (s + 1u) * BK); /* past K this parks zeros in the buffer nobody reads again */
        request(pa, pb, (s + 3u) * BK);
        __syncthreads();
    };
    /* steps in pairs, one per register set; an odd count ends with a step over zeros */
    for (uint32_t s = 0; s < steps; s += 2u) {
        step(s, pa1, pb1);
        step(s + 1u, pa0, pb0);
    }

    if constexpr (NW == 8) { /* the loop ended on a barrier: the tile buffers are free */
        float *meet = mm_lds + (wave & 3u) * (16u * 64u);
        if (kg == 1u) {
#pragma unroll
            for (int r = 0; r < 16; r++) meet[r * 64 + lane] = acc[0][0][r];
        }
        __syncthreads();
        if (kg == 1u) return;
#pragma unroll
        for (int r = 0; r < 16; r++) acc[0][0][r] = acc[0][0][r] + meet[r * 64 + lane];
    }

    /* lane (h, c) holds out[row0 + 32*(WT*wr + i) + c][col0 + 32*(WT*wc + j) + 8*q + 4*h + 0..3] in acc[i][j][4q..4q+3] */
    const bool vst = VEC && (g.ldo % 4u == 0u) && ((reinterpret_cast<uintptr_t>(g.out) & 15u) == 0u) &&
                     ((reinterpret_cast<uintptr_t>(g.residual) & 15u) == 0u);
#pragma unroll
    for (int i = 0; i < WT; i++) {
        const uint32_t row = row0 + 32u * (WT * wr + i) + c;
        if (row >= g.m) continue;
#pragma unroll
        for (int j = 0; j < WT; j++)
#pragma unroll
            for (int q = 0; q < 4; q++)
                store4<ROPE>(g, row, col0 + 32u * (WT * wc + j) + 8u * q + 4u * h,
                             make_float4(acc[i][j][4 * q + 0], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2],
                                         acc[i][j][4 * q + 3]),
                             vst);
    }
}

/* 32x32 output tile (bx, by) per workgroup, K split over the NW waves (4, or 8 for long K:
 * the serial chain of chunk loads per wave halves); the first four waves finish the tile. */
template <bool VEC, bool ROPE, bool GATED, int NW = 4, bool CROSS = false>
__device__ __forceinline__ void splitk_tile(const MatmulArgs &g, const uint32_t bx, const uint32_t by,
                                            float (*part)[16][64], float (*part_ss)[32], float *qt = nullptr) {
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5, c = lane & 31u;
    const uint32_t row = by * 32u + c, col = bx * 32u + c;
    const float *arow = g.a + (size_t)min(row, g.m - 1u) * g.lda;
    const float *bcol = g.b + min(col, g.n - 1u);
    const float *b2col = GATED ? g.b2 + min(col, g.n - 1u) : nullptr;

    float ss = 0.f; /* this lane's share of sum_k a[row][k]^2 (norm_w only) */
    /* fragments of one 32-wide K chunk: lane (h, c) holds a[row][k0 + 16h + t] and b[k0 + 16h + t][col] */
    /* Every load of a chunk is issued before anything waits: addresses past K are clamped to the
     * last valid element and the value replaced by zero afterwards, so no load sits behind a
     * branch, and the norm arithmetic (which needs the a values) comes after the b requests. */
    auto fetch = [&](uint32_t k0, float (&fa)[16], float (&fb)[16], float (&fg)[16]) __attribute__((always_inline)) {
        const uint32_t kb = k0 + 16u * h;
        if (VEC) { /* K is a multiple of 4 here: a 16-byte piece is inside or outside as a whole */
#pragma unroll
            for (int t = 0; t < 16; t += 4) {
                const float4 v = *reinterpret_cast<const float4 *>(arow + min(kb + t, g.k - 4u));
                const bool in = kb + t < g.k;
                fa[t + 0] = in ? v.x : 0.f, fa[t + 1] = in ? v.y : 0.f;
                fa[t + 2] = in ? v.z : 0.f, fa[t + 3] = in ? v.w : 0.f;
            }
        } else {
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const float v = arow[min(kb + t, g.k - 1u)];
                fa[t] = kb + t < g.k ? v : 0.f;
            }
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            const float v = bcol[(size_t)min(kb + t, g.k - 1u) * g.ldb];
            fb[t] = kb + t < g.k ? v : 0.f;
        }
        if (GATED) {
#pragma unroll
            for (int t = 0; t < 16; t++) {
                const float v = b2col[(size_t)min(kb + t, g.k - 1u) * g.ldb];
                fg[t] = kb + t < g.k ? v : 0.f;
            }
        }
        if (g.norm_w) { /* uniform: sum of squares of the raw row, then the norm weight folded into a */
            float nw[16];
#pragma unroll
            for (int t = 0; t < 16; t++) nw[t] = g.norm_w[min(kb + t, g.k - 1u)];
#pragma unroll
            for (int t = 0; t < 16; t++) {
                ss += fa[t] * fa[t];
                fa[t] *= nw[t]; /* fa is already zero past K */
            }
        }
    };

    floatx16 acc, acc2;
#pragma unroll
    for (int r = 0; r < 16; r++) acc[r] = 0.f, acc2[r] = 0.f;
    uint32_t chunks = (g.k + 31u) / 32u, first = 0u;
    if (g.slices > 1u) { /* this workgroup's share of the chunks */
        const uint32_t per = (chunks + g.slices - 1u) / g.slices;
        first = min(blockIdx.z * per, chunks);
        chunks = min(first + per, chunks);
    }
    float fa[16], fb[16], fg[GATED ? 16 : 1];
    float dummy[GATED ? 1 : 16]; /* stands in for the gate fragment when there is none */
    (void)dummy;
    uint32_t ch = first + wave;
    if (ch < chunks) {
        if constexpr (GATED) fetch(ch * 32u, fa, fb, fg);
        else fetch(ch * 32u, fa, fb, dummy);
    }
    while (ch < chunks) {
        const uint32_t nx = ch + (uint32_t)NW;
        float na[16], nb[16], ng[GATED ? 16 : 1];
        if (nx < chunks) {
            if constexpr (GATED) fetch(nx * 32u, na, nb, ng);
            else fetch(nx * 32u, na, nb, dummy);
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[t], fa[t], acc, 0, 0, 0);
            if (GATED) acc2 = __builtin_amdgcn_mfma_f32_32x32x2f32(fg[t], fa[t], acc2, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 16; t++) {
            fa[t] = na[t], fb[t] = nb[t];
            if (GATED) fg[t] = ng[t];
        }
        ch = nx;
    }

#pragma unroll
    for (int r = 0; r < 16; r++) {
        part[wave][r][lane] = acc[r];
        if (GATED) part[NW + wave][r][lane] = acc2[r];
    }
    if (g.norm_w) {
        ss += __shfl_xor(ss, 32, 64);
        if (h == 0) part_ss[wave][c] = ss;
    }
    __syncthreads();
    if (NW > 4 && wave >= 4u) return; /* no barrier follows */
    float row_scale = 1.0f;
    if (g.norm_w) {
        float tot = (part_ss[0][c] + part_ss[1][c]) + (part_ss[2][c] + part_ss[3][c]);
        if (NW > 4) tot += (part_ss[4][c] + part_ss[5][c]) + (part_ss[6][c] + part_ss[7][c]);
        row_scale = 1.0f / sqrtf(tot / (float)g.k + 1e-6f); /* reductions_cpu.c:345-346 */
    }
    /* wave w < 4 finishes register group w: out[row][col0 + 8w + 4h + 0..3] */
    auto total = [&](uint32_t first, uint32_t reg) __attribute__((always_inline)) {
        float t = (part[first + 0][reg][lane] + part[first + 1][reg][lane]) +
                  (part[first + 2][reg][lane] + part[first + 3][reg][lane]);
        if (NW > 4)
            t += (part[first + 4][reg][lane] + part[first + 5][reg][lane]) +
                 (part[first + 6][reg][lane] + part[first + 7][reg][lane]);
        return t;
    };
    float v4[4], second[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        v4[i] = total(0u, 4u * wave + i) * row_scale;
        if (GATED) {
            const float gate = total((uint32_t)NW, 4u * wave + i) * row_scale;
            if (g.out2) second[i] = gate; /* two products, two outputs */
            else v4[i] = silu_times(gate, v4[i]);
        }
    }
    if (!GATED && !CROSS && g.slices > 1u) {
        /* Device-scope stores and loads, and an explicit wait for the stores' completion before the
         * barrier that precedes this workgroup's ticket, as for the split softmax states of the
         * KV step (kv_step.h).  The waves past the fourth have left. */
        __shared__ uint32_t ticket;
        const uint32_t tile = by * gridDim.x + bx;
        float *sums = g.slice_sums + (size_t)tile * g.slices * 1024u + 4u * threadIdx.x;
#pragma unroll
        for (int i = 0; i < 4; i++)
            __hip_atomic_store(sums + (size_t)blockIdx.z * 1024u + i, v4[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        blt_vector_memory_done(); /* every wave's sums are out before thread 0 draws the ticket */
        __syncthreads();
        if (threadIdx.x == 0)
            ticket = __hip_atomic_fetch_add(&g.slice_tickets[tile], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (ticket != g.slices - 1u) return;
        if (threadIdx.x == 0) g.slice_tickets[tile] = 0u; /* re-armed for the next launch */
#pragma unroll
        for (int i = 0; i < 4; i++) v4[i] = __hip_atomic_load(sums + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        for (uint32_t z = 1; z < g.slices; z++) /* slice order, whoever comes last */
#pragma unroll
            for (int i = 0; i < 4; i++)
                v4[i] += __hip_atomic_load(sums + (size_t)z * 1024u + i, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (CROSS) {
        /* The tile is the projected query of 32 rows for head bx: park it, then wave w takes rows
         * 8w .. 8w+7 with eight lanes per row (four columns each).  Softmax as
         * blt_softmax_masked_row_inplace: maximum over finite scores, non-finite scores weigh
         * nothing, an empty or all-dead row gives zeros (same statements as kv_cross_rows_kernel). */
#pragma unroll
        for (int i = 0; i < 4; i++) qt[c * 33u + 8u * wave + 4u * h + i] = v4[i];
        __syncthreads(); /* the waves past the fourth have left */
        const uint32_t rr = 8u * wave + (lane >> 3), s8 = lane & 7u;
        const uint32_t R = by * 32u + rr;
        if (R >= g.m) return;
        const float4 q4 = make_float4(qt[rr * 33u + 4u * s8], qt[rr * 33u + 4u * s8 + 1u], qt[rr * 33u + 4u * s8 + 2u],
                                      qt[rr * 33u + 4u * s8 + 3u]);
        const uint32_t lo = g.cross_lo[R], hi = g.cross_hi[R];
        const size_t base = (size_t)(R / g.cross_rows_per_seq) * g.cross_slab_rows * g.n + bx * 32u + 4u * s8;
        auto score = [&](uint32_t j) {
            const float4 k4 = *reinterpret_cast<const float4 *>(g.cross_k + base + (size_t)j * g.n);
            float p = q4.x * k4.x + q4.y * k4.y + q4.z * k4.z + q4.w * k4.w;
            p += __shfl_xor(p, 1, 64);
            p += __shfl_xor(p, 2, 64);
            p += __shfl_xor(p, 4, 64);
            return p * g.cross_scale;
        };
        float mx = -__builtin_huge_valf();
        for (uint32_t j = lo; j < hi; j++) {
            const float sc = score(j);
            if (isfinite(sc)) mx = fmaxf(mx, sc);
        }
        float sum = 0.f;
        float4 o4 = make_float4(0.f, 0.f, 0.f, 0.f);
        for (uint32_t j = lo; j < hi; j++) {
            const float sc = score(j);
            const float e = isfinite(sc) ? expf(sc - mx) : 0.f;
            if (e == 0.f) continue;
            sum += e;
            const float4 vv = *reinterpret_cast<const float4 *>(g.cross_v + base + (size_t)j * g.n);
            o4.x += e * vv.x, o4.y += e * vv.y, o4.z += e * vv.z, o4.w += e * vv.w;
        }
        const float inv = sum > 0.f ? 1.0f / sum : 0.f;
        *reinterpret_cast<float4 *>(g.cross_out + (size_t)R * g.n + bx * 32u + 4u * s8) =
            make_float4(o4.x * inv, o4.y * inv, o4.z * inv, o4.w * inv);
        return;
    }
    if (row >= g.m) return;
    const bool vst = VEC && (g.ldo % 4u == 0u) && ((reinterpret_cast<uintptr_t>(g.out) & 15u) == 0u) &&
                     ((reinterpret_cast<uintptr_t>(g.residual) & 15u) == 0u) &&
                     ((reinterpret_cast<uintptr_t>(g.out2) & 15u) == 0u);
    const uint32_t oc = bx * 32u + 8u * wave + 4u * h;
    store4<ROPE>(g, row, oc, make_float4(v4[0], v4[1], v4[2], v4[3]), vst);
    if (GATED && g.out2) {
        MatmulArgs g2 = g;
        g2.out = g.out2;
        g2.residual = nullptr;
        store4<false>(g2, row, oc, make_float4(second[0], second[1], second[2], second[3]), vst);
    }
}

template <bool VEC, bool ROPE, bool GATED, int NW = 4, bool CROSS = false>
__global__ __launch_bounds__(64 * NW, 2) void matmul_splitk_kernel(MatmulArgs g) {
    __shared__ float part[(GATED ? 2 : 1) * NW][16][64];
    __shared__ float part_ss[NW][32];
    __shared__ float qt[CROSS ? 32 * 33 : 1];
    splitk_tile<VEC, ROPE, GATED, NW, CROSS>(g, blockIdx.x, blockIdx.y, part, part_ss, qt);
}

/* Two independent products in one launch: the tile rows of the second are
 * stacked under those of the first (rows0 tile rows); the second may carry a
 * second weight matrix.  For pairs of small products whose launches would
 * otherwise each pay the fixed launch cost. */
template <bool VEC>
__global__ __launch_bounds__(256, 2) void matmul_splitk_pair_kernel(MatmulArgs g0, MatmulArgs g1, uint32_t rows0) {
    __shared__ float part[8][16][64];
    __shared__ float part_ss[4][32];
    if (blockIdx.y < rows0) { /* uniform per workgroup */
        if (blockIdx.x * 32u >= g0.n) return;
        splitk_tile<VEC, false, false>(g0, blockIdx.x, blockIdx.y, part, part_ss);
    } else {
        if (blockIdx.x * 32u >= g1.n) return;
        splitk_tile<VEC, false, true>(g1, blockIdx.x, blockIdx.y - rows0, part, part_ss);
    }
}

constexpr uint32_t SKINNY_KC = 512; /* k values of the a rows staged in LDS at a time */

/* One output column per thread, R rows of a per workgroup (grid.y walks the row groups).  Every
 * output is the reference's own sum: k ascending, product and sum rounded separately.  What the
 * kernel is built around is the latency of that serial chain: the rows of a sit in LDS (one
 * broadcast 16-byte read per four k), the column of b is fetched sixteen k ahead of the chain --
 * the requests of block t+1 are in flight while block t is summed -- and every row gets a thread
 * per column of its own (R = 1 at launch) rather than a share of a thread. */
template <int R, bool GATED, bool CROSS = false>
__global__ __launch_bounds__(256) void matmul_skinny_kernel(MatmulArgs g) {
#pragma clang fp contract(off) /* product and sum rounded separately, as the reference's loop */
    constexpr uint32_t KC = SKINNY_KC, UN = 16;
    __shared__ __attribute__((aligned(16))) float sa[R][KC];
    __shared__ float inv_rms[R];
    __shared__ float sq[CROSS ? R : 1][CROSS ? 256 : 1]; /* the projected rows, for the cross-attention epilogue */
    const uint32_t jj = blockIdx.x * 256u + threadIdx.x;
    const uint32_t j = min(jj, g.n - 1u);
    const uint32_t r0 = blockIdx.y * R;
    float acc[R], acc2[R];
#pragma unroll
    for (int r = 0; r < R; r++) acc[r] = 0.0f, acc2[r] = 0.0f;
    const float *bcol = g.b + j;
    const float *gcol = GATED ? g.b2 + j : nullptr;
    for (uint32_t kc = 0; kc < g.k; kc += KC) {
        const uint32_t klen = min(KC, g.k - kc);
        __syncthreads(); /* the previous chunk has been consumed */
        for (uint32_t t = threadIdx.x; t < R * KC; t += 256u) {
            const uint32_t r = t / KC, kk = t % KC;
            const uint32_t row = min(r0 + r, g.m - 1u);
            sa[r][kk] = g.a[(size_t)row * g.lda + kc + min(kk, klen - 1u)];
        }
        __syncthreads();
        if (g.norm_w) { /* uniform; the host sends such a product here only when k <= KC (one chunk) */
            /* the reference's row norm (csrc/ops/reductions_cpu.c:325-352) on the staged rows: sum of
             * squares in element order by one lane per row, then x * inv_rms * w element by element */
            if ((threadIdx.x & 63u) == 0 && (threadIdx.x >> 6) < (uint32_t)R) {
                const uint32_t r = threadIdx.x >> 6;
                float sumsq = 0.0f;
                uint32_t q = 0;
                for (; q + 4u <= klen; q += 4u) {
                    const float4 t = *reinterpret_cast<const float4 *>(&sa[r][q]);
                    sumsq = sumsq + t.x * t.x;
                    sumsq = sumsq + t.y * t.y;
                    sumsq = sumsq + t.z * t.z;
                    sumsq = sumsq + t.w * t.w;
                }
                for (; q < klen; q++) sumsq = sumsq + sa[r][q] * sa[r][q];
                inv_rms[r] = 1.0f / sqrtf(sumsq / (float)klen + 1e-6f);
            }
            __syncthreads();
            for (uint32_t t = threadIdx.x; t < R * KC; t += 256u) {
                const uint32_t r = t / KC, kk = t % KC;
                if (kk < klen) sa[r][kk] = sa[r][kk] * inv_rms[r] * g.norm_w[kk];
            }
            __syncthreads();
        }
        const uint32_t full = klen / UN * UN;
        if (full) {
            float bv[UN], gv[UN];
#pragma unroll
            for (uint32_t u = 0; u < UN; u++) {
                bv[u] = bcol[(size_t)(kc + u) * g.ldb];
                gv[u] = GATED ? gcol[(size_t)(kc + u) * g.ldb] : 0.0f;
            }
            for (uint32_t k0 = 0; k0 < full; k0 += UN) {
                /* the next block's column values (the last round fetches its own block again) */
                const uint32_t kn = kc + min(k0 + UN, full - UN);
                float nb[UN], ng[UN];
#pragma unroll
                for (uint32_t u = 0; u < UN; u++) {
                    nb[u] = bcol[(size_t)(kn + u) * g.ldb];
                    ng[u] = GATED ? gcol[(size_t)(kn + u) * g.ldb] : 0.0f;
                }
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (uint32_t u4 = 0; u4 < UN; u4 += 4) {
#pragma unroll
                    for (int r = 0; r < R; r++) {
                        const float4 a4 = *reinterpret_cast<const float4 *>(&sa[r][k0 + u4]);
                        const float av[4] = {a4.x, a4.y, a4.z, a4.w};
#pragma unroll
                        for (int t = 0; t < 4; t++) {
                            acc[r] = acc[r] + av[t] * bv[u4 + t];
                            if (GATED) acc2[r] = acc2[r] + av[t] * gv[u4 + t];
                        }
                    }
                }
#pragma unroll
                for (uint32_t u = 0; u < UN; u++) bv[u] = nb[u], gv[u] = ng[u];
            }
        }
        for (uint32_t k = full; k < klen; k++) {
            const float bj = bcol[(size_t)(kc + k) * g.ldb];
            const float gj = GATED ? gcol[(size_t)(kc + k) * g.ldb] : 0.0f;
#pragma unroll
            for (int r = 0; r < R; r++) {
                acc[r] = acc[r] + sa[r][k] * bj;
                if (GATED) acc2[r] = acc2[r] + sa[r][k] * gj;
            }
        }
    }
    if (CROSS) { /* one workgroup holds whole rows (n <= 256): a wave per (row, head) */
#pragma unroll
        for (int r = 0; r < R; r++) sq[r][threadIdx.x] = acc[r];
        __syncthreads();
        const uint32_t xhd = g.cross_head_dim, heads = g.n / xhd;
        for (uint32_t p = threadIdx.x >> 6; p < (uint32_t)R * heads; p += 4u) {
            const uint32_t r = p / heads, hh = p % heads, row = r0 + r;
            if (row >= g.m) continue;
            const size_t slab = (size_t)(row / g.cross_rows_per_seq) * g.cross_slab_rows * g.n + hh * xhd;
            cross_row_head(&sq[r][hh * xhd], g.cross_k + slab, g.cross_v + slab, g.cross_lo[row], g.cross_hi[row], g.n,
                           xhd, g.cross_scale, g.cross_out + (size_t)row * g.n + hh * xhd, threadIdx.x & 63u);
        }
        return;
    }
    if (jj >= g.n) return;
#pragma unroll
    for (int r = 0; r < R; r++) {
        if (r0 + r >= g.m) continue;
        float v = (GATED && !g.out2) ? silu_times(acc2[r], acc[r]) : acc[r];
        if (g.residual) v = g.residual[(size_t)(r0 + r) * g.ldo + j] + v;
        g.out[(size_t)(r0 + r) * g.ldo + j] = v;
        if (GATED && g.out2) g.out2[(size_t)(r0 + r) * g.ldo + j] = acc2[r];
    }
}

template <int R>
void launch_skinny(const MatmulArgs &g, hipStream_t s) {
    const dim3 grid((g.n + 255u) / 256u, (g.m + R - 1u) / R);
    if (g.cross_k) blt_launch("matmul_skinny_cross", matmul_skinny_kernel<R, false, true>, grid, dim3(256), 0, s, g);
    else if (g.b2) blt_launch("matmul_skinny", matmul_skinny_kernel<R, true>, grid, dim3(256), 0, s, g);
    else blt_launch("matmul_skinny", matmul_skinny_kernel<R, false>, grid, dim3(256), 0, s, g);
}

bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

} // namespace

namespace {

enum Path { PATH_SKINNY, PATH_SPLITK, PATH_MFMA };

Path choose_path(const MatmulArgs &g) {
    const bool rope = g.rope_cos != nullptr && g.rope_cols > 0;
    /* up to this many rows the thread-per-column kernel, whose sums run in the reference's order
     * (bit-identical results) */
    constexpr uint32_t exact_rows = 32u;
    if (g.m <= exact_rows && !rope && !g.tolerant) return PATH_SKINNY;
    /* up to 143 64x64 tiles (a bit over half the compute units): quarter tiles, K split over the
     * waves.  Measured at K = 512 ... 4096: a fifth faster than the 64x64 kernel at 128 tiles, level
     * with it at 144 ... 192, a quarter slower at 256 */
    constexpr uint64_t splitk_below = 144u;
    if ((uint64_t)((g.n + TN - 1) / TN) * ((g.m + TM - 1) / TM) < splitk_below) return PATH_SPLITK;
    return PATH_MFMA;
}

/* Sums and tickets of the K slices, per (thread, stream) like the scratch of the KV step: launches
 * on one stream follow each other, launches on two streams never share them. */
struct SliceScratch {
    float *sums = nullptr;
    size_t sum_floats = 0;
    uint32_t *tickets = nullptr;
    size_t ticket_count = 0;
};
__global__ void clear_words_kernel(uint32_t *w, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256u + threadIdx.x;
    if (i < n) w[i] = 0u;
}
/* false: the scratch would have to grow while a graph capture is open (the launch then runs unsliced) */
bool slice_scratch(MatmulArgs &g, size_t tiles, hipStream_t s) {
    static thread_local std::map<hipStream_t, SliceScratch> by_stream;
    SliceScratch &sc = by_stream[blt_stream_key()];
    const size_t floats = tiles * g.slices * 1024u;
    if (blt_stream_capturing() && (floats > sc.sum_floats || tiles > sc.ticket_count)) return false;
    /* outgrown buffers are left to the process: a launch still in flight may be using them */
    if (floats > sc.sum_floats) {
        sc.sum_floats = std::max(floats, 2 * sc.sum_floats);
        HIP_CHECK(hipMalloc((void **)&sc.sums, sc.sum_floats * sizeof(float)));
    }
    if (tiles > sc.ticket_count) {
        sc.ticket_count = std::max<size_t>(2 * tiles, 1024);
        HIP_CHECK(hipMalloc((void **)&sc.tickets, sc.ticket_count * sizeof(uint32_t)));
        /* a fill kernel, not a memset, on the stream the launches follow */
        hipLaunchKernelGGL(clear_words_kernel, dim3((unsigned)((sc.ticket_count + 255) / 256)), dim3(256), 0,
                           s ? s : blt_stream(), sc.tickets, sc.ticket_count);
    }
    g.slice_sums = sc.sums;
    g.slice_tickets = sc.tickets;
    return true;
}

/* Slices of K per output tile: long K over few tiles leaves most of the chip idle and every wave
 * with a serial chain of chunk loads (2048 x 512 weights under 118 rows: 64 tiles, eight chunks per
 * wave).  As many slices as keep one chunk per wave and give one workgroup per compute unit: measured
 * over 12 ... 256 tiles and K = 1024 ... 4096, the best count was the one that brought the launch
 * to about 256 workgroups, and more made it slower again. */
uint32_t slices_for(const MatmulArgs &g, dim3 grid, bool eight) {
    if (g.b2 || g.cross_k || g.norm_w) return 1u;
    const uint32_t chunks = (g.k + 31u) / 32u, tiles = grid.x * grid.y;
    const uint32_t room = chunks / (eight ? 8u : 4u);
    if (chunks < 32u || tiles > 128u) return 1u;
    return std::max(1u, std::min(room, 256u / tiles));
}

template <bool VEC, bool ROPE>
void launch_splitk(const MatmulArgs &g_in, dim3 grid, hipStream_t s) {
    /* eight waves once every wave still gets a chunk (K >= 256) and the launch leaves the chip room for them */
    const bool eight = g_in.k >= 256u && (uint64_t)grid.x * grid.y <= 512u;
    MatmulArgs g = g_in;
    g.slices = slices_for(g, grid, eight);
    if (g.slices > 1u && slice_scratch(g, (size_t)grid.x * grid.y, s)) grid.z = g.slices;
    else g.slices = 1u;
    if (g.cross_k) {
        if constexpr (VEC && !ROPE)
            blt_launch("matmul_splitk_cross", matmul_splitk_kernel<true, false, false, 4, true>, grid, dim3(256), 0, s, g);
        return;
    }
    if (g.b2) blt_launch("matmul_splitk", matmul_splitk_kernel<VEC, ROPE, true>, grid, dim3(256), 0, s, g);
    else if (eight) blt_launch("matmul_splitk", matmul_splitk_kernel<VEC, ROPE, false, 8>, grid, dim3(512), 0, s, g);
    else blt_launch("matmul_splitk", matmul_splitk_kernel<VEC, ROPE, false>, grid, dim3(256), 0, s, g);
}

} // namespace

bool matmul_takes_gated(const MatmulArgs &g) { return choose_path(g) != PATH_MFMA; }
bool matmul_takes_cross(const MatmulArgs &g) {
    if (g.b2 || g.residual || (g.rope_cos != nullptr && g.rope_cols > 0) || g.cross_head_dim == 0u ||
        g.n % g.cross_head_dim != 0u)
        return false;
    const Path path = choose_path(g);
    if (path == PATH_SKINNY) return g.n <= 256u && g.cross_head_dim <= 256u;
    return path == PATH_SPLITK && g.cross_head_dim == 32u && g.n % 32u == 0u && g.k % 4u == 0u;
}
bool matmul_takes_norm(const MatmulArgs &g) {
    const Path path = choose_path(g);
    return path == PATH_SPLITK || (path == PATH_SKINNY && g.k <= SKINNY_KC);
}

namespace {
bool vec_ok(const MatmulArgs &g) {
    return aligned16(g.a) && aligned16(g.b) && g.lda % 4u == 0 && g.ldb % 4u == 0 && g.k % 4u == 0 && g.n % 4u == 0;
}
} // namespace

bool matmul_pair_ok(const MatmulArgs &g0, const MatmulArgs &g1) {
    const auto plain = [](const MatmulArgs &g) {
        return g.m != 0 && g.n != 0 && g.k != 0 && g.m > 32u && choose_path(g) == PATH_SPLITK && !g.residual &&
               !(g.rope_cos != nullptr && g.rope_cols > 0);
    };
    /* the first product may normalise its rows on the way (four waves: the tile code's own sums) */
    return plain(g0) && plain(g1) && g0.b2 == nullptr && g1.b2 != nullptr && g1.out2 != nullptr && !g1.norm_w;
}

void matmul_f32_launch_pair(const MatmulArgs &g0, const MatmulArgs &g1, hipStream_t s) {
    BLT_REQUIRE(matmul_pair_ok(g0, g1), "matmul: this pair of products cannot share a launch");
    const uint32_t rows0 = (g0.m + 31u) / 32u, rows1 = (g1.m + 31u) / 32u;
    const uint32_t cols = (std::max(g0.n, g1.n) + 31u) / 32u;
    const dim3 grid(cols, rows0 + rows1);
    if (vec_ok(g0) && vec_ok(g1))
        blt_launch("matmul_splitk", matmul_splitk_pair_kernel<true>, grid, dim3(256), 0, s, g0, g1, rows0);
    else blt_launch("matmul_splitk", matmul_splitk_pair_kernel<false>, grid, dim3(256), 0, s, g0, g1, rows0);
}

namespace {
template <bool VEC, bool ROPE, int WT, int NW>
void launch_mfma_as(dim3 grid, hipStream_t s, const MatmulArgs &g) {
    constexpr size_t lds = MfmaShape<WT, NW>::LDS_BYTES;
    static_assert(lds <= 64u * 1024u, "above 64 KB a kernel has to ask for its LDS first");
    blt_launch("matmul_mfma", matmul_mfma_kernel<VEC, ROPE, WT, NW>, grid, dim3(64 * NW), lds, s, g);
}
template <bool VEC, bool ROPE, int WT>
void launch_mfma(dim3 grid, hipStream_t s, const MatmulArgs &g) {
    if constexpr (WT == 1) {
        if (g.k >= 256u) { /* from eight K steps on: below, the meeting of the sums costs what the overlap gains */
            launch_mfma_as<VEC, ROPE, 1, 8>(grid, s, g);
            return;
        }
    }
    launch_mfma_as<VEC, ROPE, WT, 4>(grid, s, g);
}
} // namespace

void matmul_f32_launch(const MatmulArgs &g, hipStream_t s) {
    if (g.m == 0 || g.n == 0) return;
    const bool rope = g.rope_cos != nullptr && g.rope_cols > 0;
    const Path path = choose_path(g);
    BLT_REQUIRE(g.b2 == nullptr || path != PATH_MFMA, "matmul: the gated product is not available for this shape");
    BLT_REQUIRE(g.norm_w == nullptr || matmul_takes_norm(g), "matmul: the fused row norm is not available for this shape");
    if (path == PATH_SKINNY) {
        BLT_REQUIRE(g.cross_k == nullptr || (matmul_takes_cross(g) && g.cross_v && g.cross_out && g.cross_lo &&
                                             g.cross_hi && g.cross_rows_per_seq >= 1u),
                    "matmul: the cross-attention epilogue is not available for this shape");
        /* one row per workgroup (measured against 2 and 4 at every shape of the decoder: the extra
         * chains of a lane cost more than the re-reads of b from L2) */
        launch_skinny<1>(g, s);
        return;
    }
    const bool vec = vec_ok(g);
    if (g.cross_k) {
        BLT_REQUIRE(matmul_takes_cross(g) && vec && g.cross_v && g.cross_out && g.cross_lo && g.cross_hi &&
                        g.cross_rows_per_seq >= 1u && aligned16(g.cross_k) && aligned16(g.cross_v) &&
                        aligned16(g.cross_out),
                    "matmul: the cross-attention epilogue is not available for this shape");
    }
    if (path == PATH_SPLITK) {
        const dim3 sgrid((g.n + 31u) / 32u, (g.m + 31u) / 32u);
        if (rope) {
            if (vec) launch_splitk<true, true>(g, sgrid, s);
            else launch_splitk<false, true>(g, sgrid, s);
        } else {
            if (vec) launch_splitk<true, false>(g, sgrid, s);
            else launch_splitk<false, false>(g, sgrid, s);
        }
        return;
    }
    /* 128x128 tiles once there are enough of them to load every compute unit twice over */
    const uint32_t tx = (g.n + 2 * TN - 1) / (2 * TN), ty = (g.m + 2 * TM - 1) / (2 * TM);
    constexpr uint64_t big_from = 512u;
    /* Two large tiles are resident per compute unit, 512 at a time: a last round that fills less
     * than three eighths of the chip costs more than the large tile gains (576 tiles, 6144 x 512 .
     * 512 x 1536: 106 us against 92 with the small tile; 640: 106 / 104; 960: 142 / 151) until the
     * rounds are many. */
    const uint64_t big_tiles = (uint64_t)tx * ty, last_round = big_tiles % 512u;
    const bool short_tail = big_tiles < 2048u && last_round != 0u && last_round < 192u;
    if (big_tiles >= big_from && !short_tail) {
        const dim3 grid(tx, ty);
        if (rope) {
            if (vec) launch_mfma<true, true, 2>(grid, s, g);
            else launch_mfma<false, true, 2>(grid, s, g);
        } else {
            if (vec) launch_mfma<true, false, 2>(grid, s, g);
            else launch_mfma<false, false, 2>(grid, s, g);
        }
        return;
    }
    const dim3 grid((g.n + TN - 1) / TN, (g.m + TM - 1) / TM);
    if (rope) {
        if (vec) launch_mfma<true, true, 1>(grid, s, g);
        else launch_mfma<false, true, 1>(grid, s, g);
    } else {
        if (vec) launch_mfma<true, false, 1>(grid, s, g);
        else launch_mfma<false, false, 1>(grid, s, g);
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
    if (m == 0 || n == 0) return;
    if (k == 0) { /* an empty sum: the product is all zeros (csrc/ops/linalg_cpu.c:8-18 stores sum = 0) */
        blt_hip_memset(out->data, 0, m * n * sizeof(float));
        return;
    }
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
