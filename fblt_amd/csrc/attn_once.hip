/*
 * "once" kernel family: attention for a tile of 16 query rows whose keys are
 * few enough to be in flight all at once (up to 1024 at head width 32, 512 at
 * 64), for launches that are one trip to memory deep -- a single
 * (sequence, head) problem issued by an unmodified reference caller
 * (csrc/models/attention.c:92-128, cross_attention.c:70-96: dense additive
 * mask, weights_out set), or a handful of long problems.  At those sizes the
 * time is the chain of dependent steps between kernel entry and the last
 * store, so the chain is made as short as the arithmetic allows:
 *
 *   - a workgroup is one tile of 16 query rows and W waves; wave w owns the
 *     16-key tiles t0 + w, t0 + w + W, ... (T at most) of the tile's key span.
 *     Every operand a wave will ever need -- its query fragment, its K and V
 *     fragments, its piece of the dense mask -- is requested at entry, straight
 *     from global memory in matrix-fragment layout; no row is read twice by a
 *     workgroup, so there is nothing to share through LDS and no barrier
 *     before the arithmetic;
 *   - the softmax is exact, not running: S^T = K Q^T for all of the wave's
 *     tiles (v_mfma_f32_16x16x4_f32, the tiles' chains interleaved), the row
 *     maxima of the W waves meet once in LDS, then P = 2^(x - max) with the
 *     final maximum, O^T += V^T P^T, and the W partial outputs and sums meet
 *     in LDS: plain sums, nothing is rescaled;
 *   - the post-softmax weights, when asked for, go out from the registers that
 *     hold P, in the same sweep (the other matrix-core kernels recompute S in
 *     a second sweep);
 *   - a key tile no row of the query tile sees (above the causal diagonal,
 *     outside the window, or all -inf in the dense mask) costs its loads but
 *     no arithmetic.
 *
 * Transposed products as in the other matrix-core kernels, lane (g = lane /
 * 16, c = lane % 16): register r of a score tile is key 4 g + r, query c; row i
 * of the e-th O^T tile stands for column (HD/16) i + e of the head.  The
 * contraction index of S^T is permuted (lane group g holds floats 16 u + 4 g
 * ... + 3 of a row for u = 0 .. HD/16 - 1) so that the sixteen-byte loads of
 * the four lane groups cover 64 contiguous bytes of a row.
 *
 * Semantics as blt_attention_head_core (csrc/ops/attn_core_cpu.c:16-57,
 * vecmath_cpu.c:16-53): x = score * scale + mask, maximum over finite entries,
 * non-finite entries weigh nothing, an all-masked row gives zeros.
 *
 * Takes head widths 32 and 64 with 16-byte aligned rows; all keys, causal
 * (offset, window) or a dense mask; optional weights and (max, sum) outputs.
 */
#include "attn_device.h"
#include "attn_launch.h"
#include "attn_tile.h"
#include "hip_check.h"
#include "lane_ops.h"
#include "blt_fatal.h"
#include "launch.h"

#include <algorithm>
#include <vector>

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int HD, int W>
struct OnceShape {
    static constexpr int ROW = HD + 4;                       /* floats of a parked output row */
    static constexpr int MROW = 16 + 4;                      /* floats of a parked mask / weight row */
    static constexpr int STATS = 2 * 16 * W;                 /* [16][W] maxima, [16][W] sums   */
    /* + per wave: a tile of 16 rows (Q and K on their way to fragments, then its partial output)
     * and a tile of mask / weight pieces */
    static constexpr int FLOATS = STATS + W * 16 * ROW + W * 16 * MROW;
    static constexpr size_t BYTES = (size_t)FLOATS * sizeof(float);
};

/* Keys row i sees, [lo, hi), for the closed-form kinds (a dense mask decides inside [0, nk)). */
__device__ __forceinline__ void once_row_range(const AttnProb &p, uint32_t i, uint32_t &lo, uint32_t &hi) {
    const bool causal = p.vis == ATTN_VIS_CAUSAL;
    const uint32_t diag1 = i + p.causal_off + 1u; /* below 2^32: both terms are below 2^31 */
    hi = causal ? min(p.nk, diag1) : p.nk;
    lo = causal && p.window > 0u && diag1 > p.window ? min(diag1 - p.window, p.nk) : 0u;
    lo = min(lo, hi);
}

/* four weights of one row, columns j0 .. j0 + 3 (those below nk) */
__device__ __forceinline__ void once_store_piece(float *wrow, uint32_t j0, uint32_t nk, bool row_ok, bool vec,
                                                 const float4 w4) {
    if (!row_ok) return;
    if (vec) {
        if (j0 < nk) *reinterpret_cast<float4 *>(wrow + j0) = w4;
    } else {
        if (j0 + 0u < nk) wrow[j0 + 0u] = w4.x;
        if (j0 + 1u < nk) wrow[j0 + 1u] = w4.y;
        if (j0 + 2u < nk) wrow[j0 + 2u] = w4.z;
        if (j0 + 3u < nk) wrow[j0 + 3u] = w4.w;
    }
}

template <int HD, int W, int T, int SRC, bool DENSE>
__global__ __launch_bounds__(64 * W) void attn_once_kernel(const AttnProb *__restrict__ probs,
                                                          const AttnTile *__restrict__ tiles, AttnAffine aff) {
    using Shape = OnceShape<HD, W>;
    constexpr int QD = HD / 4;  /* floats of a row one lane group contracts */
    constexpr int NV = QD / 4;  /* 16-byte loads per fragment row           */
    constexpr int DT = HD / 16; /* 16-row tiles of O^T                      */
    constexpr int ROW = Shape::ROW;
    constexpr int LPR4 = HD / 4; /* 16-byte pieces of an output row */

    extern __shared__ __attribute__((aligned(16))) float sm[];
    float *const sm_max = sm;            /* [query c][wave] */
    float *const sm_sum = sm + 16 * W;   /* [query c][wave] */
    float *const sm_o = sm + Shape::STATS;

    AttnProb p;
    uint32_t qtile;
    if (SRC == SRC_TILES) {
        qtile = tiles[blockIdx.x].qtile; /* 16-row tiles here */
        p = probs[tiles[blockIdx.x].prob];
    } else if (SRC == SRC_SINGLE) {
        p = aff.first;
        qtile = gridDim.x - 1u - blockIdx.x; /* the long tiles of a causal problem first */
    } else {
        /* Workgroups are handed to the chip's eight dies in turn, each die with an L2 of its own.  A
         * batch of few problems (aff.reserved = 8: eight slots per round, the slots past the
         * problems exit at once) therefore keeps every problem on one die, whose L2 then fetches
         * the problem's K and V rows once for all of its tiles; otherwise the problems of a tile
         * index follow each other. */
        const uint32_t slots = aff.reserved ? aff.reserved : aff.count;
        const uint32_t prob = blockIdx.x % slots;
        if (prob >= aff.count) return; /* uniform over the workgroup, before any barrier */
        qtile = (aff.first.nq + 15u) / 16u - 1u - blockIdx.x / slots;
        affine_problem(p, aff, prob, DENSE);
    }

    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t g = lane >> 4;
    const uint32_t c = lane & 15u;

    const uint32_t q0 = qtile * 16u;
    const uint32_t row = q0 + c;
    const bool live = row < p.nq;
    const uint32_t qi = live ? row : p.nq - 1u;
    uint32_t lo, hi;
    once_row_range(p, qi, lo, hi);
    if (!live) hi = lo;
    const uint32_t vlen = hi - lo;

    /* key tiles any row of the tile sees, [t0, t1): both ends of a row's range grow with the row */
    uint32_t t0 = 0, t1 = 0;
    {
        uint32_t lo_a, hi_a, lo_b, hi_b;
        once_row_range(p, q0, lo_a, hi_a);
        once_row_range(p, min(q0 + 15u, p.nq - 1u), lo_b, hi_b);
        if (hi_a > lo_a) t0 = lo_a / 16u, t1 = (hi_b + 15u) / 16u;
    }
    const uint32_t ntiles = (p.nk + 15u) / 16u;
    const uint32_t last_key = p.nk - 1u;

    /* ---- every request of the wave, before anything waits.  Rows of Q, K, V and the mask are asked
     * for with consecutive lanes on consecutive 16-byte pieces of a row (a load whose lanes each
     * touch another row is served at a quarter of the rate, and the compute unit's one vector memory
     * path is what a tile with many keys waits for: the fewest instructions that move the bytes) and
     * turned into matrix fragments through the wave's own LDS tile. ---- */
    constexpr int LPR = HD / 4;   /* lanes per row when the wave moves a tile */
    constexpr int RPI = 64 / LPR; /* rows one load instruction covers         */
    const uint32_t prow = lane / LPR, pf = lane % LPR;
    const uint32_t mrow_i = lane >> 2, mpiece = lane & 3u; /* mask / weight tiles: 16 rows x 4 pieces */
    float *const tile = sm_o + wave * (16 * ROW);          /* becomes the wave's partial output later */
    float *const mtile = sm_o + W * (16 * ROW) + wave * (16 * Shape::MROW);

    floatx4 qg[NV], kg[T][NV], vg[T][NV], mg[T]; /* native vectors: arrays of the float4 struct were kept in scratch memory */
#pragma unroll
    for (int v = 0; v < NV; v++)
        qg[v] = *reinterpret_cast<const floatx4 *>(p.q + (size_t)min(q0 + prow + (uint32_t)(RPI * v), p.nq - 1u) * p.q_stride + 4u * pf);
    /* A tile past the span repeats the span's last tile: the loads hit the cache, nothing is computed.
     * The mask pieces go first: theirs is the only branch among the requests, and what is requested
     * after it is counted exactly when the scores wait for K but not yet for V. */
    if (DENSE) {
        const bool mvec = (p.nk % 4u == 0u) && ((reinterpret_cast<uintptr_t>(p.mask) & 15u) == 0u);
        const float *mrow = p.mask + (size_t)min(q0 + mrow_i, p.nq - 1u) * p.nk;
#pragma unroll
        for (int u = 0; u < T; u++) {
            const uint32_t kt = min(t0 + wave + (uint32_t)(W * u), t1 > 0u ? t1 - 1u : 0u);
            const uint32_t j0 = 16u * kt + 4u * mpiece;
            if (mvec) {
                mg[u] = *reinterpret_cast<const floatx4 *>(mrow + min(j0, p.nk - 4u));
            } else {
                mg[u][0] = mrow[min(j0 + 0u, last_key)], mg[u][1] = mrow[min(j0 + 1u, last_key)];
                mg[u][2] = mrow[min(j0 + 2u, last_key)], mg[u][3] = mrow[min(j0 + 3u, last_key)];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < T; u++) {
        const uint32_t kt = min(t0 + wave + (uint32_t)(W * u), t1 > 0u ? t1 - 1u : 0u);
#pragma unroll
        for (int v = 0; v < NV; v++)
            kg[u][v] = *reinterpret_cast<const floatx4 *>(
                p.k + (size_t)min(16u * kt + prow + (uint32_t)(RPI * v), last_key) * p.k_stride + 4u * pf);
    }
#pragma unroll
    for (int u = 0; u < T; u++) {
        const uint32_t kt = min(t0 + wave + (uint32_t)(W * u), t1 > 0u ? t1 - 1u : 0u);
#pragma unroll
        for (int v = 0; v < NV; v++)
            vg[u][v] = *reinterpret_cast<const floatx4 *>(
                p.v + (size_t)min(16u * kt + prow + (uint32_t)(RPI * v), last_key) * p.v_stride + 4u * pf);
    }

    /* ---- fragments: lane (g, c) holds floats [g QD, (g + 1) QD) of row c.  The tile is the wave's
     * own and LDS serves a wave's requests in order, so tile after tile goes through it without
     * a barrier. ---- */
    float qf[QD];
    float kf[T][QD];
    float mk[T][4];
    if (DENSE) {
#pragma unroll
        for (int u = 0; u < T; u++) {
            *reinterpret_cast<floatx4 *>(mtile + mrow_i * Shape::MROW + 4u * mpiece) = mg[u];
            const float4 t = *reinterpret_cast<const float4 *>(mtile + c * Shape::MROW + 4u * g);
            mk[u][0] = t.x, mk[u][1] = t.y, mk[u][2] = t.z, mk[u][3] = t.w;
        }
    }
    /* (written out: register arrays handed to a lambda by reference end up in scratch memory) */
#pragma unroll
    for (int v = 0; v < NV; v++)
        *reinterpret_cast<floatx4 *>(tile + (prow + (uint32_t)(RPI * v)) * ROW + 4u * pf) = qg[v];
#pragma unroll
    for (int s = 0; s < QD; s += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(tile + c * ROW + g * QD + s);
        qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
    }
#pragma unroll
    for (int u = 0; u < T; u++) {
#pragma unroll
        for (int v = 0; v < NV; v++)
            *reinterpret_cast<floatx4 *>(tile + (prow + (uint32_t)(RPI * v)) * ROW + 4u * pf) = kg[u][v];
#pragma unroll
        for (int s = 0; s < QD; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(tile + c * ROW + g * QD + s);
            kf[u][s + 0] = t.x, kf[u][s + 1] = t.y, kf[u][s + 2] = t.z, kf[u][s + 3] = t.w;
        }
    }

    /* ---- phase 1: scores of the wave's tiles, their maximum per query ---- */
    const float scale2 = p.scale * LOG2E; /* log2 units: weights are 2^(x - max) */
    float x[T][4];
    bool on[T]; /* uniform over the wave: the tile is inside the span and some row sees some of it */
    float mt = neg_inf();
#pragma unroll
    for (int u = 0; u < T; u++) {
        const uint32_t kt = t0 + wave + (uint32_t)(W * u);
        on[u] = kt < t1;
        if (DENSE && on[u]) { /* a tile the mask closes for every row: no arithmetic */
            /* not -inf: a finite bias, or +inf / NaN (which the softmax drops element by element) */
            const bool open = !(mk[u][0] == neg_inf() && mk[u][1] == neg_inf() && mk[u][2] == neg_inf() &&
                                mk[u][3] == neg_inf());
            on[u] = __builtin_amdgcn_ballot_w64(open) != 0ull;
        }
#pragma unroll
        for (int r = 0; r < 4; r++) x[u][r] = neg_inf();
    }
    /* Two accumulators per tile where the wave has one or two tiles, so that no instruction waits
     * for its predecessor; with more tiles their chains interleave and one accumulator each does. */
    constexpr int NA = T <= 2 ? 2 : 1;
    floatx4 sa[T][NA];
    bool all_on = true;
#pragma unroll
    for (int u = 0; u < T; u++) {
        all_on = all_on & on[u];
#pragma unroll
        for (int a = 0; a < NA; a++) sa[u][a] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    if (all_on) {
#pragma unroll
        for (int s = 0; s < QD; s += NA)
#pragma unroll
            for (int u = 0; u < T; u++)
#pragma unroll
                for (int a = 0; a < NA; a++)
                    sa[u][a] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u][s + a], qf[s + a], sa[u][a], 0, 0, 0);
    } else {
#pragma unroll
        for (int u = 0; u < T; u++) {
            if (on[u]) {
#pragma unroll
                for (int s = 0; s < QD; s += NA)
#pragma unroll
                    for (int a = 0; a < NA; a++)
                        sa[u][a] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u][s + a], qf[s + a], sa[u][a], 0, 0, 0);
            }
        }
    }
    /* while the matrix cores work on the scores: the V rows -> fragments through the same tile; element
     * (d, r) of tile u is column DT c + d of row 4 g + r -- the key whose weight register r of the scores
     * holds, so P^T needs no exchange */
    float vf[T][DT][4];
#pragma unroll
    for (int u = 0; u < T; u++) {
#pragma unroll
        for (int v = 0; v < NV; v++)
            *reinterpret_cast<floatx4 *>(tile + (prow + (uint32_t)(RPI * v)) * ROW + 4u * pf) = vg[u][v];
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float *vrow = tile + (4u * g + r) * ROW + DT * c;
            if constexpr (DT == 2) {
                const float2 t = *reinterpret_cast<const float2 *>(vrow);
                vf[u][0][r] = t.x, vf[u][1][r] = t.y;
            } else {
                static_assert(DT == 4, "head widths 32 and 64");
                const float4 t = *reinterpret_cast<const float4 *>(vrow);
                vf[u][0][r] = t.x, vf[u][1][r] = t.y, vf[u][2][r] = t.z, vf[u][3][r] = t.w;
            }
        }
    }
#pragma unroll
    for (int u = 0; u < T; u++) {
        if (on[u]) {
            const uint32_t rel = 16u * (t0 + wave + (uint32_t)(W * u)) + 4u * g - lo;
#pragma unroll
            for (int r = 0; r < 4; r++) {
                float t;
                const float dot = NA == 2 ? sa[u][0][r] + sa[u][NA - 1][r] : sa[u][0][r];
                if (DENSE) t = (dot * p.scale + mk[u][r]) * LOG2E;
                else t = dot * scale2;
                const bool vis = ((rel + r) < vlen) & isfinite(t);
                x[u][r] = vis ? t : neg_inf();
                mt = fmaxf(mt, x[u][r]);
            }
        }
    }
    mt = swap32(swap16(mt, OpMax()), OpMax());
    if (g == 0) sm_max[c * W + wave] = mt;
    __syncthreads();

    /* ---- phase 2: the final maximum, weights, the wave's share of O^T ---- */
    float M = neg_inf();
#pragma unroll
    for (int w4 = 0; w4 < W; w4 += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(sm_max + c * W + w4);
        M = fmaxf(fmaxf(M, fmaxf(t.x, t.y)), fmaxf(t.z, t.w));
    }
    const float Ms = M == neg_inf() ? 0.f : M;
    float ps = 0.f;
#pragma unroll
    for (int u = 0; u < T; u++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            x[u][r] = fast_exp2(x[u][r] - Ms); /* 2^(-inf) = 0 */
            ps += x[u][r];
        }
    ps = swap32(swap16(ps, OpSum()), OpSum());
    if (g == 0) sm_sum[c * W + wave] = ps;

    floatx4 oacc[DT];
#pragma unroll
    for (int d = 0; d < DT; d++) oacc[d] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < T; u++) {
        if (on[u]) {
#pragma unroll
            for (int r = 0; r < 4; r++)
#pragma unroll
                for (int d = 0; d < DT; d++)
                    oacc[d] = __builtin_amdgcn_mfma_f32_16x16x4f32(vf[u][d][r], x[u][r], oacc[d], 0, 0, 0);
        }
    }
    /* lane (g, c) holds columns 4 DT g ... of query row c: park them */
    {
        float *dst = tile + c * ROW + 4 * DT * g;
        if constexpr (DT == 2) {
#pragma unroll
            for (int r = 0; r < 4; r += 2)
                *reinterpret_cast<float4 *>(dst + 2 * r) = make_float4(oacc[0][r], oacc[1][r], oacc[0][r + 1], oacc[1][r + 1]);
        } else {
#pragma unroll
            for (int r = 0; r < 4; r++)
                *reinterpret_cast<float4 *>(dst + 4 * r) = make_float4(oacc[0][r], oacc[1][r], oacc[2][r], oacc[3][r]);
        }
    }
    __syncthreads();

    /* ---- phase 3: sums of the W partials; weights from the registers that hold P ---- */
    if (p.weights) {
        float L = 0.f;
#pragma unroll
        for (int w4 = 0; w4 < W; w4 += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(sm_sum + c * W + w4);
            L += (t.x + t.y) + (t.z + t.w);
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        /* a tile of weights leaves as it came in: through the wave's piece tile, so that the lanes of
         * a store are consecutive pieces of a row */
        const uint32_t wrow_i = q0 + mrow_i;
        float *wrow = p.weights + (size_t)wrow_i * p.nk;
        const bool wvec = (p.nk % 4u == 0u) && ((reinterpret_cast<uintptr_t>(p.weights) & 15u) == 0u);
#pragma unroll
        for (int u = 0; u < T; u++) {
            const uint32_t kt = t0 + wave + (uint32_t)(W * u);
            if (kt < t1) {
                *reinterpret_cast<float4 *>(mtile + c * Shape::MROW + 4u * g) =
                    make_float4(x[u][0] * inv, x[u][1] * inv, x[u][2] * inv, x[u][3] * inv);
                const float4 w4 = *reinterpret_cast<const float4 *>(mtile + mrow_i * Shape::MROW + 4u * mpiece);
                once_store_piece(wrow, 16u * kt + 4u * mpiece, p.nk, wrow_i < p.nq, wvec, w4);
            }
        }
        /* key tiles outside the span: zeros */
        for (uint32_t kt = wave; kt < ntiles; kt += W)
            if (kt < t0 || kt >= t1)
                once_store_piece(wrow, 16u * kt + 4u * mpiece, p.nk, wrow_i < p.nq, wvec, make_float4(0.f, 0.f, 0.f, 0.f));
    }
    /* thread = (row, 16-byte piece of the row) */
    const uint32_t mr = tid / LPR4, mf = tid % LPR4;
    if (mr < 16u) {
        float L = 0.f, Mr = neg_inf();
#pragma unroll
        for (int w4 = 0; w4 < W; w4 += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(sm_sum + mr * W + w4);
            L += (t.x + t.y) + (t.z + t.w);
            const float4 mx = *reinterpret_cast<const float4 *>(sm_max + mr * W + w4);
            Mr = fmaxf(fmaxf(Mr, fmaxf(mx.x, mx.y)), fmaxf(mx.z, mx.w));
        }
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
        for (int w = 0; w < W; w++) {
            const float4 t = *reinterpret_cast<const float4 *>(sm_o + w * (16 * ROW) + mr * ROW + 4u * mf);
            o.x += t.x, o.y += t.y, o.z += t.z, o.w += t.w;
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        const uint32_t orow = q0 + mr;
        if (orow < p.nq) {
            *reinterpret_cast<float4 *>(p.out + (size_t)orow * p.out_stride + 4u * mf) =
                make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
            if (mf == 0 && p.lse) {
                p.lse[2 * (size_t)orow + 0] = Mr * LN2; /* back to natural units */
                p.lse[2 * (size_t)orow + 1] = L;
            }
        }
    }
}

template <int HD, int W, int T, int SRC, bool DENSE>
void once_launch_kernel(const AttnProb *dprobs, const AttnTile *dtiles, const AttnAffine &aff, uint32_t nblocks,
                        bool pieces, hipStream_t s) {
    using Shape = OnceShape<HD, W>;
    static const bool raised = [] { /* more than the 64 KB a kernel may use without asking */
        if (Shape::BYTES > 64u * 1024u)
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&attn_once_kernel<HD, W, T, SRC, DENSE>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)Shape::BYTES));
        return true;
    }();
    (void)raised;
    /* the piece tiles (mask in, weights out) sit at the end of the workgroup's LDS: a launch with neither
     * does without them, and a fourth workgroup of eight waves then fits a compute unit */
    const size_t lds = DENSE || pieces ? Shape::BYTES : Shape::BYTES - (size_t)W * 16 * Shape::MROW * sizeof(float);
    blt_launch("attn_once", attn_once_kernel<HD, W, T, SRC, DENSE>, dim3(nblocks), dim3(64 * W), lds, s, dprobs, dtiles,
               aff);
}

template <int HD, int W, int T, int SRC>
void once_launch_as(const AttnProb *dprobs, const AttnTile *dtiles, const AttnAffine &aff, uint32_t nblocks, bool dense,
                    bool pieces, hipStream_t s) {
    if (dense) once_launch_kernel<HD, W, T, SRC, true>(dprobs, dtiles, aff, nblocks, pieces, s);
    else once_launch_kernel<HD, W, T, SRC, false>(dprobs, dtiles, aff, nblocks, pieces, s);
}

/* `tiles` = 16-key tiles the longest 16-row tile of the launch spans: sizes the workgroups */
template <int SRC>
void once_launch_shape(const AttnProb *dprobs, const AttnTile *dtiles, const AttnAffine &aff, uint32_t nblocks,
                       uint32_t hd, uint32_t tiles, bool dense, bool pieces, hipStream_t s) {
    BLT_REQUIRE(tiles <= attn_once_tiles_max(hd), "attention: internal: the once kernel was given rows it does not hold");
    if (hd == 32u) {
        if (tiles <= 8u) once_launch_as<32, 8, 1, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
        else if (tiles <= 16u) once_launch_as<32, 16, 1, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
        else if (tiles <= 32u) once_launch_as<32, 16, 2, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
        else once_launch_as<32, 16, 4, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
    } else {
        if (tiles <= 8u) once_launch_as<64, 8, 1, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
        else if (tiles <= 16u) once_launch_as<64, 16, 1, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
        else once_launch_as<64, 16, 2, SRC>(dprobs, dtiles, aff, nblocks, dense, pieces, s);
    }
}

} // namespace

/* most 16-key tiles a 16-row tile may span at head width hd (sixteen waves, four / two tiles each) */
uint32_t attn_once_tiles_max(uint32_t hd) { return hd == 32u ? 64u : 32u; }

/* 16-key tiles the longest 16-row tile of the problem spans */
uint32_t attn_once_span_tiles(const AttnProb &d) {
    if (d.nq == 0 || d.nk == 0) return 0;
    if (d.vis != ATTN_VIS_CAUSAL) return (d.nk + 15u) / 16u;
    uint32_t most = 0;
    for (uint32_t q0 = 0; q0 < d.nq; q0 += 16u) {
        const uint64_t first = (uint64_t)q0 + d.causal_off + 1u;
        const uint64_t last = (uint64_t)std::min(q0 + 15u, d.nq - 1u) + d.causal_off + 1u;
        const uint64_t hi = std::min<uint64_t>(d.nk, last);
        uint64_t lo = 0;
        if (d.window > 0 && first > d.window) lo = std::min<uint64_t>(first - d.window, d.nk);
        if (std::min<uint64_t>(d.nk, first) <= lo) continue; /* the first row sees nothing: the tile computes nothing */
        most = std::max<uint32_t>(most, (uint32_t)((hi + 15u) / 16u - lo / 16u));
    }
    return most;
}

/* shapes the kernel is able to run: the longest 16-row tile's keys fit the waves' registers */
bool attn_once_can(const AttnProb &d) {
    if (!((d.hd == 32u || d.hd == 64u) && (d.flags & ATTN_FLAG_VEC4) != 0 && d.nq >= 1u && d.nk >= 1u)) return false;
    if (!(d.vis == ATTN_VIS_ALL || d.vis == ATTN_VIS_CAUSAL || d.vis == ATTN_VIS_DENSE)) return false;
    return attn_once_span_tiles(d) <= attn_once_tiles_max(d.hd);
}

/* Work items (16-row tiles) for problems [base, base+count), longest first. */
void attn_once_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles) {
    struct Item {
        AttnTile t;
        uint32_t work;
    };
    std::vector<Item> items;
    for (uint32_t n = 0; n < count; n++) {
        const AttnProb &d = host[base + n];
        const uint32_t nqt = (d.nq + 15u) / 16u;
        for (uint32_t t = 0; t < nqt; t++) {
            uint64_t hi = d.nk, lo = 0;
            if (d.vis == ATTN_VIS_CAUSAL) {
                const uint64_t last = std::min<uint64_t>((uint64_t)t * 16u + 15u, d.nq - 1u) + d.causal_off;
                hi = std::min<uint64_t>(hi, last + 1u);
                if (d.window > 0) {
                    const uint64_t first = (uint64_t)t * 16u + d.causal_off;
                    lo = first + 1u > d.window ? first + 1u - d.window : 0u;
                }
            }
            Item it;
            it.t.prob = base + n;
            it.t.qtile = t;
            it.work = hi > lo ? (uint32_t)((hi - lo + 15u) / 16u) : 0u;
            items.push_back(it);
        }
    }
    std::stable_sort(items.begin(), items.end(), [](const Item &a, const Item &b) { return a.work > b.work; });
    for (const Item &it : items) tiles.push_back(it.t);
}

void attn_once_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, uint32_t span_tiles,
                      bool dense, hipStream_t s) {
    if (ntiles == 0) return;
    AttnAffine none;
    __builtin_memset(&none, 0, sizeof(none));
    /* a list may hold problems that want their weights: the piece tiles stay */
    once_launch_shape<SRC_TILES>(dprobs, dtiles, none, ntiles, hd, span_tiles, dense, true, s);
}

void attn_once_launch_single(const AttnProb &single, hipStream_t s) {
    const uint32_t nblocks = (single.nq + 15u) / 16u;
    if (nblocks == 0) return;
    AttnAffine a;
    __builtin_memset(&a, 0, sizeof(a));
    a.first = single;
    once_launch_shape<SRC_SINGLE>(nullptr, nullptr, a, nblocks, single.hd, attn_once_span_tiles(single),
                                  single.vis == ATTN_VIS_DENSE, single.weights != nullptr, s);
}

void attn_once_launch_affine(const AttnAffine &aff, hipStream_t s) {
    const uint32_t nqt = (aff.first.nq + 15u) / 16u;
    if (aff.count == 0 || nqt == 0) return;
    AttnAffine a = aff;
    /* Fewer problems than dies, and no more tiles per problem than a die has compute units: one die per
     * problem (eight workgroup slots per tile index, see the kernel).  Measured at 4 heads x 512 rows:
     * the launch fetches K and V once instead of twice. */
    a.reserved = aff.count < 8u && nqt <= 32u ? 8u : 0u;
    const uint32_t nblocks = (a.reserved ? a.reserved : aff.count) * nqt;
    once_launch_shape<SRC_AFFINE>(nullptr, nullptr, a, nblocks, aff.first.hd, attn_once_span_tiles(aff.first),
                                  aff.first.vis == ATTN_VIS_DENSE, aff.first.weights != nullptr, s);
}
