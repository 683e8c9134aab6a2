/*
 * "mfma" kernel family: fused QK^T -> online softmax -> PV on the fp32 matrix
 * cores of gfx950 (v_mfma_f32_32x32x2_f32), for prefill and block shapes.
 *
 * Work item = one tile of 32 query rows of one (sequence, head) problem, run
 * by a workgroup of four wavefronts (eight when the launch has about as
 * many workgroups as compute units or fewer, and the head dim is 32).  The waves
 * split the tile's key tiles (32 keys each) round-robin, each keeps its own
 * running (max, sum, output) and they merge once through LDS at the end, so
 * the serial chain per wave is a quarter (an eighth) of the row's key tiles.
 *
 * Both contractions are computed TRANSPOSED so that no operand ever has to be
 * re-laid-out between them:
 *
 *   S^T[key, query] = sum_d K[key, d] * Q[query, d]       A = K, B = Q^T
 *   O^T[d,   query] = sum_key V[key, d] * P^T[key, query]  A = V^T, B = P^T
 *
 * In the 32x32 accumulator layout lane L holds column (L % 32) -- one query --
 * in all 16 registers, so a lane's softmax statistics, its P^T values (which
 * are exactly the B operand of the second contraction) and its output
 * accumulators all belong to the same query: the rescale by exp(m_old-m_new)
 * is lane-local and the only cross-lane traffic per tile is one exchange with
 * lane L^32 for the row maximum.
 *
 * Operand fetch: lane (half h = L/32, c = L%32) reads head-dim elements
 * [h*HD/2, (h+1)*HD/2) of K row c straight from global memory with 16-byte
 * loads (the MFMA contraction index is permuted accordingly for both A and
 * B); V rows are read one dword per lane, 32 lanes covering 128 contiguous
 * bytes of a row.  K/V tiles are not shared between the waves of a
 * workgroup (they work on different keys), so there is nothing to stage in
 * LDS; LDS only carries the final merge.
 *
 * Bound: MFMA for long rows (2*HD/2 + 2*HD/2 ... = HD MFMAs of 64 cycles per
 * 32x32 tile against ~8*HD bytes of K/V), launch/latency for the small
 * shapes.
 */
#include "attn_device.h"
#include "attn_launch.h"
#include "attn_tile.h"
#include "hip_check.h"
#include "launch.h"

#include <algorithm>
#include <cstdlib>

namespace {

/* HALF = HD/2 floats of one row starting at element d0.  EXACT: 16-byte
 * aligned rows and head_dim == HD, so no element needs a guard. */
template <int HALF, bool EXACT>
__device__ __forceinline__ void load_half_row(float (&dst)[HALF], const float *row, uint32_t d0, uint32_t hd,
                                              bool vec4) {
    if (EXACT) {
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(row + d0 + s);
            dst[s + 0] = t.x;
            dst[s + 1] = t.y;
            dst[s + 2] = t.z;
            dst[s + 3] = t.w;
        }
    } else if (vec4) {
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
            if (d0 + s < hd) t = *reinterpret_cast<const float4 *>(row + d0 + s);
            dst[s + 0] = t.x;
            dst[s + 1] = t.y;
            dst[s + 2] = t.z;
            dst[s + 3] = t.w;
        }
    } else {
#pragma unroll
        for (int s = 0; s < HALF; s++) dst[s] = d0 + s < hd ? row[d0 + s] : 0.f;
    }
}

/* ---- operand movement helpers (register arrays by reference so they stay in registers) ---- */

/* 32 rows x HD floats, rows [row0, row0+32) clamped to nrows-1: consecutive
 * lanes take consecutive 16-byte pieces of a row; one wave moves the tile. */
template <int HD>
__device__ __forceinline__ void tile_to_regs(float (&kg)[HD / 2], const float *base, uint32_t stride,
                                             uint32_t row0, uint32_t nrows, uint32_t lane) {
    constexpr int LPR = HD / 4;
#pragma unroll
    for (int t = 0; t < HD / 8; t++) {
        const uint32_t r = t * (64 / LPR) + lane / LPR;
        const uint32_t j = min(row0 + r, nrows - 1u);
        const float4 x = *reinterpret_cast<const float4 *>(base + (size_t)j * stride + 4u * (lane % LPR));
        kg[4 * t + 0] = x.x;
        kg[4 * t + 1] = x.y;
        kg[4 * t + 2] = x.z;
        kg[4 * t + 3] = x.w;
    }
}

template <int HD>
__device__ __forceinline__ void regs_to_lds(const float (&kg)[HD / 2], float *dst, uint32_t lane) {
    constexpr int LPR = HD / 4;
    constexpr int ROW = HD + 4;
#pragma unroll
    for (int t = 0; t < HD / 8; t++) {
        const uint32_t r = t * (64 / LPR) + lane / LPR;
        *reinterpret_cast<float4 *>(dst + r * ROW + 4u * (lane % LPR)) =
            make_float4(kg[4 * t + 0], kg[4 * t + 1], kg[4 * t + 2], kg[4 * t + 3]);
    }
}

/* generic tile move (unaligned rows or head_dim < HD): element by element */
template <int HD>
__device__ __forceinline__ void tile_to_lds_slow(float *dst, const float *base, uint32_t stride, uint32_t row0,
                                                 uint32_t nrows, uint32_t hd, uint32_t first, uint32_t step) {
    constexpr int ROW = HD + 4;
    for (uint32_t e = first; e < 32u * HD; e += step) {
        const uint32_t r = e / HD, d = e % HD;
        const uint32_t j = min(row0 + r, nrows - 1u);
        dst[r * ROW + d] = d < hd ? base[(size_t)j * stride + d] : 0.f;
    }
}

/* MFMA fragment of lane (h, c): row c, floats [h*HD/2, (h+1)*HD/2) */
template <int HD>
__device__ __forceinline__ void frag_from_lds(float (&dst)[HD / 2], const float *src, uint32_t h, uint32_t c) {
    constexpr int ROW = HD + 4;
    constexpr int HALF = HD / 2;
#pragma unroll
    for (int s4 = 0; s4 < HALF; s4 += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(src + c * ROW + h * HALF + s4);
        dst[s4 + 0] = t.x;
        dst[s4 + 1] = t.y;
        dst[s4 + 2] = t.z;
        dst[s4 + 3] = t.w;
    }
}

/* LDS of one workgroup.  Q tile and per-wave K tiles are row-major with a
 * 4-float pad per row: a lane's 16-byte fragment reads (row = lane % 32) then
 * fall on distinct banks for every 16 lanes.  The output merge reuses the K
 * area once the key loop is over. */
template <int HD, bool STAGE, int NW>
struct MfmaLds {
    static constexpr int ROW = HD + 4;
    static constexpr int Q_FLOATS = STAGE ? 32 * ROW : 0;
    static constexpr int K_FLOATS = STAGE ? NW * 32 * ROW : 0;
    static constexpr int MERGE_FLOATS = 3 * HD * 33;
    static constexpr int BODY_FLOATS = K_FLOATS > MERGE_FLOATS ? K_FLOATS : MERGE_FLOATS;
};

/* NW = wavefronts per workgroup: 4, or 8 for launches with too few workgroups
 * to occupy the chip (each wave's serial chain of key tiles halves). */
template <int HD, int SRC, bool EXACT, bool DENSE, int NW>
__global__ __launch_bounds__(64 * NW, HD <= 64 ? 2 : 1) void attn_mfma_kernel(const AttnProb *__restrict__ probs,
                                                                            const AttnTile *__restrict__ tiles,
                                                                            AttnAffine aff) {
    constexpr uint32_t NT = 64u * NW; /* threads */
    constexpr int HALF = HD / 2;
    constexpr int DB = HD / 32; /* 32-wide blocks of the head dim */
    /* K and Q tiles go through LDS (coalesced global reads, transposing LDS
     * reads) whenever they fit the 64 KB a workgroup may declare statically */
    constexpr bool STAGE = HD <= 64;
    using Lds = MfmaLds<HD, STAGE, NW>;
    constexpr int ROW = Lds::ROW;

    __shared__ float sm_m[NW][32];
    __shared__ float sm_l[NW][32];
    __shared__ __attribute__((aligned(16))) float sm_q[Lds::Q_FLOATS > 0 ? Lds::Q_FLOATS : 4];
    __shared__ __attribute__((aligned(16))) float sm_body[Lds::BODY_FLOATS];
    uint32_t qtile;
    AttnProb p;
    if (SRC == SRC_TILES) {
        qtile = tiles[blockIdx.x].qtile;
        p = probs[tiles[blockIdx.x].prob];
    } else if (SRC == SRC_SINGLE) {
        /* block b takes query tile (last - b): later tiles of a causal problem are the long ones */
        qtile = gridDim.x - 1u - blockIdx.x;
        p = aff.first;
    } else {
        /* consecutive blocks are different problems of the same query tile,
         * longest tiles first; all tiles of a problem sit at blockIdx = prob
         * (mod count), i.e. on one die when count is a multiple of the die count */
        const uint32_t prob = blockIdx.x % aff.count;
        qtile = aff.nqt - 1u - blockIdx.x / aff.count;
        affine_problem(p, aff, prob, DENSE);
    }

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5;
    const uint32_t c = lane & 31u;
    const bool vec4 = EXACT || (p.flags & ATTN_FLAG_VEC4) != 0;

    const uint32_t q0 = qtile * 32u;
    const uint32_t row = q0 + c;
    const bool live = row < p.nq;
    const uint32_t i = live ? row : p.nq - 1u;

    uint32_t lo, hi;
    row_key_range(p, i, lo, hi);
    if (!live) hi = lo;

    /* key tiles any row of this query tile can see [tlo, thi), and the keys
     * every row sees [flo, fhi): closed form unless rows carry their own ranges */
    uint32_t tlo, thi, flo, fhi;
    if (p.vis == ATTN_VIS_RANGE) {
        tlo = hi > lo ? lo : 0xFFFFFFFFu, thi = hi > lo ? hi : 0u;
        flo = lo, fhi = hi;
#pragma unroll
        for (int off = 1; off < 32; off <<= 1) {
            tlo = min(tlo, (uint32_t)__shfl_xor((int)tlo, off, 64));
            thi = max(thi, (uint32_t)__shfl_xor((int)thi, off, 64));
            flo = max(flo, (uint32_t)__shfl_xor((int)flo, off, 64));
            fhi = min(fhi, (uint32_t)__shfl_xor((int)fhi, off, 64));
        }
    } else {
        span_key_bounds(p, q0, min(q0 + 31u, p.nq - 1u), tlo, thi, flo, fhi);
    }
    const uint32_t kt_lo = thi > tlo ? tlo / 32u : 0u;
    const uint32_t kt_hi = thi > tlo ? (thi + 31u) / 32u : 0u;

    const float *mrow = DENSE ? p.mask + (size_t)i * p.nk : nullptr;
    const float scale2 = p.scale * LOG2E; /* scores are kept in log2 units: weights are 2^(x - m) */

    floatx16 oacc[DB];
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[b][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    /* ---- operand movement ----
     * STAGE: a tile (32 rows x HD floats) is read from global memory with
     * consecutive lanes on consecutive 16-byte pieces of a row (a few cache
     * lines per load instruction instead of one per lane), parked in LDS and
     * read back as MFMA fragments (lane = row).  !STAGE: fragments are read
     * straight from global memory. */
    constexpr int LPR = HD / 4;          /* lanes per row, 16-byte pieces           */
    float kg[HD / 2]; /* one 32-row tile spread over the wave, 16 bytes per lane and step */
    float *my_k = sm_body + (STAGE ? wave * 32 * ROW : 0);

    float qf[HALF];
    float kf[HALF];
    float vf[DB][16];

    if (STAGE) {
        /* the query tile is shared by the waves: each brings its share */
        if (EXACT) {
            constexpr int QPT = 32 * LPR / NT > 0 ? 32 * LPR / NT : 1; /* float4 per thread */
#pragma unroll
            for (int t = 0; t < QPT; t++) {
                const uint32_t e = threadIdx.x + NT * t;
                if (e < 32u * LPR) {
                    const uint32_t r = e / LPR, f4 = e % LPR;
                    const uint32_t qi = min(q0 + r, p.nq - 1u);
                    *reinterpret_cast<float4 *>(sm_q + r * ROW + 4u * f4) =
                        *reinterpret_cast<const float4 *>(p.q + (size_t)qi * p.q_stride + 4u * f4);
                }
            }
        } else {
            tile_to_lds_slow<HD>(sm_q, p.q, p.q_stride, q0, p.nq, p.hd, threadIdx.x, NT);
        }
    } else {
        load_half_row<HALF, EXACT>(qf, p.q + (size_t)i * p.q_stride, h * HALF, p.hd, vec4);
    }

    /* K tile kt: global -> (registers ->) this wave's LDS area, in two steps
     * so the global reads can be in flight while other work runs */
#define K_REQUEST(kt_)                                                                                             \
    do {                                                                                                           \
        if (STAGE) {                                                                                               \
            if (EXACT) tile_to_regs<HD>(kg, p.k, p.k_stride, (kt_) * 32u, p.nk, lane);                             \
        } else {                                                                                                   \
            const uint32_t j_ = min((kt_) * 32u + c, p.nk - 1u);                                                   \
            load_half_row<HALF, EXACT>(kf, p.k + (size_t)j_ * p.k_stride, h * HALF, p.hd, vec4);                   \
        }                                                                                                          \
    } while (0)
#define K_PARK(kt_)                                                                                                \
    do {                                                                                                           \
        if (STAGE) {                                                                                               \
            if (EXACT) regs_to_lds<HD>(kg, my_k, lane);                                                            \
            else tile_to_lds_slow<HD>(my_k, p.k, p.k_stride, (kt_) * 32u, p.nk, p.hd, lane, 64u);                  \
        }                                                                                                          \
    } while (0)

    auto fetch_v = [&](uint32_t kt) __attribute__((always_inline)) {
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const uint32_t j = min(kt * 32u + acc_key(s, h), p.nk - 1u);
            const float *vrow = p.v + (size_t)j * p.v_stride;
#pragma unroll
            for (int b = 0; b < DB; b++) vf[b][s] = (EXACT || (b * 32u + c) < p.hd) ? vrow[b * 32 + c] : 0.f;
        }
    };

    uint32_t kt = kt_lo + wave;
    if (kt < kt_hi) {
        K_REQUEST(kt);
        fetch_v(kt);
    }
    if (STAGE) {
        __syncthreads(); /* query tile complete */
        frag_from_lds<HD>(qf, sm_q, h, c);
        if (kt < kt_hi) K_PARK(kt);
    }
    while (kt < kt_hi) {
        const uint32_t k0 = kt * 32u;
        const uint32_t ktn = kt + NW;

        if (STAGE) {
            frag_from_lds<HD>(kf, my_k, h, c);
            /* the next tile's K rows travel while this tile is worked on */
            if (ktn < kt_hi) K_REQUEST(ktn);
        }

        /* ---- S^T = K Q^T ---- */
        floatx16 sacc;
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < HALF; s++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[s], qf[s], sacc, 0, 0, 0);
        if (!STAGE && ktn < kt_hi) K_REQUEST(ktn);

        /* ---- scale, mask, tile maximum ---- */
        float x[16];
        float mt = neg_inf();
        const bool all_seen = !DENSE && k0 >= flo && k0 + 32u <= fhi; /* uniform: no row masks any key */
        /* lo <= j < hi as one unsigned compare, widened to "always" on tiles every row sees whole:
         * written with && the sixteen tests become sixteen pairs of branches */
        const uint32_t vlo = all_seen ? 0u : lo;
        const uint32_t vlen = all_seen ? 0xFFFFFFFFu : (hi > lo ? hi - lo : 0u);
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t j = k0 + acc_key(r, h);
            float t;
            if (DENSE) t = (sacc[r] * p.scale + mrow[min(j, p.nk - 1u)]) * LOG2E;
            else t = sacc[r] * scale2;
            const bool vis = ((j - vlo) < vlen) & isfinite(t);
            x[r] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[r]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float mn = fmaxf(m, mt);
        const float ms = mn == neg_inf() ? 0.f : mn; /* nothing seen yet: keep the differences finite */
        const float alpha = fast_exp2(m - ms);
        float ps = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            x[r] = fast_exp2(x[r] - ms);
            ps += x[r];
        }
        l = l * alpha + ps;
        m = mn;

        /* ---- O^T = O^T * alpha + V^T P^T ---- */
#pragma unroll
        for (int b = 0; b < DB; b++) {
#pragma unroll
            for (int r = 0; r < 16; r++) oacc[b][r] *= alpha;
#pragma unroll
            for (int s = 0; s < 16; s++)
                oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vf[b][s], x[s], oacc[b], 0, 0, 0);
        }
        if (ktn < kt_hi) {
            fetch_v(ktn);
            K_PARK(ktn);
        }
        kt = ktn;
    }

    /* both halves of a column carry the same m, their sums add */
    l += __shfl_xor(l, 32, 64);

    /* ---- merge the four waves (the merge area overlays the K tiles) ----
     * QUARTER (head dims whose four partial outputs fit the LDS body): every
     * wave parks its partial O^T and merges a quarter of the columns for all
     * 32 rows, reading the four partials from LDS in its own fragment layout.
     * Otherwise wave 0 merges the other three into its registers. */
    constexpr bool QUARTER = NW * HD * 33 <= Lds::BODY_FLOATS;
    static_assert(QUARTER || NW == 4, "the single-merger path is written for four waves");
    float(*sm_o)[HD][33] = reinterpret_cast<float(*)[HD][33]>(sm_body);
    if (STAGE) __syncthreads();
    if (h == 0) {
        sm_m[wave][c] = m;
        sm_l[wave][c] = l;
    }
    if (QUARTER || wave > 0) {
        const uint32_t slot = QUARTER ? wave : wave - 1u;
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) sm_o[slot][b * 32 + acc_key(r, h)][c] = oacc[b][r];
    }
    __syncthreads();

    float M = neg_inf(), L = 0.f;
    if (QUARTER || wave == 0) {
#pragma unroll
        for (int w = 0; w < NW; w++) M = fmaxf(M, sm_m[w][c]);
        const float Ms = M == neg_inf() ? 0.f : M;
        float f[NW];
#pragma unroll
        for (int w = 0; w < NW; w++) {
            f[w] = fast_exp2(sm_m[w][c] - Ms);
            L += sm_l[w][c] * f[w];
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        float *orow = p.out + (size_t)i * p.out_stride;
        if (QUARTER) {
            /* DB * 4 groups of four consecutive columns, shared out over the waves */
            constexpr int GPW = DB * 4 / NW > 0 ? DB * 4 / NW : 1;
#pragma unroll
            for (int k = 0; k < GPW; k++) {
                const uint32_t gid = wave * GPW + k;
                if (gid >= (uint32_t)(DB * 4)) break; /* more waves than groups */
                const uint32_t d0 = (gid >> 2) * 32u + 8u * (gid & 3u) + 4u * h;
                float o4[4];
#pragma unroll
                for (int e = 0; e < 4; e++) {
                    float acc = 0.f;
#pragma unroll
                    for (int w = 0; w < NW; w++) acc += sm_o[w][d0 + e][c] * f[w];
                    o4[e] = acc * inv;
                }
                if (live) {
                    if (vec4) {
                        if (EXACT || d0 < p.hd)
                            *reinterpret_cast<float4 *>(orow + d0) = make_float4(o4[0], o4[1], o4[2], o4[3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (d0 + e < p.hd) orow[d0 + e] = o4[e];
                    }
                }
            }
        } else {
#pragma unroll
            for (int b = 0; b < DB; b++) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const uint32_t d = b * 32 + acc_key(r, h);
                    float acc = oacc[b][r] * f[0];
#pragma unroll
                    for (int w = 1; w < 4; w++) acc += sm_o[w - 1][d][c] * f[w];
                    oacc[b][r] = acc * inv;
                }
                if (live) {
#pragma unroll
                    for (int g = 0; g < 4; g++) {
                        const uint32_t d0 = b * 32 + 8 * g + 4 * h;
                        if (vec4) {
                            if (EXACT || d0 < p.hd)
                                *reinterpret_cast<float4 *>(orow + d0) = make_float4(
                                    oacc[b][4 * g + 0], oacc[b][4 * g + 1], oacc[b][4 * g + 2], oacc[b][4 * g + 3]);
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; e++)
                                if (d0 + e < p.hd) orow[d0 + e] = oacc[b][4 * g + e];
                        }
                    }
                }
            }
        }
        if (wave == 0 && live && h == 0 && p.lse) {
            p.lse[2 * (size_t)i + 0] = M * LN2; /* back to natural units */
            p.lse[2 * (size_t)i + 1] = L;
        }
    }

    if (!p.weights) return;

    /* ---- optional: post-softmax weights for every column of the tile's rows ---- */
    __syncthreads();
    if (wave == 0 && h == 0) {
        sm_m[0][c] = M;
        sm_l[0][c] = L;
    }
    __syncthreads();
    M = sm_m[0][c];
    L = sm_l[0][c];
    const float invL = L > 0.f ? 1.0f / L : 0.f;
    float *wrow = p.weights + (size_t)i * p.nk;
    const bool wvec = (p.nk % 4u == 0u) && ((reinterpret_cast<uintptr_t>(p.weights) & 15u) == 0u);
    const uint32_t nkt = (p.nk + 31u) / 32u;
    for (uint32_t wt = wave; wt < nkt; wt += NW) {
        const uint32_t k0 = wt * 32u;
        float w[16];
#pragma unroll
        for (int r = 0; r < 16; r++) w[r] = 0.f;
        if (wt >= kt_lo && wt < kt_hi) {
            K_REQUEST(wt);
            if (STAGE) {
                K_PARK(wt);
                frag_from_lds<HD>(kf, my_k, h, c);
            }
            floatx16 sacc;
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
            for (int s = 0; s < HALF; s++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[s], qf[s], sacc, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t j = k0 + acc_key(r, h);
                float t;
                if (DENSE) t = (sacc[r] * p.scale + mrow[min(j, p.nk - 1u)]) * LOG2E;
                else t = sacc[r] * scale2;
                const bool vis = j >= lo && j < hi && isfinite(t);
                w[r] = vis ? fast_exp2(t - M) * invL : 0.f;
            }
        }
        if (live) {
#pragma unroll
            for (int g = 0; g < 4; g++) {
                const uint32_t j0 = k0 + 8 * g + 4 * h;
                if (wvec) {
                    if (j0 < p.nk)
                        *reinterpret_cast<float4 *>(wrow + j0) =
                            make_float4(w[4 * g + 0], w[4 * g + 1], w[4 * g + 2], w[4 * g + 3]);
                } else {
#pragma unroll
                    for (int e = 0; e < 4; e++)
                        if (j0 + e < p.nk) wrow[j0 + e] = w[4 * g + e];
                }
            }
        }
    }
}

#undef K_REQUEST
#undef K_PARK

template <int HD, int SRC>
void launch_variant(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t nblocks, const AttnAffine &aff,
                    bool exact, bool dense, hipStream_t s) {
    const dim3 grid(nblocks);
    if constexpr (HD == 32) {
        /* fewer workgroups than the compute units can spread: eight waves each (their K tiles fit
         * LDS at this head dim); measured: ahead up to 256 workgroups, level at 512 */
        constexpr uint32_t below = 320u;
        if (exact && nblocks < below) {
            if (dense)
                blt_launch("attn_mfma", attn_mfma_kernel<HD, SRC, true, true, 8>, grid, dim3(512), 0, s, dprobs, dtiles,
                           aff);
            else
                blt_launch("attn_mfma", attn_mfma_kernel<HD, SRC, true, false, 8>, grid, dim3(512), 0, s, dprobs,
                           dtiles, aff);
            return;
        }
    }
    const dim3 block(256);
    if (exact && dense)
        blt_launch("attn_mfma", attn_mfma_kernel<HD, SRC, true, true, 4>, grid, block, 0, s, dprobs, dtiles, aff);
    else if (exact)
        blt_launch("attn_mfma", attn_mfma_kernel<HD, SRC, true, false, 4>, grid, block, 0, s, dprobs, dtiles, aff);
    else if (dense)
        blt_launch("attn_mfma", attn_mfma_kernel<HD, SRC, false, true, 4>, grid, block, 0, s, dprobs, dtiles, aff);
    else
        blt_launch("attn_mfma", attn_mfma_kernel<HD, SRC, false, false, 4>, grid, block, 0, s, dprobs, dtiles, aff);
}

template <int SRC>
void launch_hd(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t nblocks, const AttnAffine &aff, uint32_t hd,
               bool vec4, bool dense, hipStream_t s) {
    if (hd <= 32u) launch_variant<32, SRC>(dprobs, dtiles, nblocks, aff, vec4 && hd == 32u, dense, s);
    else if (hd <= 64u) launch_variant<64, SRC>(dprobs, dtiles, nblocks, aff, vec4 && hd == 64u, dense, s);
    else launch_variant<128, SRC>(dprobs, dtiles, nblocks, aff, vec4 && hd == 128u, dense, s);
}

} // namespace

/* shapes the kernel is able to run */
bool attn_mfma_can(const AttnProb &d) { return d.hd <= 128u && d.nk >= 1u && d.nq >= 1u; }

/* shapes it is the better choice for */
bool attn_mfma_takes(const AttnProb &d) {
    if (!attn_mfma_can(d)) return false;
    /* per-row ranges are short (a patch's bytes) unless the caller says otherwise: the rows family
     * reads less.  Document-causal self-attention comes as ranges as long as the document: measured
     * at 128 ... 2048 rows, both head widths, the two families are level at ranges of 16 keys, this
     * one is 1.5 times faster at 32 and 9 ... 13 times at 512 and more. */
    constexpr uint32_t span_min = 24u;
    if (d.vis == ATTN_VIS_RANGE && d.range_span < span_min) return false;
    return d.nq >= 16u;
}

/* Work items for problems [base, base+count), longest first. */
void attn_mfma_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles) {
    struct Item {
        AttnTile t;
        uint32_t work;
    };
    std::vector<Item> items;
    for (uint32_t n = 0; n < count; n++) {
        const AttnProb &d = host[base + n];
        const uint32_t nqt = (d.nq + 31u) / 32u;
        for (uint32_t t = 0; t < nqt; t++) {
            uint64_t hi = d.nk, lo = 0;
            if (d.vis == ATTN_VIS_CAUSAL) {
                const uint64_t last = std::min<uint64_t>((uint64_t)t * 32u + 31u, d.nq - 1u) + d.causal_off;
                hi = std::min<uint64_t>(hi, last + 1u);
                if (d.window > 0) {
                    const uint64_t first = (uint64_t)t * 32u + d.causal_off;
                    lo = first + 1u > d.window ? first + 1u - d.window : 0u;
                }
            }
            Item it;
            it.t.prob = base + n;
            it.t.qtile = t;
            it.work = hi > lo ? (uint32_t)((hi - lo + 31u) / 32u) : 0u;
            items.push_back(it);
        }
    }
    std::stable_sort(items.begin(), items.end(), [](const Item &a, const Item &b) { return a.work > b.work; });
    for (const Item &it : items) tiles.push_back(it.t);
}

/* Tile-list launch: every problem of the list has head_dim hd; `vec4` and
 * `dense` must hold for all of them (the caller buckets by these). */
void attn_mfma_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, bool vec4,
                      bool dense, hipStream_t s) {
    if (ntiles == 0) return;
    AttnAffine none;
    __builtin_memset(&none, 0, sizeof(none));
    launch_hd<SRC_TILES>(dprobs, dtiles, ntiles, none, hd, vec4, dense, s);
}

void attn_mfma_launch_single(const AttnProb &single, hipStream_t s) {
    const uint32_t ntiles = (single.nq + 31u) / 32u;
    if (ntiles == 0) return;
    AttnAffine a;
    __builtin_memset(&a, 0, sizeof(a));
    a.first = single;
    launch_hd<SRC_SINGLE>(nullptr, nullptr, ntiles, a, single.hd, (single.flags & ATTN_FLAG_VEC4) != 0,
                          single.vis == ATTN_VIS_DENSE, s);
}

void attn_mfma_launch_affine(const AttnAffine &aff, hipStream_t s) {
    const uint32_t blocks = aff.count * aff.nqt;
    if (blocks == 0) return;
    launch_hd<SRC_AFFINE>(nullptr, nullptr, blocks, aff, aff.first.hd, (aff.first.flags & ATTN_FLAG_VEC4) != 0,
                          aff.first.vis == ATTN_VIS_DENSE, s);
}
