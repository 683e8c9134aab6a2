/*
 * "rows" kernel family: one query row per group of G lanes.
 *
 * The universal attention kernel of the backend: any nq, nk, head_dim, any
 * strides, every visibility kind, weights_out and lse_out.  A group of G
 * lanes owns one query row; lane g of the group owns head-dim elements
 * 4*(g + G*t) .. +3 for t < T.  The group walks the row's key range with an
 * online softmax (running max, running sum, running output), so K and V are
 * each read once and no score matrix is materialised.  It is the fast path
 * for problems whose rows see only a few keys (byte<->patch cross-attention:
 * 1..16 keys per row) and the fallback for shapes the tiled MFMA kernel does
 * not take.  HBM-bound by construction; no LDS.
 */
#include "attn_device.h"
#include "attn_launch.h"
#include "attn_tile.h"
#include "launch.h"

namespace {

template <int G>
__device__ __forceinline__ float group_sum(float x) {
#pragma unroll
    for (int o = 1; o < G; o <<= 1) x += __shfl_xor(x, o, 64);
    return x;
}

/* Four head-dim elements starting at d (zero past head_dim). */
__device__ __forceinline__ float4 load4(const float *row, uint32_t d, uint32_t hd, bool vec4) {
    if (vec4) {
        if (d < hd) return *reinterpret_cast<const float4 *>(row + d);
        return make_float4(0.f, 0.f, 0.f, 0.f);
    }
    float4 r;
    r.x = d + 0 < hd ? row[d + 0] : 0.f;
    r.y = d + 1 < hd ? row[d + 1] : 0.f;
    r.z = d + 2 < hd ? row[d + 2] : 0.f;
    r.w = d + 3 < hd ? row[d + 3] : 0.f;
    return r;
}

/* The same for 16-byte aligned rows with head_dim a multiple of four, without a branch around the
 * load: a branch there makes the compiler wait for every load in flight before the next one is
 * issued, and a trip's loads are meant to travel together. */
__device__ __forceinline__ float4 load4_aligned(const float *row, uint32_t d, uint32_t hd) {
    const bool in = d < hd;
    const float4 t = *reinterpret_cast<const float4 *>(row + (in ? d : 0u));
    return in ? t : make_float4(0.f, 0.f, 0.f, 0.f);
}

__device__ __forceinline__ void store4(float *row, uint32_t d, uint32_t hd, bool vec4, float4 x) {
    if (vec4) {
        if (d < hd) *reinterpret_cast<float4 *>(row + d) = x;
        return;
    }
    if (d + 0 < hd) row[d + 0] = x.x;
    if (d + 1 < hd) row[d + 1] = x.y;
    if (d + 2 < hd) row[d + 2] = x.z;
    if (d + 3 < hd) row[d + 3] = x.w;
}

__device__ __forceinline__ float dot4(float4 a, float4 b) { return a.x * b.x + a.y * b.y + a.z * b.z + a.w * b.w; }

/* One group's walk over its row's key range [lo, hi): U keys per trip with all loads of the trip
 * issued before any arithmetic; the wave makes as many trips as its longest row needs.  A trip is
 * a trip to memory -- at the sizes this kernel is the fast path for (a patch's 1..16 bytes per row)
 * the whole range goes out in ONE, so U is sixteen for aligned rows at the common head widths.
 * Rows with fewer keys repeat their last one (clamped address, weight zero): nothing in the trip
 * sits behind a branch. */
template <int G, int T, bool VEC4>
__device__ __forceinline__ void rows_walk(const AttnProb &p, const float4 (&q)[T], float4 (&o)[T], float &m, float &l,
                                          const uint32_t lo, const uint32_t hi, const float *mrow, const uint32_t g) {
    constexpr int U = !VEC4 ? (T > 2 ? 1 : 4) : (T > 2 ? 1 : (T == 2 ? 4 : 16)); /* wide heads: fewer keys in flight (registers) */
    uint32_t trips = (hi - lo + U - 1) / U;
#pragma unroll
    for (int off = G; off < 64; off <<= 1) trips = max(trips, (uint32_t)__shfl_xor((int)trips, off, 64));
    const uint32_t last = hi > lo ? hi - 1u : 0u; /* a readable key of this row (row 0 when it has none) */

    for (uint32_t trip = 0; trip < trips; trip++) {
        float4 kk[U][T], vv[U][T];
        float bias[U];
        uint32_t jj[U];
#pragma unroll
        for (int u = 0; u < U; u++) {
            jj[u] = lo + trip * U + u;
            const uint32_t jr = p.nk ? min(min(jj[u], last), p.nk - 1u) : 0u;
            const float *krow = p.k + (size_t)jr * p.k_stride;
            const float *vrow = p.v + (size_t)jr * p.v_stride;
#pragma unroll
            for (int t = 0; t < T; t++) {
                if constexpr (VEC4) {
                    kk[u][t] = load4_aligned(krow, 4u * (g + G * t), p.hd);
                    vv[u][t] = load4_aligned(vrow, 4u * (g + G * t), p.hd);
                } else {
                    kk[u][t] = load4(krow, 4u * (g + G * t), p.hd, false);
                    vv[u][t] = load4(vrow, 4u * (g + G * t), p.hd, false);
                }
            }
            bias[u] = mrow ? mrow[jr] : 0.f;
        }
        float x[U];
        float mt = neg_inf();
#pragma unroll
        for (int u = 0; u < U; u++) {
            float part = 0.f;
#pragma unroll
            for (int t = 0; t < T; t++) part += dot4(q[t], kk[u][t]);
            const float sc = group_sum<G>(part) * p.scale + bias[u];
            x[u] = (jj[u] < hi && isfinite(sc)) ? sc : neg_inf();
            mt = fmaxf(mt, x[u]);
        }
        if (mt != neg_inf()) { /* uniform per group */
            const float mn = fmaxf(m, mt);
            const float a = softmax_exp(m - mn);
            l *= a;
#pragma unroll
            for (int t = 0; t < T; t++) {
                o[t].x *= a;
                o[t].y *= a;
                o[t].z *= a;
                o[t].w *= a;
            }
#pragma unroll
            for (int u = 0; u < U; u++) {
                const float w = softmax_exp(x[u] - mn); /* exp(-inf) = 0 for keys not taken */
                l += w;
#pragma unroll
                for (int t = 0; t < T; t++) {
                    o[t].x += w * vv[u][t].x;
                    o[t].y += w * vv[u][t].y;
                    o[t].z += w * vv[u][t].z;
                    o[t].w += w * vv[u][t].w;
                }
            }
            m = mn;
        }
    }
}

/* SRC: where the workgroup finds its problem (attn_tile.h): a device array, the kernel arguments
 * (one problem), or the kernel arguments of a strided batch -- the last two need no trip to memory
 * before the row ranges and the rows themselves can be requested. */
template <int G, int T, int SRC>
__global__ __launch_bounds__(256) void attn_rows_kernel(const AttnProb *__restrict__ probs, uint32_t prob_base,
                                                        AttnAffine aff) {
    constexpr int ROWS_PER_WAVE = 64 / G;
    constexpr int ROWS_PER_BLOCK = 4 * ROWS_PER_WAVE;

    AttnProb p;
    if (SRC == SRC_TILES) p = probs[prob_base + blockIdx.y];
    else if (SRC == SRC_SINGLE) p = aff.first;
    else affine_problem(p, aff, prob_base + blockIdx.y, aff.first.vis == ATTN_VIS_DENSE);
    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t g = lane % G;
    const uint32_t row = blockIdx.x * ROWS_PER_BLOCK + wave * ROWS_PER_WAVE + lane / G;
    /* whole wave past the end: leave (uniform per wave) */
    if (blockIdx.x * ROWS_PER_BLOCK + wave * ROWS_PER_WAVE >= p.nq) return;

    const bool live = row < p.nq;
    const uint32_t i = live ? row : p.nq - 1;
    const bool vec4 = (p.flags & ATTN_FLAG_VEC4) != 0;

    /* the query row is requested before the row's key range is read: the two travel together, and the
     * keys' addresses wait for the range only */
    float4 q[T], o[T];
    const float *qrow = p.q + (size_t)i * p.q_stride;
#pragma unroll
    for (int t = 0; t < T; t++) {
        q[t] = vec4 ? load4_aligned(qrow, 4u * (g + G * t), p.hd) : load4(qrow, 4u * (g + G * t), p.hd, false);
        o[t] = make_float4(0.f, 0.f, 0.f, 0.f);
    }
    uint32_t lo, hi;
    row_key_range(p, i, lo, hi);
    if (!live) hi = lo;

    float m = neg_inf(), l = 0.f;
    const float *mrow = p.vis == ATTN_VIS_DENSE ? p.mask + (size_t)i * p.nk : nullptr;
    if (vec4) rows_walk<G, T, true>(p, q, o, m, l, lo, hi, mrow, g);
    else rows_walk<G, T, false>(p, q, o, m, l, lo, hi, mrow, g);

    if (live) {
        const float inv = l > 0.f ? 1.0f / l : 0.f;
        float *orow = p.out + (size_t)i * p.out_stride;
#pragma unroll
        for (int t = 0; t < T; t++) {
            float4 r = make_float4(o[t].x * inv, o[t].y * inv, o[t].z * inv, o[t].w * inv);
            store4(orow, 4u * (g + G * t), p.hd, vec4, r);
        }
        if (p.lse && g == 0) {
            p.lse[2 * (size_t)i + 0] = m;
            p.lse[2 * (size_t)i + 1] = l;
        }
    }

    if (p.weights) {
        /* second sweep: every column of the row gets its weight (0 where the
         * key is not visible), recomputed against the final (m, l) */
        float *wrow = p.weights + (size_t)i * p.nk;
        uint32_t wn = live ? p.nk : 0;
#pragma unroll
        for (int off = G; off < 64; off <<= 1) wn = max(wn, (uint32_t)__shfl_xor((int)wn, off, 64));
        for (uint32_t j = 0; j < wn; j++) {
            const float *krow = p.k + (size_t)j * p.k_stride;
            float part = 0.f;
#pragma unroll
            for (int t = 0; t < T; t++) part += dot4(q[t], load4(krow, 4u * (g + G * t), p.hd, vec4));
            float x = group_sum<G>(part) * p.scale;
            if (mrow) x += mrow[j];
            float w = 0.f;
            if (j >= lo && j < hi && isfinite(x) && l > 0.f) w = softmax_exp(x - m) / l;
            if (live && g == 0) wrow[j] = w;
        }
    }
}

/* `aff`: NULL = problems [base, base + count) of the device array; count == 0 in it = its first
 * problem alone; else the strided batch it describes, problems [base, base + count) of it */
template <int G, int T>
void launch_rows(const AttnProb *dprobs, uint32_t base, uint32_t count, uint32_t max_nq, const AttnAffine *aff,
                 hipStream_t s) {
    constexpr int ROWS_PER_BLOCK = 4 * (64 / G);
    dim3 grid((max_nq + ROWS_PER_BLOCK - 1) / ROWS_PER_BLOCK, count, 1);
    if (aff && aff->count == 0) {
        blt_launch("attn_rows", attn_rows_kernel<G, T, SRC_SINGLE>, grid, dim3(256), 0, s, dprobs, base, *aff);
    } else if (aff) {
        blt_launch("attn_rows", attn_rows_kernel<G, T, SRC_AFFINE>, grid, dim3(256), 0, s, dprobs, base, *aff);
    } else {
        AttnAffine none;
        __builtin_memset(&none, 0, sizeof(none));
        blt_launch("attn_rows", attn_rows_kernel<G, T, SRC_TILES>, grid, dim3(256), 0, s, dprobs, base, none);
    }
}

void dispatch_rows(const AttnProb *dprobs, uint32_t b, uint32_t n, uint32_t hd, uint32_t max_nq,
                   const AttnAffine *single, hipStream_t s) {
    const uint32_t chunks = (hd + 3) / 4;
    if (chunks <= 1) launch_rows<1, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 2) launch_rows<2, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 4) launch_rows<4, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 8) launch_rows<8, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 16) launch_rows<16, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 32) launch_rows<32, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 64) launch_rows<64, 1>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 128) launch_rows<64, 2>(dprobs, b, n, max_nq, single, s);
    else if (chunks <= 256) launch_rows<64, 4>(dprobs, b, n, max_nq, single, s);
    else launch_rows<64, 16>(dprobs, b, n, max_nq, single, s);
}

} // namespace

/* All problems [base, base+count) share head_dim `hd`. */
void attn_rows_launch(const AttnProb *dprobs, uint32_t base, uint32_t count, uint32_t hd, uint32_t max_nq,
                      hipStream_t s) {
    /* grid.y is limited to 65535 */
    for (uint32_t done = 0; done < count;) {
        const uint32_t n = count - done < 65535u ? count - done : 65535u;
        dispatch_rows(dprobs, base + done, n, hd, max_nq, nullptr, s);
        done += n;
    }
}

void attn_rows_launch_single(const AttnProb &single, hipStream_t s) {
    if (single.nq == 0) return;
    AttnAffine a;
    __builtin_memset(&a, 0, sizeof(a));
    a.first = single; /* count stays 0: one problem */
    dispatch_rows(nullptr, 0, 1, single.hd, single.nq, &a, s);
}

/* A strided batch: the descriptors travel in the kernel arguments. */
void attn_rows_launch_affine(const AttnAffine &aff, hipStream_t s) {
    if (aff.count == 0 || aff.first.nq == 0) return;
    for (uint32_t done = 0; done < aff.count;) { /* grid.y is limited to 65535 */
        const uint32_t n = aff.count - done < 65535u ? aff.count - done : 65535u;
        dispatch_rows(nullptr, done, n, aff.first.hd, aff.first.nq, &aff, s);
        done += n;
    }
}
