/*
 * "mfma" kernel family: fused QK^T -> online softmax -> PV on the fp32 matrix
 * cores of gfx950 (v_mfma_f32_32x32x2_f32), for prefill and block shapes.
 *
 * Work item = one tile of 32 query rows of one (sequence, head) problem, run
 * by a workgroup of four wavefronts.  The four waves split the tile's key
 * tiles (32 keys each) round-robin, each keeps its own running (max, sum,
 * output) and they merge once through LDS at the end, so the serial chain per
 * wave is a quarter of the row's key tiles.
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
#include "hip_check.h"
#include "launch.h"

#include <algorithm>

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

/* key (within a 32-key tile) that accumulator register r of lane half h holds */
__device__ __forceinline__ constexpr uint32_t acc_key(uint32_t r, uint32_t h) { return 8u * (r >> 2) + 4u * h + (r & 3u); }

template <int HALF> /* HALF = HD/2 floats of one row, starting at element d0 */
__device__ __forceinline__ void load_half_row(float (&dst)[HALF], const float *row, uint32_t d0, uint32_t hd,
                                              bool vec4) {
    if (vec4) {
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

template <int HD, bool SINGLE>
__global__ __launch_bounds__(256) void attn_mfma_kernel(const AttnProb *__restrict__ probs,
                                                        const AttnTile *__restrict__ tiles, AttnProb single) {
    constexpr int HALF = HD / 2;
    constexpr int DB = HD / 32; /* 32-wide blocks of the head dim */

    __shared__ float sm_m[4][32];
    __shared__ float sm_l[4][32];
    __shared__ float sm_o[3][HD][33];

    /* SINGLE: the one problem arrives as a kernel argument and block b takes
     * query tile (last - b): later tiles of a causal problem are the long ones */
    const uint32_t qtile = SINGLE ? gridDim.x - 1u - blockIdx.x : tiles[blockIdx.x].qtile;
    const AttnProb p = SINGLE ? single : probs[tiles[blockIdx.x].prob];

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5;
    const uint32_t c = lane & 31u;
    const bool vec4 = (p.flags & ATTN_FLAG_VEC4) != 0;

    const uint32_t q0 = qtile * 32u;
    const uint32_t row = q0 + c;
    const bool live = row < p.nq;
    const uint32_t i = live ? row : p.nq - 1u;

    uint32_t lo, hi;
    row_key_range(p, i, lo, hi);
    if (!live) hi = lo;

    /* key tiles any row of this query tile can see */
    uint32_t tlo = hi > lo ? lo : 0xFFFFFFFFu, thi = hi > lo ? hi : 0u;
#pragma unroll
    for (int off = 1; off < 32; off <<= 1) {
        tlo = min(tlo, (uint32_t)__shfl_xor((int)tlo, off, 64));
        thi = max(thi, (uint32_t)__shfl_xor((int)thi, off, 64));
    }
    const uint32_t kt_lo = thi > tlo ? tlo / 32u : 0u;
    const uint32_t kt_hi = thi > tlo ? (thi + 31u) / 32u : 0u;

    float qf[HALF];
    load_half_row<HALF>(qf, p.q + (size_t)i * p.q_stride, h * HALF, p.hd, vec4);

    const float *mrow = p.vis == ATTN_VIS_DENSE ? p.mask + (size_t)i * p.nk : nullptr;

    floatx16 oacc[DB];
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[b][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    for (uint32_t kt = kt_lo + wave; kt < kt_hi; kt += 4u) {
        const uint32_t k0 = kt * 32u;
        /* ---- fetch ---- */
        float kf[HALF];
        {
            const uint32_t j = min(k0 + c, p.nk - 1u);
            load_half_row<HALF>(kf, p.k + (size_t)j * p.k_stride, h * HALF, p.hd, vec4);
        }
        float vf[DB][16];
#pragma unroll
        for (int s = 0; s < 16; s++) {
            const uint32_t j = min(k0 + acc_key(s, h), p.nk - 1u);
            const float *vrow = p.v + (size_t)j * p.v_stride;
#pragma unroll
            for (int b = 0; b < DB; b++) vf[b][s] = (b * 32u + c) < p.hd ? vrow[b * 32 + c] : 0.f;
        }

        /* ---- S^T = K Q^T ---- */
        floatx16 sacc;
#pragma unroll
        for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
        for (int s = 0; s < HALF; s++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[s], qf[s], sacc, 0, 0, 0);

        /* ---- scale, mask, tile maximum ---- */
        float x[16];
        float mt = neg_inf();
#pragma unroll
        for (int r = 0; r < 16; r++) {
            const uint32_t j = k0 + acc_key(r, h);
            float t = sacc[r] * p.scale;
            if (mrow) t += mrow[min(j, p.nk - 1u)];
            const bool vis = j >= lo && j < hi && isfinite(t);
            x[r] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[r]);
        }
        mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
        const float mn = fmaxf(m, mt);
        const float alpha = m == neg_inf() ? 0.f : softmax_exp(m - mn);
        float ps = 0.f;
#pragma unroll
        for (int r = 0; r < 16; r++) {
            x[r] = x[r] == neg_inf() ? 0.f : softmax_exp(x[r] - mn);
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
    }

    /* both halves of a column carry the same m, their sums add */
    l += __shfl_xor(l, 32, 64);

    /* ---- merge the four waves ---- */
    if (h == 0) {
        sm_m[wave][c] = m;
        sm_l[wave][c] = l;
    }
    if (wave > 0) {
#pragma unroll
        for (int b = 0; b < DB; b++)
#pragma unroll
            for (int r = 0; r < 16; r++) sm_o[wave - 1][b * 32 + acc_key(r, h)][c] = oacc[b][r];
    }
    __syncthreads();

    float M = neg_inf(), L = 0.f;
    if (wave == 0) {
#pragma unroll
        for (int w = 0; w < 4; w++) M = fmaxf(M, sm_m[w][c]);
        float f[4];
#pragma unroll
        for (int w = 0; w < 4; w++) {
            const float mw = sm_m[w][c];
            f[w] = mw == neg_inf() ? 0.f : softmax_exp(mw - M);
            L += sm_l[w][c] * f[w];
        }
        const float inv = L > 0.f ? 1.0f / L : 0.f;
        float *orow = p.out + (size_t)i * p.out_stride;
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
                        if (d0 < p.hd)
                            *reinterpret_cast<float4 *>(orow + d0) =
                                make_float4(oacc[b][4 * g + 0], oacc[b][4 * g + 1], oacc[b][4 * g + 2], oacc[b][4 * g + 3]);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++)
                            if (d0 + e < p.hd) orow[d0 + e] = oacc[b][4 * g + e];
                    }
                }
            }
        }
        if (live && h == 0 && p.lse) {
            p.lse[2 * (size_t)i + 0] = M;
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
    for (uint32_t kt = wave; kt < nkt; kt += 4u) {
        const uint32_t k0 = kt * 32u;
        float w[16];
#pragma unroll
        for (int r = 0; r < 16; r++) w[r] = 0.f;
        if (kt >= kt_lo && kt < kt_hi) {
            float kf[HALF];
            const uint32_t jr = min(k0 + c, p.nk - 1u);
            load_half_row<HALF>(kf, p.k + (size_t)jr * p.k_stride, h * HALF, p.hd, vec4);
            floatx16 sacc;
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
            for (int s = 0; s < HALF; s++) sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(kf[s], qf[s], sacc, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; r++) {
                const uint32_t j = k0 + acc_key(r, h);
                float t = sacc[r] * p.scale;
                if (mrow) t += mrow[min(j, p.nk - 1u)];
                const bool vis = j >= lo && j < hi && isfinite(t);
                w[r] = vis ? softmax_exp(t - M) * invL : 0.f;
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

template <int HD>
void launch_mfma(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, const AttnProb *single,
                 hipStream_t s) {
    if (single) {
        blt_launch("attn_mfma", attn_mfma_kernel<HD, true>, dim3(ntiles), dim3(256), 0, s, dprobs, dtiles, *single);
    } else {
        AttnProb none;
        __builtin_memset(&none, 0, sizeof(none));
        blt_launch("attn_mfma", attn_mfma_kernel<HD, false>, dim3(ntiles), dim3(256), 0, s, dprobs, dtiles, none);
    }
}

} // namespace

/* shapes the kernel is able to run */
bool attn_mfma_can(const AttnProb &d) { return d.hd <= 128u && d.nk >= 1u && d.nq >= 1u; }

/* shapes it is the better choice for */
bool attn_mfma_takes(const AttnProb &d) {
    if (!attn_mfma_can(d)) return false;
    if (d.vis == ATTN_VIS_RANGE) return false; /* per-row ranges are short: the rows family reads less */
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

void attn_mfma_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, hipStream_t s) {
    if (ntiles == 0) return;
    if (hd <= 32u) launch_mfma<32>(dprobs, dtiles, ntiles, nullptr, s);
    else if (hd <= 64u) launch_mfma<64>(dprobs, dtiles, ntiles, nullptr, s);
    else launch_mfma<128>(dprobs, dtiles, ntiles, nullptr, s);
}

void attn_mfma_launch_single(const AttnProb &single, hipStream_t s) {
    const uint32_t ntiles = (single.nq + 31u) / 32u;
    if (ntiles == 0) return;
    if (single.hd <= 32u) launch_mfma<32>(nullptr, nullptr, ntiles, &single, s);
    else if (single.hd <= 64u) launch_mfma<64>(nullptr, nullptr, ntiles, &single, s);
    else launch_mfma<128>(nullptr, nullptr, ntiles, &single, s);
}
