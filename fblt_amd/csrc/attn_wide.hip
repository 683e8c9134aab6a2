/*
 * "wide" kernel family: the matrix-core attention forward for batches large
 * enough to fill the chip several times over, where throughput matters and
 * per-launch latency does not.
 *
 * Work item = 128 consecutive query rows of one (sequence, head) problem.
 * The four wavefronts of the workgroup own one 32-row query tile each and
 * walk the key tiles (32 keys) TOGETHER: every K and V tile is brought from
 * global memory once per workgroup, with fully coalesced 16-byte loads, into
 * a double-buffered LDS area and read from there by all four waves as MFMA
 * fragments.  Nothing is split along the keys, so there is no merge: a wave
 * keeps its own running (max, sum, output) from the first key tile to the
 * last and writes its 32 output rows itself.  Against the latency-oriented
 * kernel in attn_mfma.hip this removes the per-tile query load, the
 * four-way merge and three quarters of the K/V traffic to L2.
 *
 * Arithmetic is the transposed formulation shared with attn_mfma.hip:
 *   S^T[key, query] = K Q^T,  O^T[d, query] = V^T P^T
 * so a lane's softmax statistics, P^T operands and output accumulators all
 * belong to one query and the only cross-lane step per tile is one exchange
 * with lane L^32 for the maximum.  Scores live in log2 units (the query
 * fragment is pre-multiplied by scale*log2(e)); the accumulator is rescaled
 * only on tiles where some row's maximum actually moved.
 *
 * Causal problems: the workgroup walks the union of its four tiles' key
 * ranges; a wave skips the arithmetic (not the loads or barriers) of key
 * tiles outside its own range.  Because later groups of a causal problem see
 * more keys, a work item is a PAIR of groups (g, G-1-g) run back to back, so
 * every workgroup of a problem does the same amount of work.
 *
 * Non-finite scores (the reference drops such keys) are handled
 * optimistically: the key loop runs without per-element finiteness tests --
 * on gfx950 the fp32 matrix instructions and the vector ALU share issue
 * cycles, so every VALU instruction saved is matrix time gained -- and a NaN
 * or +inf score necessarily leaves a non-finite row sum behind; a workgroup
 * that finds one re-runs its group with the tests compiled in.
 *
 * Shapes: head_dim 32 or 64 exactly, 16-byte aligned rows, no weights
 * output, any visibility except per-row ranges.  Bound: MFMA (HD MFMAs of 64
 * cycles per 32x32 tile pair against ~500 VALU cycles of softmax that a
 * second resident wave hides).
 */
#include "attn_device.h"
#include "attn_launch.h"
#include "attn_tile.h"
#include "hip_check.h"
#include "launch.h"

#include <algorithm>

namespace {

/* One 128-row group of problem p.  CHECK: test every score for finiteness.
 * Returns (to every thread of the workgroup that asks) whether this lane's
 * row ended with a non-finite sum, which only happens when !CHECK let a
 * non-finite score through; nothing is stored in that case. */
template <int HD, bool DENSE, bool CHECK>
__device__ __forceinline__ bool wide_group(const AttnProb &p, uint32_t group, float (&sm_k)[2][32 * (HD + 4)],
                                           float (&sm_v)[2][32 * (HD + 4)]) {
    constexpr int HALF = HD / 2;
    constexpr int DB = HD / 32;
    constexpr int ROW = HD + 4;
    constexpr int LPR = HD / 4;            /* 16-byte pieces per row               */
    constexpr int PIECES = 32 * LPR / 256; /* pieces of one tile per thread        */

    const uint32_t lane = threadIdx.x & 63u;
    const uint32_t wave = threadIdx.x >> 6;
    const uint32_t h = lane >> 5;
    const uint32_t c = lane & 31u;

    const uint32_t g0 = group * 128u;       /* first row of the workgroup */
    /* which of the four query tiles a wave owns rotates with the group index:
     * under a causal mask the later tiles are longer, and waves with the same
     * index tend to share a SIMD across resident workgroups */
    const uint32_t q0 = g0 + ((wave + group) & 3u) * 32u; /* first row of this wave */
    const uint32_t row = q0 + c;
    const bool live = row < p.nq;
    const uint32_t i = live ? row : p.nq - 1u;

    uint32_t lo, hi;
    row_key_range(p, i, lo, hi);
    if (!live) hi = lo;

    /* key spans of the workgroup and of this wave, in tiles; all wave-uniform */
    uint32_t glo, ghi, wlo = 0xFFFFFFFFu, whi = 0u, flo = 0u, fhi = 0u, dummy0, dummy1;
    span_key_bounds(p, g0, min(g0 + 127u, p.nq - 1u), glo, ghi, dummy0, dummy1);
    if (q0 < p.nq) span_key_bounds(p, q0, min(q0 + 31u, p.nq - 1u), wlo, whi, flo, fhi);
    const bool g_any = ghi > glo, w_any = whi > wlo;
    const uint32_t gt_lo = __builtin_amdgcn_readfirstlane(g_any ? glo / 32u : 0u);
    const uint32_t gt_hi = __builtin_amdgcn_readfirstlane(g_any ? (ghi + 31u) / 32u : 0u);
    const uint32_t kt_lo = __builtin_amdgcn_readfirstlane(w_any ? wlo / 32u : 0u);
    const uint32_t kt_hi = __builtin_amdgcn_readfirstlane(w_any ? (whi + 31u) / 32u : 0u);
    flo = __builtin_amdgcn_readfirstlane(flo);
    fhi = __builtin_amdgcn_readfirstlane(fhi);

    const float scale2 = p.scale * LOG2E;
    const float *mrow = DENSE ? p.mask + (size_t)i * p.nk : nullptr;
    const bool mvec = DENSE && (p.nk % 4u == 0u) && ((reinterpret_cast<uintptr_t>(p.mask) & 15u) == 0u);

    /* ---- query fragment: row c, floats [h*HALF, (h+1)*HALF), pre-scaled ---- */
    float qf[HALF];
    {
        const float *qrow = p.q + (size_t)i * p.q_stride + h * HALF;
#pragma unroll
        for (int s = 0; s < HALF; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(qrow + s);
            qf[s + 0] = t.x * scale2;
            qf[s + 1] = t.y * scale2;
            qf[s + 2] = t.z * scale2;
            qf[s + 3] = t.w * scale2;
        }
    }

    floatx16 oacc[DB];
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int r = 0; r < 16; r++) oacc[b][r] = 0.f;
    float m = neg_inf(), l = 0.f;

    /* ---- tile movement: thread t carries pieces t, t+256, ... of K and of V ---- */
    float pk[4 * PIECES], pv[4 * PIECES];
    auto request = [&](uint32_t kt) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < PIECES; u++) {
            const uint32_t e = threadIdx.x + 256u * u;
            const uint32_t j = min(kt * 32u + e / LPR, p.nk - 1u);
            const float4 a = *reinterpret_cast<const float4 *>(p.k + (size_t)j * p.k_stride + 4u * (e % LPR));
            const float4 b = *reinterpret_cast<const float4 *>(p.v + (size_t)j * p.v_stride + 4u * (e % LPR));
            pk[4 * u + 0] = a.x, pk[4 * u + 1] = a.y, pk[4 * u + 2] = a.z, pk[4 * u + 3] = a.w;
            pv[4 * u + 0] = b.x, pv[4 * u + 1] = b.y, pv[4 * u + 2] = b.z, pv[4 * u + 3] = b.w;
        }
    };
    auto park = [&](uint32_t buf) __attribute__((always_inline)) {
#pragma unroll
        for (int u = 0; u < PIECES; u++) {
            const uint32_t e = threadIdx.x + 256u * u;
            const uint32_t off = (e / LPR) * ROW + 4u * (e % LPR);
            *reinterpret_cast<float4 *>(&sm_k[buf][off]) =
                make_float4(pk[4 * u + 0], pk[4 * u + 1], pk[4 * u + 2], pk[4 * u + 3]);
            *reinterpret_cast<float4 *>(&sm_v[buf][off]) =
                make_float4(pv[4 * u + 0], pv[4 * u + 1], pv[4 * u + 2], pv[4 * u + 3]);
        }
    };

    if (gt_lo < gt_hi) {
        request(gt_lo);
        park(0);
    }
    __syncthreads();

    for (uint32_t kt = gt_lo; kt < gt_hi; kt++) {
        const uint32_t buf = (kt - gt_lo) & 1u;
        const bool more = kt + 1u < gt_hi;
        if (more) request(kt + 1u); /* travels while this tile is worked on */

        if (kt >= kt_lo && kt < kt_hi) {
            const uint32_t k0 = kt * 32u;
            const float *ks = sm_k[buf];
            const float *vs = sm_v[buf];

            /* dense mask values for this lane's 16 keys: requested before the first contraction */
            float mk[16];
            if (DENSE) {
#pragma unroll
                for (int g = 0; g < 4; g++) {
                    const uint32_t j0 = k0 + 8u * g + 4u * h;
                    if (mvec) {
                        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
                        if (j0 < p.nk) t = *reinterpret_cast<const float4 *>(mrow + j0);
                        mk[4 * g + 0] = t.x, mk[4 * g + 1] = t.y, mk[4 * g + 2] = t.z, mk[4 * g + 3] = t.w;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; e++) mk[4 * g + e] = mrow[min(j0 + e, p.nk - 1u)];
                    }
                }
            }

            /* ---- S^T = K Q^T ---- */
            floatx16 sacc;
#pragma unroll
            for (int r = 0; r < 16; r++) sacc[r] = 0.f;
#pragma unroll
            for (int s4 = 0; s4 < HALF; s4 += 4) {
                const float4 t = *reinterpret_cast<const float4 *>(ks + c * ROW + h * HALF + s4);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(t.x, qf[s4 + 0], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(t.y, qf[s4 + 1], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(t.z, qf[s4 + 2], sacc, 0, 0, 0);
                sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(t.w, qf[s4 + 3], sacc, 0, 0, 0);
            }

            /* ---- mask, tile maximum ----
             * Interior tiles (no row masks any key) take the scores as they
             * are; edge tiles compare the key's offset into the row's range
             * with one unsigned test.  No per-element branches. */
            float x[16];
            float mt = neg_inf();
            const bool all_seen = !DENSE && k0 >= flo && k0 + 32u <= fhi; /* wave-uniform */
            if (all_seen) {
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    const float t = sacc[r];
                    x[r] = (!CHECK || isfinite(t)) ? t : neg_inf();
                    mt = fmaxf(mt, x[r]);
                }
            } else {
                const uint32_t rel = k0 + 4u * h - lo, len = hi - lo;
#pragma unroll
                for (int r = 0; r < 16; r++) {
                    float t = sacc[r];
                    if (DENSE) t += mk[r] * LOG2E;
                    const bool vis = (rel + (8u * (r >> 2) + (r & 3u)) < len) & (!CHECK || isfinite(t));
                    x[r] = vis ? t : neg_inf();
                    mt = fmaxf(mt, x[r]);
                }
            }
            mt = fmaxf(mt, __shfl_xor(mt, 32, 64));
            const float mn = fmaxf(m, mt);
            const float ms = mn == neg_inf() ? 0.f : mn; /* nothing seen yet: keep the differences finite */
            if (__any(mn > m)) {
                const float alpha = fast_exp2(m - ms);
                l *= alpha;
#pragma unroll
                for (int b = 0; b < DB; b++)
#pragma unroll
                    for (int r = 0; r < 16; r++) oacc[b][r] *= alpha;
                m = mn;
            }
            float ps = 0.f;
#pragma unroll
            for (int r = 0; r < 16; r++) {
                x[r] = fast_exp2(x[r] - ms);
                ps += x[r];
            }
            l += ps;

            /* ---- O^T += V^T P^T ---- */
#pragma unroll
            for (int s = 0; s < 16; s++) {
                const float *vrow = vs + acc_key(s, h) * ROW + c;
#pragma unroll
                for (int b = 0; b < DB; b++)
                    oacc[b] = __builtin_amdgcn_mfma_f32_32x32x2f32(vrow[32 * b], x[s], oacc[b], 0, 0, 0);
            }
        }

        if (more) park(buf ^ 1u);
        __syncthreads();
    }

    /* both halves of a column carry the same m, their sums add */
    l += __shfl_xor(l, 32, 64);
    if (!CHECK && !isfinite(l)) return true;
    if (!live) return false;

    const float inv = l > 0.f ? 1.0f / l : 0.f;
    float *orow = p.out + (size_t)i * p.out_stride;
#pragma unroll
    for (int b = 0; b < DB; b++)
#pragma unroll
        for (int g = 0; g < 4; g++)
            *reinterpret_cast<float4 *>(orow + b * 32 + 8 * g + 4 * h) =
                make_float4(oacc[b][4 * g + 0] * inv, oacc[b][4 * g + 1] * inv, oacc[b][4 * g + 2] * inv,
                            oacc[b][4 * g + 3] * inv);
    if (h == 0 && p.lse) {
        p.lse[2 * (size_t)i + 0] = m * LN2; /* back to natural units */
        p.lse[2 * (size_t)i + 1] = l;
    }
    return false;
}

/* Work item encoding shared by the three sources: two group indices, the
 * second one WIDE_NO_GROUP when the item is a single group. */
constexpr uint32_t WIDE_NO_GROUP = 0xFFFFu;

/* item t of a problem with G groups, paired: (G-1-t, t), the middle one alone */
__device__ __forceinline__ void wide_pair(uint32_t t, uint32_t G, uint32_t &ga, uint32_t &gb) {
    ga = G - 1u - t;
    gb = t < ga ? t : WIDE_NO_GROUP;
}

template <int HD, int SRC, bool DENSE>
__global__ __launch_bounds__(256, 2) void attn_wide_kernel(const AttnProb *__restrict__ probs,
                                                           const AttnTile *__restrict__ tiles, AttnAffine aff) {
    constexpr int TILE = 32 * (HD + 4);
    __shared__ __attribute__((aligned(16))) float sm_k[2][TILE];
    __shared__ __attribute__((aligned(16))) float sm_v[2][TILE];

    uint32_t ga, gb = WIDE_NO_GROUP;
    AttnProb p;
    if (SRC == SRC_TILES) {
        const uint32_t code = tiles[blockIdx.x].qtile;
        ga = code & 0xFFFFu, gb = code >> 16;
        p = probs[tiles[blockIdx.x].prob];
    } else if (SRC == SRC_SINGLE) {
        p = aff.first;
        if (aff.reserved) wide_pair(blockIdx.x, aff.nqt, ga, gb);
        else ga = aff.nqt - 1u - blockIdx.x; /* causal with a window: the long groups start first */
    } else {
        /* consecutive blocks are different problems of the same item index,
         * so all groups of one problem land on one die (shared L2) whenever
         * the problem count is a multiple of the die count */
        const uint32_t prob = blockIdx.x % aff.count;
        if (aff.reserved) wide_pair(blockIdx.x / aff.count, aff.nqt, ga, gb);
        else ga = aff.nqt - 1u - blockIdx.x / aff.count;
        affine_problem(p, aff, prob, DENSE);
    }

    for (int pass = 0; pass < 2; pass++) {
        const uint32_t group = pass == 0 ? ga : gb;
        if (group == WIDE_NO_GROUP) break;
        const bool bad = wide_group<HD, DENSE, false>(p, group, sm_k, sm_v);
        if (__syncthreads_or(bad)) wide_group<HD, DENSE, true>(p, group, sm_k, sm_v);
    }
}

template <int SRC>
void launch_wide(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t nblocks, const AttnAffine &aff, uint32_t hd,
                 bool dense, hipStream_t s) {
    const dim3 grid(nblocks), block(256);
    if (hd == 32u && dense)
        blt_launch("attn_wide", attn_wide_kernel<32, SRC, true>, grid, block, 0, s, dprobs, dtiles, aff);
    else if (hd == 32u)
        blt_launch("attn_wide", attn_wide_kernel<32, SRC, false>, grid, block, 0, s, dprobs, dtiles, aff);
    else if (dense)
        blt_launch("attn_wide", attn_wide_kernel<64, SRC, true>, grid, block, 0, s, dprobs, dtiles, aff);
    else
        blt_launch("attn_wide", attn_wide_kernel<64, SRC, false>, grid, block, 0, s, dprobs, dtiles, aff);
}

} // namespace

/* shapes the kernel is able to run */
bool attn_wide_can(const AttnProb &d) {
    return (d.hd == 32u || d.hd == 64u) && (d.flags & ATTN_FLAG_VEC4) != 0 && d.weights == nullptr &&
           d.vis != ATTN_VIS_RANGE && d.nk >= 1u && d.nq >= 1u && d.nq <= 0xFFFEu * 128u; /* group indices travel in 16 bits */
}

uint32_t attn_wide_groups(const AttnProb &d) { return (d.nq + 127u) / 128u; }

/* Causal problems without a window: group g sees ~g+1 times the keys of group
 * 0, so groups are run in pairs (g, G-1-g) of equal total work.  Short
 * problems keep single groups: their imbalance is bounded by a few tiles and
 * twice the workgroups hide more latency. */
bool attn_wide_pairs(const AttnProb &d) {
    return d.vis == ATTN_VIS_CAUSAL && d.window == 0u && attn_wide_groups(d) >= 8u;
}

/* work items of one problem */
uint32_t attn_wide_items(const AttnProb &d) {
    const uint32_t G = attn_wide_groups(d);
    return attn_wide_pairs(d) ? (G + 1u) / 2u : G;
}

/* Work items for problems [base, base+count), longest first. */
void attn_wide_make_tiles(const AttnProb *host, uint32_t base, uint32_t count, std::vector<AttnTile> &tiles) {
    struct Item {
        AttnTile t;
        uint32_t work;
    };
    auto key_tiles = [](const AttnProb &d, uint32_t g) -> uint32_t {
        uint64_t hi = d.nk, lo = 0;
        if (d.vis == ATTN_VIS_CAUSAL) {
            const uint64_t last = std::min<uint64_t>((uint64_t)g * 128u + 127u, d.nq - 1u) + d.causal_off;
            hi = std::min<uint64_t>(hi, last + 1u);
            if (d.window > 0) {
                const uint64_t first = (uint64_t)g * 128u + d.causal_off;
                lo = first + 1u > d.window ? first + 1u - d.window : 0u;
            }
        }
        return hi > lo ? (uint32_t)((hi - lo + 31u) / 32u) : 0u;
    };
    std::vector<Item> items;
    for (uint32_t n = 0; n < count; n++) {
        const AttnProb &d = host[base + n];
        const uint32_t G = attn_wide_groups(d);
        const bool pairs = attn_wide_pairs(d);
        const uint32_t n_items = attn_wide_items(d);
        for (uint32_t t = 0; t < n_items; t++) {
            const uint32_t ga = pairs ? G - 1u - t : t;
            const uint32_t gb = pairs && t < ga ? t : 0xFFFFu;
            Item it;
            it.t.prob = base + n;
            it.t.qtile = ga | (gb << 16);
            it.work = key_tiles(d, ga) + (gb != 0xFFFFu ? key_tiles(d, gb) : 0u);
            items.push_back(it);
        }
    }
    std::stable_sort(items.begin(), items.end(), [](const Item &a, const Item &b) { return a.work > b.work; });
    for (const Item &it : items) tiles.push_back(it.t);
}

void attn_wide_launch(const AttnProb *dprobs, const AttnTile *dtiles, uint32_t ntiles, uint32_t hd, bool dense,
                      hipStream_t s) {
    if (ntiles == 0) return;
    AttnAffine none;
    __builtin_memset(&none, 0, sizeof(none));
    launch_wide<SRC_TILES>(dprobs, dtiles, ntiles, none, hd, dense, s);
}

void attn_wide_launch_single(const AttnProb &single, hipStream_t s) {
    AttnAffine a;
    __builtin_memset(&a, 0, sizeof(a));
    a.first = single;
    a.nqt = attn_wide_groups(single);
    a.reserved = attn_wide_pairs(single) ? 1u : 0u;
    launch_wide<SRC_SINGLE>(nullptr, nullptr, attn_wide_items(single), a, single.hd, single.vis == ATTN_VIS_DENSE, s);
}

/* The batch descriptor of the mfma family, re-read for this kernel: `nqt`
 * counts 128-row groups and `reserved` says whether groups run in pairs. */
void attn_wide_launch_affine(const AttnAffine &aff_in, hipStream_t s) {
    AttnAffine aff = aff_in;
    aff.nqt = attn_wide_groups(aff.first);
    aff.reserved = attn_wide_pairs(aff.first) ? 1u : 0u;
    const uint32_t blocks = aff.count * attn_wide_items(aff.first);
    if (blocks == 0) return;
    launch_wide<SRC_AFFINE>(nullptr, nullptr, blocks, aff, aff.first.hd, aff.first.vis == ATTN_VIS_DENSE, s);
}
