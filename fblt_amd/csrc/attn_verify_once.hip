/*
 * Block step of the KV cache for blocks of at most 16 rows over a prefix short
 * enough to be in flight all at once (BLT-D/DV draft and verify blocks of 4 ...
 * 16 rows over a few hundred cached keys, csrc/infer/block_generation.c:156-266;
 * chunks of a prompt, csrc/infer/kv_cache.c:229-236).  The attention statements
 * of csrc/infer/kv_cache.c:343-390 as in the other block kernels -- new K (rotated)
 * and V rows written through first, then every new row attends the cached rows
 * and the new ones -- in the frame of the once kernel of the prefill path
 * (attn_once.hip):
 *
 *   - one workgroup per (sequence, head), W = 4, 8, 12 or 16 waves (the launch's
 *     choice: as few as give the longest sequence's tiles a slot); the sequence
 *     is walked as ceil(len / 16) tiles of cached rows followed by ONE tile that
 *     holds the step's new rows, wave w owning tiles w, w + W, ... (T at most).
 *     Which of the two a tile is, is uniform over the wave: base pointer, pitch
 *     and row limit are scalar selects;
 *   - every row the wave will need is requested at entry, Q, K and V rows alike
 *     with consecutive lanes on consecutive 16-byte pieces of a row (they become
 *     matrix fragments through the wave's own LDS tile): one trip to memory for
 *     the whole step, and the fewest vector memory instructions that move the
 *     bytes -- a (sequence, head) pair has ONE compute unit's vector memory path
 *     (64 bytes a cycle) for all its K and V rows, and that path is what the
 *     longest pair of a launch waits for;
 *   - a wave is on its own until its share is parked: the scores of all its
 *     tiles (v_mfma_f32_16x16x4_f32, chains interleaved), weights against its
 *     own maximum per row, O^T += V^T P^T, then [maximum, sum, partial rows]
 *     into LDS.  One barrier; the merge scales the W partials to the common
 *     maximum.  The waves' rows come through the compute unit's vector memory
 *     path one after the other, so the early waves' arithmetic hides under the
 *     late waves' requests; a barrier between scores and weights (one maximum
 *     for all waves, plain sums in the merge) would put every wave's second
 *     contraction behind the last wave's first;
 *
 * Lengths from device memory (commit through the sequence's ticket, capacity
 * guard) or from the kernel arguments, as in the other step kernels (kv_step.h).
 */
#include "blt_hip.h"
#include "blt_fatal.h"
#include "hip_check.h"
#include "attn_device.h"
#include "attn_tile.h"
#include "kv_step.h"
#include "launch.h"
#include "lane_ops.h"

#include <algorithm>

namespace {

typedef float floatx4 __attribute__((ext_vector_type(4)));

template <int HD>
struct BlockOnceShape {
    static constexpr int ROW = HD + 4;  /* floats of a parked row */
    static constexpr int WMAX = 16;     /* waves of a workgroup at most; pitch of the statistics rows */
    static constexpr int STATS = 2 * 16 * WMAX; /* [16][WMAX] maxima, [16][WMAX] sums */
    static constexpr size_t bytes(uint32_t waves) { return (size_t)(STATS + waves * 16 * ROW) * sizeof(float); }
};

template <int HD, int T, bool KARG>
__global__ __launch_bounds__(1024) void kv_block_once_kernel(StepArgs a, LensArg<KARG> lens) {
    kv_fetch_arguments(a);
    using Shape = BlockOnceShape<HD>;
    constexpr int WP = Shape::WMAX;
    const uint32_t W = blockDim.x >> 6; /* a multiple of four */
    constexpr int HALF = HD / 2;
    constexpr int QD = HD / 4;  /* floats of a row one lane group contracts */
    constexpr int NV = QD / 4;  /* 16-byte loads per lane and 16-row tile   */
    constexpr int DT = HD / 16; /* 16-row tiles of O^T                      */
    constexpr int ROW = Shape::ROW;
    constexpr int LPR = HD / 4;   /* lanes per row when the wave moves a tile */
    constexpr int RPI = 64 / LPR; /* rows one load instruction covers         */

    extern __shared__ __attribute__((aligned(16))) float sm[];
    float *const sm_max = sm;          /* [query c][wave] */
    float *const sm_sum = sm + 16 * WP; /* [query c][wave] */
    float *const sm_o = sm + Shape::STATS;
    __shared__ uint32_t sm_ticket;

    const uint32_t b = blockIdx.y;
    const uint32_t head = blockIdx.z;
    const uint32_t tid = threadIdx.x;
    const uint32_t lane = tid & 63u;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const uint32_t g = lane >> 4;
    const uint32_t c = lane & 15u;
    const uint32_t prow = lane / LPR, pf = lane % LPR;

    const uint32_t len = kv_len_of(a, lens, b) + a.len_bias;
    const uint32_t nk = len + a.n;
    if (!KARG && kv_over_capacity(a, nk)) return; /* uniform over the sequence's workgroups */
    const size_t slab = (size_t)b * a.max_seq_len;
    const size_t newrow0 = (size_t)b * a.n_seq;
    const uint32_t cached_tiles = (len + 15u) / 16u; /* then the tile with the new rows */

    const float *const cache_k = a.cache_k + slab * a.embed_dim + head * HD;
    const float *const cache_v = a.cache_v + slab * a.embed_dim + head * HD;
    const float *const new_k = a.k_rows + newrow0 * a.k_stride + head * HD;
    const float *const new_v = a.v_rows + newrow0 * a.v_stride + head * HD;
    const uint32_t cache_pitch = a.embed_dim * 4u, newk_pitch = a.k_stride * 4u, newv_pitch = a.v_stride * 4u;
    const uint32_t last_cached = len > 0u ? len - 1u : 0u, last_new = a.n - 1u;

    /* ---- every request of the wave, before anything waits ---- */
    floatx4 qg[NV], kg[T][NV];
    {
        const char *qb = reinterpret_cast<const char *>(a.q_rows + newrow0 * a.q_stride + head * HD);
#pragma unroll
        for (int v = 0; v < NV; v++)
            qg[v] = *reinterpret_cast<const floatx4 *>(qb + min(prow + (uint32_t)(RPI * v), last_new) * (a.q_stride * 4u) + 16u * pf);
    }
    floatx4 vg[T][NV];
#pragma unroll
    for (int u = 0; u < T; u++) {
        /* a tile past the sequence's last repeats it: the loads hit the cache, nothing is computed */
        const uint32_t ti = min(wave + W * u, cached_tiles);
        const bool fresh = ti == cached_tiles; /* wave-uniform: scalar selects */
        const char *kb = reinterpret_cast<const char *>(fresh ? new_k : cache_k);
        const uint32_t kp = fresh ? newk_pitch : cache_pitch;
        const uint32_t row0 = fresh ? 0u : ti * 16u, limit = fresh ? last_new : last_cached;
#pragma unroll
        for (int v = 0; v < NV; v++)
            kg[u][v] = *reinterpret_cast<const floatx4 *>(kb + min(row0 + prow + (uint32_t)(RPI * v), limit) * kp + 16u * pf);
    }
#pragma unroll
    for (int u = 0; u < T; u++) {
        const uint32_t ti = min(wave + W * u, cached_tiles);
        const bool fresh = ti == cached_tiles;
        const char *vb = reinterpret_cast<const char *>(fresh ? new_v : cache_v);
        const uint32_t vp = fresh ? newv_pitch : cache_pitch;
        const uint32_t row0 = fresh ? 0u : ti * 16u, limit = fresh ? last_new : last_cached;
#pragma unroll
        for (int v = 0; v < NV; v++)
            vg[u][v] = *reinterpret_cast<const floatx4 *>(vb + min(row0 + prow + (uint32_t)(RPI * v), limit) * vp + 16u * pf);
    }

    /* ---- the new rows: rotate queries and keys at their own positions, write keys and values
     * through (kv_cache.c:343-366); then rows -> fragments through the wave's own LDS tile (LDS
     * serves a wave's requests in order: tile after tile goes through it without a barrier) ---- */
    float *const tile = sm_o + wave * (16 * ROW); /* becomes the wave's partial output later */
    float qf[QD], kf[T][QD];
    if (a.rope_cos) {
#pragma unroll
        for (int v = 0; v < NV; v++) {
            const size_t at = (size_t)(len + min(prow + (uint32_t)(RPI * v), last_new)) * HALF + 2u * pf;
            const float4 t = rope_rotate4(make_float4(qg[v][0], qg[v][1], qg[v][2], qg[v][3]), a.rope_cos + at, a.rope_sin + at);
            qg[v][0] = t.x, qg[v][1] = t.y, qg[v][2] = t.z, qg[v][3] = t.w;
        }
    }
#pragma unroll
    for (int v = 0; v < NV; v++) *reinterpret_cast<floatx4 *>(tile + (prow + (uint32_t)(RPI * v)) * ROW + 4u * pf) = qg[v];
#pragma unroll
    for (int s = 0; s < QD; s += 4) {
        const float4 t = *reinterpret_cast<const float4 *>(tile + c * ROW + g * QD + s);
        qf[s + 0] = t.x, qf[s + 1] = t.y, qf[s + 2] = t.z, qf[s + 3] = t.w;
    }
#pragma unroll
    for (int u = 0; u < T; u++) {
        const uint32_t ti = wave + W * u;
        if (ti == cached_tiles) { /* this wave holds the new rows */
#pragma unroll
            for (int v = 0; v < NV; v++) {
                const uint32_t r = prow + (uint32_t)(RPI * v);
                const bool real = r < a.n;
                if (a.rope_cos && real) {
                    const size_t at = (size_t)(len + r) * HALF + 2u * pf;
                    const float4 t = rope_rotate4(make_float4(kg[u][v][0], kg[u][v][1], kg[u][v][2], kg[u][v][3]),
                                                  a.rope_cos + at, a.rope_sin + at);
                    kg[u][v][0] = t.x, kg[u][v][1] = t.y, kg[u][v][2] = t.z, kg[u][v][3] = t.w;
                }
                if (a.write_through && real) {
                    const size_t at = (slab + len + r) * a.embed_dim + head * HD + 4u * pf;
                    *reinterpret_cast<floatx4 *>(a.cache_k + at) = kg[u][v];
                    *reinterpret_cast<floatx4 *>(a.cache_v + at) = vg[u][v];
                }
            }
        }
#pragma unroll
        for (int v = 0; v < NV; v++)
            *reinterpret_cast<floatx4 *>(tile + (prow + (uint32_t)(RPI * v)) * ROW + 4u * pf) = kg[u][v];
#pragma unroll
        for (int s = 0; s < QD; s += 4) {
            const float4 t = *reinterpret_cast<const float4 *>(tile + c * ROW + g * QD + s);
            kf[u][s + 0] = t.x, kf[u][s + 1] = t.y, kf[u][s + 2] = t.z, kf[u][s + 3] = t.w;
        }
    }

    /* the keys this lane's query row (row c of the block) sees, as absolute positions [vis_lo, vis_hi):
     * block rows see everything, causal rows up to their own position inside the window
     * (kv_cache.c:229-236), padding rows nothing */
    uint32_t vis_lo = 0, vis_hi = nk;
    if (!a.block_kind) {
        const uint32_t qpos = len + c;
        vis_hi = min(vis_hi, qpos + 1u);
        if (a.window > 0u && qpos + 1u > a.window) vis_lo = qpos + 1u - a.window;
    }
    if (c >= a.n) vis_hi = 0;
    const float scale2 = a.scale * LOG2E; /* log2 units: weights are 2^(x - max) */

    /* ---- phase 1: scores of the wave's tiles, the wave's maximum per query ---- */
    constexpr int NA = T <= 2 ? 2 : 1; /* accumulators per tile: with three tiles and more their chains interleave */
    floatx4 sa[T][NA];
    bool on[T], all_on = true;
#pragma unroll
    for (int u = 0; u < T; u++) {
        on[u] = wave + W * u <= cached_tiles;
        all_on = all_on & on[u];
#pragma unroll
        for (int k = 0; k < NA; k++) sa[u][k] = floatx4{0.f, 0.f, 0.f, 0.f};
    }
    if (all_on) {
#pragma unroll
        for (int s = 0; s < QD; s += NA)
#pragma unroll
            for (int u = 0; u < T; u++)
#pragma unroll
                for (int k = 0; k < NA; k++)
                    sa[u][k] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u][s + k], qf[s + k], sa[u][k], 0, 0, 0);
    } else {
#pragma unroll
        for (int u = 0; u < T; u++) {
            if (on[u]) {
#pragma unroll
                for (int s = 0; s < QD; s += NA)
#pragma unroll
                    for (int k = 0; k < NA; k++)
                        sa[u][k] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[u][s + k], qf[s + k], sa[u][k], 0, 0, 0);
            }
        }
    }
    /* while the matrix cores work on the scores: the V rows -> fragments, through the same tile: element (d, r) of tile u is column DT c + d of row
     * 4 g + r -- the key whose weight register r of the scores holds, so P^T needs no exchange */
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

    float x[T][4];
    float mt = neg_inf();
#pragma unroll
    for (int u = 0; u < T; u++) {
        const uint32_t ti = wave + W * u;
        const bool fresh = ti == cached_tiles;
        const uint32_t j0 = fresh ? len : ti * 16u; /* absolute position of the tile's first key */
        const uint32_t j_end = fresh ? nk : len;    /* rows past it are clamped repeats */
        const uint32_t hi = min(vis_hi, j_end);
        const uint32_t span = on[u] && hi > vis_lo ? hi - vis_lo : 0u;
        const uint32_t rel = j0 + 4u * g - vis_lo;
#pragma unroll
        for (int r = 0; r < 4; r++) {
            const float t = (NA == 2 ? sa[u][0][r] + sa[u][NA - 1][r] : sa[u][0][r]) * scale2;
            const bool vis = ((rel + r) < span) & isfinite(t);
            x[u][r] = vis ? t : neg_inf();
            mt = fmaxf(mt, x[u][r]);
        }
    }
    mt = swap32(swap16(mt, OpMax()), OpMax());

    /* ---- phase 2: weights against the wave's own maximum, the wave's share of O^T.  Nothing waits for
     * another wave here: the waves' rows arrive one after the other through the compute unit's one
     * vector memory path, and the early ones are done before the late ones have their keys ---- */
    const float ms = mt == neg_inf() ? 0.f : mt;
    float ps = 0.f;
#pragma unroll
    for (int u = 0; u < T; u++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
            x[u][r] = fast_exp2(x[u][r] - ms); /* 2^(-inf) = 0 */
            ps += x[u][r];
        }
    ps = swap32(swap16(ps, OpSum()), OpSum());
    if (g == 0) sm_max[c * WP + wave] = mt, sm_sum[c * WP + wave] = ps;

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
    /* every wave of the workgroup has read the old length: draw the sequence's ticket now, look at it last */
    const uint32_t early_ticket = kv_draw_early_ticket(a, b);

    /* ---- phase 3: four threads per (row, 16-byte piece of the row), each folds every fourth wave's
     * partial, scaled to the row's maximum over all waves; the four meet inside their quad of lanes ---- */
    const uint32_t part = tid & 3u;
    for (uint32_t cell = tid >> 2; cell < 16u * LPR; cell += blockDim.x >> 2) { /* uniform over a quad */
        const uint32_t mr = cell / LPR, mf = cell % LPR;
        float M = neg_inf();
        for (uint32_t w4 = 0; w4 < W; w4 += 4u) {
            const float4 t = *reinterpret_cast<const float4 *>(sm_max + mr * WP + w4);
            M = fmaxf(fmaxf(M, fmaxf(t.x, t.y)), fmaxf(t.z, t.w));
        }
        const float Ms = M == neg_inf() ? 0.f : M;
        float L = 0.f;
        float4 o = make_float4(0.f, 0.f, 0.f, 0.f);
        for (uint32_t w = part; w < W; w += 4u) {
            const float4 t = *reinterpret_cast<const float4 *>(sm_o + w * (16 * ROW) + mr * ROW + 4u * mf);
            const float f = fast_exp2(sm_max[mr * WP + w] - Ms); /* a wave without a visible key: 2^(-inf) = 0 */
            L += sm_sum[mr * WP + w] * f;
            o.x += t.x * f, o.y += t.y * f, o.z += t.z * f, o.w += t.w * f;
        }
        L = key_sum<4>(L), o.x = key_sum<4>(o.x), o.y = key_sum<4>(o.y), o.z = key_sum<4>(o.z), o.w = key_sum<4>(o.w);
        if (part == 0u && mr < a.n) {
            const float inv = L > 0.f ? 1.0f / L : 0.f;
            *reinterpret_cast<float4 *>(a.combined + (newrow0 + mr) * a.out_stride + head * HD + 4u * mf) =
                make_float4(o.x * inv, o.y * inv, o.z * inv, o.w * inv);
        }
    }
    kv_finish_sequence<HD>(a, 16u, b, nk, &sm_ticket, early_ticket);
}

template <int HD, int T>
void block_once_launch_as(const StepArgs &a, uint32_t batch, uint32_t waves, const uint32_t *host_lens, hipStream_t s) {
    using Shape = BlockOnceShape<HD>;
    const dim3 grid(1, batch, a.num_heads), block(64 * waves);
    const size_t lds = Shape::bytes(waves);
    if (host_lens) {
        static const bool raised = [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&kv_block_once_kernel<HD, T, true>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)Shape::bytes(Shape::WMAX)));
            return true;
        }();
        (void)raised;
        KargLens lens;
        for (uint32_t b = 0; b < batch; b++) lens.v[b] = host_lens[b];
        blt_launch("kv_block_once", kv_block_once_kernel<HD, T, true>, grid, block, lds, s, a, lens);
    } else {
        static const bool raised = [] {
            HIP_CHECK(hipFuncSetAttribute(reinterpret_cast<const void *>(&kv_block_once_kernel<HD, T, false>),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)Shape::bytes(Shape::WMAX)));
            return true;
        }();
        (void)raised;
        blt_launch("kv_block_once", kv_block_once_kernel<HD, T, false>, grid, block, lds, s, a, DeviceLens{0u});
    }
}

} // namespace

/* Launch of the once block kernel: at most 16 rows per sequence from row 0 on, one split, and a prefix
 * whose 16-key tiles (plus the one with the new rows) fit the waves' registers; false when it does
 * not take the shape.  host_lens: NULL (device lengths) or `batch` <= KARG_SEQS lengths. */
bool kv_block_once_launch(const StepArgs &a_in, uint32_t batch, uint32_t head_dim, const uint32_t *host_lens,
                          hipStream_t s) {
    if (a_in.q0 != 0u || a_in.n > 16u || a_in.n == 0u || a_in.splits != 1u) return false;
    const uint32_t tiles = (a_in.span + 15u) / 16u + 1u; /* what the longest sequence of the launch may need */
    const uint32_t per_wave = (tiles + 15u) / 16u;       /* tiles a wave holds at once */
    /* as few waves as give every tile a slot, in fours: a slot without a tile still costs its requests */
    const uint32_t waves = std::min(16u, ((tiles + per_wave - 1u) / per_wave + 3u) / 4u * 4u);
    StepArgs a = a_in;
    a.hpb = 1, a.slices = 1, a.by_length = 0;
    if (head_dim == 32u) {
        switch (per_wave) {
        case 1: block_once_launch_as<32, 1>(a, batch, waves, host_lens, s); break;
        case 2: block_once_launch_as<32, 2>(a, batch, waves, host_lens, s); break;
        case 3: block_once_launch_as<32, 3>(a, batch, waves, host_lens, s); break;
        case 4: block_once_launch_as<32, 4>(a, batch, waves, host_lens, s); break;
        default: return false;
        }
    } else if (head_dim == 64u) {
        switch (per_wave) {
        case 1: block_once_launch_as<64, 1>(a, batch, waves, host_lens, s); break;
        case 2: block_once_launch_as<64, 2>(a, batch, waves, host_lens, s); break;
        default: return false;
        }
    } else {
        return false;
    }
    return true;
}
